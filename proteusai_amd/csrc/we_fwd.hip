// Isotropic Wavefunction Embedding forward for gfx950 (MI355X).
//
// What it computes (reference semantics, magnitude 1/|r|, no dropout):
//   utils/model_utils/wf_embedding/isotropic/cuda/wf_embedding_kernel.cu:181-250
//   tests/wf_embed/wf_embed.py:91-129 (dense PyTorch statement)
//
// Mapping to the machine.  The reference gives one 64-thread block to one
// observer, puts one source per thread and reduces every (source-block, k)
// product across the warp with shuffles and shared-memory atomics.  Here the
// roles are turned round so that no cross-lane traffic exists at all:
//   - a LANE owns one observer i; a WAVE owns 64 observers and a tile of KT
//     wavenumbers, whose 4*KT running sums live in VGPRs for the whole kernel;
//   - the wavenumbers of the tile are wave-uniform and sit in SGPRs;
//   - sources are streamed: the workgroup (4 waves = the same 64 observers,
//     4 wavenumber tiles) stages blocks of source coordinates in LDS, already
//     compacted to the unpadded ones, and every lane reads the same source with
//     one broadcast ds_read_b128;
//   - per (pair, k) the wave issues: v_mul (phase, in revolutions), v_sin, v_cos,
//     2 x v_fmac (embedding), 2 x v_add (cos/sin sums); v_sin/v_cos take
//     revolutions and are exact-period for |phase| <= 256, so the explicit range
//     reduction (v_fract) is issued only for a source whose phase can exceed
//     that for some lane of the wave (a wave-uniform branch per source).
// Padded sources never reach the inner loop (compaction), padded observers are
// computed as ordinary lanes and written as zeros, and the self/coincident pair
// (r^2 == 0) runs through the loop with r = 0 and 1/r = 0: it adds exactly
// cos(0) = 1 to each cos sum and nothing else, and the count of such pairs is
// subtracted once at the end.  No branch in the inner loop depends on a lane.

#include <hip/hip_runtime.h>
#include <stdint.h>
#include "proteus_hip.h"
#include "we_ranked.h"

namespace {

constexpr int WE_WAVES   = 4;
constexpr int WE_THREADS = WE_WAVES * 64;
constexpr int WE_JB      = 256;   // sources staged per LDS block (one per thread)
constexpr float WE_MAX_REV = 250.0f;

// Value of the MAG template parameter for "weight 1/r, no cos/sin sums" (the caller passed no buffers for them:
// inference, where nothing is kept for the backward; two of the four accumulations per unit fall away).
constexpr int WE_MAG_NO_SUMS = -1;

// Wavenumbers per phase batch of the inner loop (0: leave the order to the compiler).  On gfx950 a
// vector instruction whose operands are all vector registers issues in about 2.4 clocks per wave once a
// SIMD holds three or more waves, one with a scalar-register operand in 4, a transcendental in 8; an
// ordinary instruction placed between two transcendentals of the same wave costs 4 whatever its operands
// (measured with proteus_probe_valu_rate).  So the loop does the scalar-operand phase products of a batch
// first, then its sines and cosines, then its accumulations, which then run at the fast rate.
#ifndef WE_BATCH
#define WE_BATCH 16
#endif   // v_sin_f32 / v_cos_f32 accept |x| <= 256 revolutions; keep a margin

__device__ __forceinline__ float sgpr(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, v)));
}

// Inner loop: every lane (observer) against the nk staged sources, KT wavenumbers each.
// FRACT: reduce the phase to [0,1) revolutions before v_sin/v_cos (needed only when it can exceed
// the +-256 revolutions those instructions accept).
// MAG: the weight m(r) of a source (isotropic/cuda/wf_embedding_kernel.cu:192-206): 0: 1, 1: 1/r,
// 2: 1/log2(r), 3: 1/sqrt(r).  The embedding sums m cos, m sin and the saved sums m r cos, m r sin
// (kernel.cu:224-238); for MAG 1 the latter weight is 1 and the accumulation a plain add.
template <int KT, bool FRACT, int MAG>
__device__ __forceinline__ void stream_sources(const float4* s_keys, const int first, const int step, const int nk,
                                               const float xi, const float yi, const float zi,
                                               const float (&kr)[KT],
                                               float (&acc_oc)[KT], float (&acc_os)[KT],
                                               float (&acc_c)[KT], float (&acc_s)[KT], float& nzero)
{
    float4 knext = s_keys[first];                 // (reads at most WE_WAVES entries past nk: the array is padded)
#pragma unroll 1
    for (int jj = first; jj < nk; jj += step) {
        const float4 kj = knext;
        knext = s_keys[jj + step];
        const float dx = xi - kj.x, dy = yi - kj.y, dz = zi - kj.z;
        const float r2 = dx * dx + dy * dy + dz * dz;
        const bool  ok = r2 != 0.0f;
        const float inv = ok ? __builtin_amdgcn_rsqf(r2) : 0.0f;
        // one Newton step on r = r2 * rsq(r2): r is then within 1 ulp of sqrt(r2)
        const float r0 = r2 * inv;
        const float e  = __builtin_fmaf(-r0, r0, r2);
        const float r  = __builtin_fmaf(e, 0.5f * inv, r0);
        float m = inv, mr = 1.0f;
        if (MAG == WE_MAG_NO_SUMS) {
            // weight 1/r, nothing kept for the backward
        } else if (MAG == 1) {
            nzero += ok ? 0.0f : 1.0f;       // the r = 0 pair adds cos(0) = 1 to the cos sums: counted, removed at the end
        } else {
            // the r = 0 pair gets weight 0 in both sums
            if (MAG == 0) m = ok ? 1.0f : 0.0f;
            if (MAG == 2) m = ok ? __builtin_amdgcn_rcpf(__builtin_amdgcn_logf(r)) : 0.0f;   // v_log_f32 is log2
            if (MAG == 3) m = ok ? __builtin_amdgcn_rsqf(r) : 0.0f;
            mr = m * r;
        }
        // The wavenumbers are taken in batches and each batch in three phases (phases, then sines and
        // cosines, then the accumulations), kept apart by scheduling barriers: see WE_BATCH.
        constexpr int B = (WE_BATCH > 0 && WE_BATCH < KT) ? WE_BATCH : KT;
#pragma unroll
        for (int t0 = 0; t0 < KT; t0 += B) {
            float sn[B], cs[B];
#pragma unroll
            for (int u = 0; u < B; ++u) {
                float ph = r * kr[t0 + u];
                if (FRACT) ph = __builtin_amdgcn_fractf(ph);
                sn[u] = ph;
            }
            if (WE_BATCH > 0) __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int u = 0; u < B; ++u) {
                cs[u] = __builtin_amdgcn_cosf(sn[u]);
                sn[u] = __builtin_amdgcn_sinf(sn[u]);
            }
            if (WE_BATCH > 0) __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int u = 0; u < B; ++u) {
                const int t = t0 + u;
                acc_oc[t] = __builtin_fmaf(cs[u], m, acc_oc[t]);
                acc_os[t] = __builtin_fmaf(sn[u], m, acc_os[t]);
                if (MAG == WE_MAG_NO_SUMS) continue;
                if (MAG == 1) { acc_c[t] += cs[u]; acc_s[t] += sn[u]; }
                else          { acc_c[t] = __builtin_fmaf(cs[u], mr, acc_c[t]); acc_s[t] = __builtin_fmaf(sn[u], mr, acc_s[t]); }
            }
            if (WE_BATCH > 0) __builtin_amdgcn_sched_barrier(0);
        }
    }
}

// Everything after the prologue, for one choice of FRACT: the running sums live only inside this
// function, so the two instantiations a kernel holds never have their accumulators alive together.
template <int KT, bool SPLIT, bool FRACT, int MAG>
__device__ __forceinline__ void we_body(float4* s_keys, int* s_wcount, float* s_red,
                                        const float* __restrict__ cz, const uint8_t* __restrict__ mz, const int layout,
                                        float* __restrict__ out, float* __restrict__ cos_sums, float* __restrict__ sin_sums,
                                        const int N, const int j_end, const int K, const size_t zN,
                                        const int tid, const int lane, const int wave,
                                        const int i, const bool i_in, const bool i_valid,
                                        const float xi, const float yi, const float zi,
                                        const int k0, const bool wave_active, const float (&kr)[KT])
{
    float acc_oc[KT], acc_os[KT], acc_c[KT], acc_s[KT];
#pragma unroll
    for (int t = 0; t < KT; ++t) { acc_oc[t] = 0.f; acc_os[t] = 0.f; acc_c[t] = 0.f; acc_s[t] = 0.f; }
    float nzero = 0.f;

    {
        for (int jb = 0; jb < j_end; jb += WE_JB) {
            // -- stage one block of sources, keeping only the unpadded ones --
            const int  j    = jb + tid;
            const bool j_in = j < j_end;
            const int  jc   = j_in ? j : N - 1;
            float xj, yj, zj;
            if (layout == PROTEUS_COORDS_SOA) { xj = cz[jc]; yj = cz[(size_t)N + jc]; zj = cz[2 * (size_t)N + jc]; }
            else                              { xj = cz[3 * (size_t)jc]; yj = cz[3 * (size_t)jc + 1]; zj = cz[3 * (size_t)jc + 2]; }
            const bool j_valid = j_in && !(mz && mz[jc]);

            const uint64_t bal   = __builtin_amdgcn_ballot_w64(j_valid);
            const int      below = __builtin_popcountll(bal & ((1ull << lane) - 1ull));
            __syncthreads();                       // previous block fully consumed
            if (lane == 0) s_wcount[wave] = __builtin_popcountll(bal);
            __syncthreads();
            int base = 0, nk = 0;
#pragma unroll
            for (int w = 0; w < WE_WAVES; ++w) { const int c = s_wcount[w]; base += (w < wave) ? c : 0; nk += c; }
            if (j_valid) s_keys[base + below] = make_float4(xj, yj, zj, 0.f);
            __syncthreads();
            nk = __builtin_amdgcn_readfirstlane(nk);

            if (!wave_active) continue;

            // -- stream the staged sources --
            if (SPLIT) stream_sources<KT, FRACT, MAG>(s_keys, wave, WE_WAVES, nk, xi, yi, zi, kr, acc_oc, acc_os, acc_c, acc_s, nzero);
            else       stream_sources<KT, FRACT, MAG>(s_keys, 0, 1, nk, xi, yi, zi, kr, acc_oc, acc_os, acc_c, acc_s, nzero);
        }
    }

    if (SPLIT) {
        // ---- the four waves' partial sums meet in LDS, one wave at a time; wave 0 writes the rows ----
        float* q = s_red + lane;
#pragma unroll 1
        for (int w = 1; w < WE_WAVES; ++w) {
            __syncthreads();
            if (wave == w) {
#pragma unroll
                for (int t = 0; t < KT; ++t) {
                    q[(4 * t + 0) * 64] = acc_oc[t]; q[(4 * t + 1) * 64] = acc_os[t];
                    q[(4 * t + 2) * 64] = acc_c[t];  q[(4 * t + 3) * 64] = acc_s[t];
                }
                q[4 * KT * 64] = nzero;
            }
            __syncthreads();
            if (wave == 0) {
#pragma unroll
                for (int t = 0; t < KT; ++t) {
                    acc_oc[t] += q[(4 * t + 0) * 64]; acc_os[t] += q[(4 * t + 1) * 64];
                    acc_c[t]  += q[(4 * t + 2) * 64]; acc_s[t]  += q[(4 * t + 3) * 64];
                }
                nzero += q[4 * KT * 64];
            }
        }
        if (wave > 0) return;
    }

    if (!wave_active || !i_in) return;

    // ---- epilogue: each lane writes its own rows ----
    const size_t row = zN + (size_t)i;
    float* o  = out      + row * (size_t)(2 * K) + 2 * (size_t)k0;

    // padded observer: exact zeros, whatever its lane accumulated (its coordinates may hold anything, NaN included,
    // so the sums are selected away, not multiplied by zero)
    auto kept = [&](const float v) { return i_valid ? v : 0.0f; };
    float* pc = nullptr;
    float* ps = nullptr;
    if (MAG != WE_MAG_NO_SUMS) { pc = cos_sums + row * (size_t)K + k0; ps = sin_sums + row * (size_t)K + k0; }
    if (k0 + KT <= K && (K & 1) == 0 && (KT & 3) == 0 && (K & 3) == 0) {
        // full tile, rows 16-byte aligned: vector stores
#pragma unroll
        for (int t = 0; t < KT; t += 2) {
            float4 v = make_float4(kept(acc_oc[t]), kept(acc_os[t]), kept(acc_oc[t + 1]), kept(acc_os[t + 1]));
            *reinterpret_cast<float4*>(o + 2 * t) = v;
        }
#pragma unroll
        for (int t = 0; t < KT; t += 4) {
            if (MAG == WE_MAG_NO_SUMS) break;
            float4 c = make_float4(kept(acc_c[t] - nzero), kept(acc_c[t + 1] - nzero),
                                   kept(acc_c[t + 2] - nzero), kept(acc_c[t + 3] - nzero));
            float4 s = make_float4(kept(acc_s[t]), kept(acc_s[t + 1]), kept(acc_s[t + 2]), kept(acc_s[t + 3]));
            *reinterpret_cast<float4*>(pc + t) = c;
            *reinterpret_cast<float4*>(ps + t) = s;
        }
    } else {
#pragma unroll
        for (int t = 0; t < KT; ++t) {
            if (k0 + t < K) {
                o[2 * t]     = kept(acc_oc[t]);
                o[2 * t + 1] = kept(acc_os[t]);
                if (MAG == WE_MAG_NO_SUMS) continue;
                pc[t] = kept(acc_c[t] - nzero);
                ps[t] = kept(acc_s[t]);
            }
        }
    }
}

// Rows of 64 observers that are all padded: zeros for the wavenumbers this wave (this workgroup, with SPLIT: its
// wave 0) is responsible for.
template <int KT, bool SPLIT, int MAG>
__device__ __forceinline__ void we_write_zero_rows(float* __restrict__ out, float* __restrict__ cos_sums, float* __restrict__ sin_sums,
                                                   const int K, const size_t zN, const int i, const bool i_in, const int wave, const int ytile)
{
    if (SPLIT && wave > 0) return;
    const int k0 = SPLIT ? ytile * KT : (ytile * WE_WAVES + wave) * KT;
    if (k0 >= K || !i_in) return;
    const size_t row = zN + (size_t)i;
    float* o = out + row * (size_t)(2 * K) + 2 * (size_t)k0;
    for (int t = 0; t < KT && k0 + t < K; ++t) {
        o[2 * t] = 0.0f; o[2 * t + 1] = 0.0f;
        if (MAG != WE_MAG_NO_SUMS) { cos_sums[row * (size_t)K + k0 + t] = 0.0f; sin_sums[row * (size_t)K + k0 + t] = 0.0f; }
    }
}

// KT     wavenumbers per wave (4*KT accumulators per lane)
// SPLIT  small problems: the four waves of a workgroup share ONE wavenumber tile and split the staged
//        sources between them (wave w takes sources w, w+4, ...); the partial sums meet in LDS at the
//        end.  Four times as many workgroups for the same KT, still no atomics, still deterministic.
// fract_mode  0: a workgroup reduces the phase explicitly (v_fract) only if some phase of its waves can
//        leave +-WE_MAX_REV revolutions; 1: always; -1: never (a measuring aid, valid only for bounded phases)
template <int KT, bool SPLIT, int MAG>
__global__ __launch_bounds__(WE_THREADS, (KT == 32 && SPLIT) ? 3 : 1)
void we_fwd_kernel(const float* __restrict__ coords, const int layout,
                   const float* __restrict__ wavenumbers,
                   const uint8_t* __restrict__ mask,
                   float* __restrict__ out, float* __restrict__ cos_sums, float* __restrict__ sin_sums,
                   const int N, const int K, const int fract_mode)
{
    __shared__ float4 s_keys[WE_JB + WE_WAVES];   // padding: the stream loop reads one step ahead
    __shared__ int    s_wcount[WE_WAVES];
    __shared__ float  s_box[WE_WAVES][6];
    __shared__ int    s_last[WE_WAVES];
    __shared__ float  s_red[SPLIT ? (4 * KT + 1) * 64 : 1];

    const int tid  = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    int z      = blockIdx.z;
    int ytile  = blockIdx.y;

    // Workgroup (x, y, z) takes observer block x + a z + 5 y (mod the number of blocks), a = 0.618 of that number made
    // odd: the same set of blocks per (y, z), in another order.  Workgroups that are resident together then belong to
    // different parts of their sequences, and in a batch of ragged lengths the blocks of padded observers (which
    // leave at once) are spread over the launch instead of coming in runs: 10-15 % off such batches, nothing
    // changes for full ones.
    const unsigned we_rot = ((unsigned)(0.6180339887f * (float)gridDim.x + 0.5f)) | 1u;
    // (32-bit safe: a <= 0.62 x 65536 blocks, z taken modulo the number of blocks first, y < 4096)
    int iblock = (int)((blockIdx.x + we_rot * (blockIdx.z % gridDim.x) + 5u * blockIdx.y) % gridDim.x);

    // A padded batch of a few items is handed out by the number of sources of its items instead (we_ranked.h)
    proteus_we::we_ranked_workgroup(mask, N, z, ytile, iblock);

    const size_t zN = (size_t)z * (size_t)N;
    const float* cz = coords + zN * 3;
    const uint8_t* mz = mask ? mask + zN : nullptr;

    // ---- this lane's observer ----
    const int  i      = iblock * 64 + lane;
    const bool i_in   = i < N;
    const int  ic     = i_in ? i : N - 1;
    float xi, yi, zi;
    if (layout == PROTEUS_COORDS_SOA) { xi = cz[ic]; yi = cz[(size_t)N + ic]; zi = cz[2 * (size_t)N + ic]; }
    else                              { xi = cz[3 * (size_t)ic]; yi = cz[3 * (size_t)ic + 1]; zi = cz[3 * (size_t)ic + 2]; }
    const bool i_valid = i_in && !(mz && mz[ic]);

    // Every wave of the workgroup sees the same 64 observers, so this exit is
    // uniform over the workgroup and happens before the first barrier.
    const bool any_valid = __builtin_amdgcn_ballot_w64(i_valid) != 0;
    if (!any_valid) {
        // 64 padded (or out-of-range) observers: zeros, and nothing else to do (in a batch of ragged lengths this is a
        // large share of the workgroups)
        we_write_zero_rows<KT, SPLIT, MAG>(out, cos_sums, sin_sums, K, zN, i, i_in, wave, ytile);
        return;
    }

    // ---- this wave's wavenumbers, converted to revolutions per angstrom ----
    const int  k0          = SPLIT ? ytile * KT : (ytile * WE_WAVES + wave) * KT;
    const bool wave_active = k0 < K;
    float kr[KT];
#pragma unroll
    for (int t = 0; t < KT; ++t) {
        const int k = k0 + t;
        const float w = (k < K) ? wavenumbers[k] : 0.0f;
        kr[t] = sgpr((float)((double)w * 0.15915494309189533577));
    }
    float kr_max = 0.f;
#pragma unroll
    for (int t = 0; t < KT; ++t) kr_max = fmaxf(kr_max, fabsf(kr[t]));

    // ---- can any phase of this wave leave the +-256 revolutions v_sin/v_cos accept? ----
    bool wg_safe = false;
    // Bounding box of the unpadded coordinates of the batch item (a few loads per thread, once), then the
    // distance from each observer to its farthest corner bounds every r_ij of the lane.  The same pass finds
    // where the unpadded sources end: the blocks of sources behind that are never staged.
    int j_end = 0;
    {
        float lo[3] = {3.0e38f, 3.0e38f, 3.0e38f}, hi[3] = {-3.0e38f, -3.0e38f, -3.0e38f};
        int last = 0;
        for (int j = tid; j < N; j += WE_THREADS) {
            if (mz && mz[j]) continue;
            last = j + 1;
            float p[3];
            if (layout == PROTEUS_COORDS_SOA) { p[0] = cz[j]; p[1] = cz[(size_t)N + j]; p[2] = cz[2 * (size_t)N + j]; }
            else                              { p[0] = cz[3 * (size_t)j]; p[1] = cz[3 * (size_t)j + 1]; p[2] = cz[3 * (size_t)j + 2]; }
#pragma unroll
            for (int c = 0; c < 3; ++c) { lo[c] = fminf(lo[c], p[c]); hi[c] = fmaxf(hi[c], p[c]); }
        }
#pragma unroll
        for (int c = 0; c < 3; ++c)
            for (int o = 32; o > 0; o >>= 1) { lo[c] = fminf(lo[c], __shfl_xor(lo[c], o)); hi[c] = fmaxf(hi[c], __shfl_xor(hi[c], o)); }
        for (int o = 32; o > 0; o >>= 1) last = max(last, __shfl_xor(last, o));
        if (lane == 0) {
#pragma unroll
            for (int c = 0; c < 3; ++c) { s_box[wave][c] = lo[c]; s_box[wave][3 + c] = hi[c]; }
            s_last[wave] = last;
        }
        __syncthreads();
        j_end = max(max(s_last[0], s_last[1]), max(s_last[2], s_last[3]));
#pragma unroll
        for (int c = 0; c < 3; ++c) {
            lo[c] = fminf(fminf(s_box[0][c], s_box[1][c]), fminf(s_box[2][c], s_box[3][c]));
            hi[c] = fmaxf(fmaxf(s_box[0][3 + c], s_box[1][3 + c]), fmaxf(s_box[2][3 + c], s_box[3][3 + c]));
        }
        const float fx = fmaxf(fabsf(xi - lo[0]), fabsf(xi - hi[0]));
        const float fy = fmaxf(fabsf(yi - lo[1]), fabsf(yi - hi[1]));
        const float fz = fmaxf(fabsf(zi - lo[2]), fabsf(zi - hi[2]));
        const float rfar = __builtin_sqrtf(fx * fx + fy * fy + fz * fz);
        // NaN-safe: anything that is not provably below the limit takes the reducing path
        // (a padded observer's lane, whose coordinates may hold anything, has no say)
        const bool wave_safe = __builtin_amdgcn_ballot_w64(i_valid && !(rfar * kr_max < WE_MAX_REV)) == 0;
        if (lane == 0) s_wcount[wave] = wave_safe ? 1 : 0;
        __syncthreads();
        wg_safe = (s_wcount[0] & s_wcount[1] & s_wcount[2] & s_wcount[3]) != 0;
    }
    const bool use_fract = fract_mode > 0 || (fract_mode == 0 && !wg_safe);
    if (use_fract)
        we_body<KT, SPLIT, true, MAG>(s_keys, s_wcount, s_red, cz, mz, layout, out, cos_sums, sin_sums, N, j_end, K, zN, tid, lane, wave,
                                 i, i_in, i_valid, xi, yi, zi, k0, wave_active, kr);
    else
        we_body<KT, SPLIT, false, MAG>(s_keys, s_wcount, s_red, cz, mz, layout, out, cos_sums, sin_sums, N, j_end, K, zN, tid, lane, wave,
                                  i, i_in, i_valid, xi, yi, zi, k0, wave_active, kr);
}


// fract: 0 = each workgroup picks, 1 = always reduce, -1 = never reduce (only valid when every phase
// is known to stay within +-256 revolutions; a measuring aid)
struct WeVariant { const char* name; int kt; bool split; int fract; };
// index 0 is "automatic"; the others force a tile
const WeVariant kVariants[] = {
    {"auto", 0, false, 0},
    {"kt32", 32, false, 0},
    {"kt16", 16, false, 0},
    {"kt8", 8, false, 0},
    {"kt16_split", 16, true, 0},
    {"kt8_split", 8, true, 0},
    {"kt32_split", 32, true, 0},
    {"kt32_fract", 32, false, 1},
    {"kt32_nofract_unchecked", 32, false, -1},
    {"kt4_split", 4, true, 0},
};
constexpr int kNumVariants = (int)(sizeof(kVariants) / sizeof(kVariants[0]));

template <int KT, bool SPLIT, int MAG = 1>
int launch(const float* coords, int layout, const float* wn, const uint8_t* mask,
           float* out, float* cs, float* ss, int Z, int N, int K, int fract, hipStream_t st)
{
    const int iblocks = (N + 63) / 64;
    const int ktiles  = SPLIT ? (K + KT - 1) / KT : (K + KT * WE_WAVES - 1) / (KT * WE_WAVES);
    dim3 grid(iblocks, ktiles, Z);
    hipLaunchKernelGGL((we_fwd_kernel<KT, SPLIT, MAG>), grid, dim3(WE_THREADS), 0, st,
                       coords, layout, wn, mask, out, cs, ss, N, K, fract);
    return (int)hipGetLastError();
}

}  // namespace

extern "C" int proteus_we_num_variants(void) { return kNumVariants; }

extern "C" const char* proteus_we_variant_name(int tuning) {
    return (tuning >= 0 && tuning < kNumVariants) ? kVariants[tuning].name : nullptr;
}

extern "C" int proteus_we_fwd_check(const float* coords, int coords_layout,
                                    const float* wavenumbers, const uint8_t* mask,
                                    const float* out, const float* cos_sums, const float* sin_sums,
                                    int Z, int N, int K, int tuning)
{
    (void)mask;
    if (!coords || !wavenumbers || !out) return PROTEUS_ERR_NULL_POINTER;
    if ((cos_sums == nullptr) != (sin_sums == nullptr)) return PROTEUS_ERR_NULL_POINTER;    // both or neither
    if (Z <= 0 || N <= 0 || K <= 0) return PROTEUS_ERR_BAD_SHAPE;
    if (N > PROTEUS_WE_MAX_N || K > PROTEUS_WE_MAX_K || Z > 65535) return PROTEUS_ERR_BAD_SHAPE;
    if (coords_layout != PROTEUS_COORDS_SOA && coords_layout != PROTEUS_COORDS_AOS) return PROTEUS_ERR_BAD_LAYOUT;
    if (tuning < 0 || tuning >= kNumVariants) return PROTEUS_ERR_BAD_TUNING;
    if (((uintptr_t)out & 15) || ((uintptr_t)cos_sums & 15) || ((uintptr_t)sin_sums & 15)) return PROTEUS_ERR_BAD_ALIGNMENT;
    return PROTEUS_OK;
}

extern "C" int proteus_we_fwd(const float* coords, int coords_layout,
                              const float* wavenumbers, const uint8_t* mask,
                              float* out, float* cos_sums, float* sin_sums,
                              int Z, int N, int K, int tuning, void* stream)
{
    const int rc = proteus_we_fwd_check(coords, coords_layout, wavenumbers, mask, out, cos_sums, sin_sums, Z, N, K, tuning);
    if (rc != PROTEUS_OK) return rc;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);

    int kt = kVariants[tuning].kt;
    bool split = kVariants[tuning].split;
    const int fract = kVariants[tuning].fract;
    const long iblocks = ((long)N + 63) / 64 * Z;
    if (tuning == 0) {
        // Pick the (wavenumber tile, source split) pair with the least estimated time.  Per source a wave
        // issues KT x (1 scalar-operand product, 2 transcendentals, 4 accumulations) + about 15 ordinary
        // instructions and a v_rsq; what an instruction costs depends on how many waves share the SIMD
        // (clocks per wave instruction, measured: vector-operand 5.8 / 2.9 / 2.5, scalar-operand
        // 4.8 / 4.15 / 4.0, transcendental 10.3 / 9.0 / 8.3 with 1 / 2 / 3+ waves).  `occ` is what the
        // kernel's registers allow.  Ties keep the earlier candidate.
        static const int cand_kt[7]    = {32, 32, 16, 16, 8, 8, 4};
        static const int cand_split[7] = {1, 0, 1, 0, 1, 0, 1};
        static const int cand_occ[7]   = {3, 2, 4, 4, 8, 8, 8};
        double best = 1e300;
        for (int c = 0; c < 7; ++c) {
            const int  ckt = cand_kt[c];
            const bool csp = cand_split[c] != 0;
            if (csp && N < 2 * WE_WAVES) continue;          // (fewer sources than a split could share out)
            const long ktiles = ((long)K + ckt - 1) / ckt;
            const long nwaves = csp ? iblocks * ktiles * WE_WAVES : iblocks * ((ktiles + WE_WAVES - 1) / WE_WAVES) * WE_WAVES;
            const double keys = csp ? (double)N / WE_WAVES : (double)N;
            const double q    = (double)nwaves / 1024.0;                 // waves per SIMD over the whole launch
            const int    w    = q > cand_occ[c] ? cand_occ[c] : (q <= 1.0 ? 1 : (int)(q + 0.999));
            const double cv = w <= 1 ? 5.8 : (w == 2 ? 2.9 : 2.5);
            const double cs = w <= 1 ? 4.8 : (w == 2 ? 4.15 : 4.0);
            const double ct = w <= 1 ? 10.3 : (w == 2 ? 9.0 : 8.3);
            const double per_wave = keys * (ckt * (cs + 2.0 * ct + 4.0 * cv) + 15.0 * cv + ct + 30.0);
            double est = (q > w ? q : (double)w) * per_wave;
            // A batch that comes with a padding mask is taken to be ragged.  While the widest tile gives at most 1024
            // workgroups (little more than one round of the chip), halving the tile makes twice as many workgroups of
            // half the length, which even out better than the wider tile saves: 8 x 1024 with lengths 128-1024 runs
            // 5-30 % faster (six draws of the lengths), the same batch without padding 2 % slower.
            if (mask && ckt == 32 && csp && nwaves <= 4096) est *= 1.10;
            if (est < best * 0.999) { best = est; kt = ckt; split = csp; }
        }
    }
#define WE_GO(KT_) (!cos_sums ? (split ? launch<KT_, true, WE_MAG_NO_SUMS>(coords, coords_layout, wavenumbers, mask, out, cos_sums, sin_sums, Z, N, K, fract, st) \
                                      : launch<KT_, false, WE_MAG_NO_SUMS>(coords, coords_layout, wavenumbers, mask, out, cos_sums, sin_sums, Z, N, K, fract, st)) \
                    : (split ? launch<KT_, true>(coords, coords_layout, wavenumbers, mask, out, cos_sums, sin_sums, Z, N, K, fract, st) \
                             : launch<KT_, false>(coords, coords_layout, wavenumbers, mask, out, cos_sums, sin_sums, Z, N, K, fract, st)))
    switch (kt) {
        case 32: return WE_GO(32);
        case 16: return WE_GO(16);
        case 4:  return WE_GO(4);
        default: return WE_GO(8);
    }
#undef WE_GO
}

namespace {
template <int MAG>
int launch_mag(bool split, const float* coords, int layout, const float* wn, const uint8_t* mask,
               float* out, float* cs, float* ss, int Z, int N, int K, hipStream_t st)
{
    return split ? launch<8, true, MAG>(coords, layout, wn, mask, out, cs, ss, Z, N, K, 0, st)
                 : launch<16, false, MAG>(coords, layout, wn, mask, out, cs, ss, Z, N, K, 0, st);
}
}  // namespace

extern "C" int proteus_we_legacy_fwd(const float* coords, int coords_layout,
                                     const float* wavenumbers, const uint8_t* mask,
                                     float* out, float* cos_sums, float* sin_sums,
                                     int Z, int N, int K, int magnitude_type, void* stream)
{
    if (magnitude_type < 0 || magnitude_type > 3) return PROTEUS_ERR_UNSUPPORTED;
    if (magnitude_type == 1)
        return proteus_we_fwd(coords, coords_layout, wavenumbers, mask, out, cos_sums, sin_sums, Z, N, K, 0, stream);
    if (!cos_sums || !sin_sums) return PROTEUS_ERR_NULL_POINTER;      // the variant without sums exists for 1/r only
    const int rc = proteus_we_fwd_check(coords, coords_layout, wavenumbers, mask, out, cos_sums, sin_sums, Z, N, K, 0);
    if (rc != PROTEUS_OK) return rc;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    // two tilings only for the rarely used weights: 16 wavenumbers per wave, or, while that leaves SIMDs
    // idle, 8 per workgroup with the sources split over its four waves
    const long iblocks = ((long)N + 63) / 64 * Z;
    const long nwaves  = iblocks * (((long)K + 63) / 64) * WE_WAVES;
    const bool split   = nwaves < 2048 && N >= 4 * 64;
    switch (magnitude_type) {
        case 0:  return launch_mag<0>(split, coords, coords_layout, wavenumbers, mask, out, cos_sums, sin_sums, Z, N, K, st);
        case 2:  return launch_mag<2>(split, coords, coords_layout, wavenumbers, mask, out, cos_sums, sin_sums, Z, N, K, st);
        default: return launch_mag<3>(split, coords, coords_layout, wavenumbers, mask, out, cos_sums, sin_sums, Z, N, K, st);
    }
}
