// Anisotropic (C-beta scaled, learnable wavenumber) Wavefunction Embedding forward for gfx950.
//
// What it computes (reference semantics):
//   utils/model_utils/wf_embedding/anisotropic/cb_scaling/learnable_wavenumbers/cuda/wf_embedding_kernel.cu:100-206
//   tests/wf_embed/wf_embed_aniso_learnCB_learnK.py:117-163 (dense PyTorch statement of `out`)
// For observer i, source j, wavenumber index k, with R = a_i - a_j, r = |R|, A = (b_j . R)/r:
//     phase = (r - cb_k A) k_k,   real = cos(phase)/r,   imag = sin(phase)/r
//     out [i,2k] = sum_j real                    out [i,2k+1] = sum_j imag
//     d_k [i,2k] = sum_j -imag (r - cb_k A)      d_k [i,2k+1] = sum_j  real (r - cb_k A)
//     d_cb[i,2k] = sum_j  imag k_k A             d_cb[i,2k+1] = sum_j -real k_k A
// over the pairs with both tokens unpadded and r != 0.
//
// The machine mapping is the isotropic kernel's: a lane owns an observer, a wave owns 64 observers and
// KT wavenumbers whose running sums stay in VGPRs, the workgroup stages compacted source blocks in LDS and
// every lane reads a source with broadcast ds_reads.  Six sums per wavenumber are kept, none of which
// depends on cb_k or k_k outside the phase, so the per-(pair,k) work is 2 phase ops, v_fract, v_sin, v_cos
// and 6 accumulations:
//     S1 = sum c/r   S2 = sum s/r   S3 = sum c   S4 = sum s   S5 = sum c A/r   S6 = sum s A/r
//     out = (S1, S2)   d_k = (-S4 + cb S6,  S3 - cb S5)   d_cb = (k S6, -k S5)
// The r == 0 pair runs through the loop with 1/r = 0, r = 0, A = 0: it adds cos(0) = 1 to S3 only, and the
// count of such pairs is subtracted at the end.

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>
#include "proteus_hip.h"
#include "we_ranked.h"

namespace {

constexpr int WA_WAVES   = 4;
constexpr int WA_THREADS = WA_WAVES * 64;
constexpr int WA_JB      = 256;   // sources staged per LDS block (one per thread)
// v_sin / v_cos take revolutions and are exact-period up to 256 of them: phases that provably stay below this need no
// explicit reduction (v_fract)
constexpr float WA_MAX_REV = 250.0f;

__device__ __forceinline__ float sgpr(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, v)));
}

// KT     wavenumbers per wave (6*KT accumulators per lane)
// SPLIT  the four waves share one wavenumber tile and split the staged sources; partial sums meet in LDS
// GRADS  false: only the embedding is wanted (d_cb = d_k = NULL): two sums per wavenumber instead of six
template <int KT, bool SPLIT, bool GRADS>
__global__ __launch_bounds__(WA_THREADS)
void we_aniso_fwd_kernel(const float* __restrict__ coordsA, const float* __restrict__ coordsB, const int layout,
                         const float* __restrict__ cb_magnitudes, const float* __restrict__ wavenumbers,
                         const uint8_t* __restrict__ mask,
                         float* __restrict__ out, float* __restrict__ d_cb, float* __restrict__ d_k,
                         const int N, const int K)
{
    __shared__ float4 s_ka[WA_JB + WA_WAVES];    // source positions   (padding: the loop reads one step ahead)
    __shared__ float4 s_kb[WA_JB + WA_WAVES];    // source C-beta vectors
    __shared__ int    s_wcount[WA_WAVES];
    __shared__ float  s_box[WA_WAVES][8];        // per wave: bounding box of the unpadded positions, largest |b|^2
    __shared__ int    s_last[WA_WAVES];
    constexpr int NS = GRADS ? 6 : 2;            // running sums per wavenumber
    __shared__ float  s_red[SPLIT ? (WA_WAVES - 1) * (NS * KT + 1) * 64 : 1];

    const int tid  = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // (observer blocks taken in a rotated order per (y, z), as in the isotropic kernel: in a batch of ragged lengths the
    // workgroups that are resident together then belong to different parts of their sequences; a padded batch of a
    // few items is handed out by the number of sources of its items instead, see we_ranked.h)
    int z = blockIdx.z, ytile = blockIdx.y;
    const unsigned wa_rot = ((unsigned)(0.6180339887f * (float)gridDim.x + 0.5f)) | 1u;
    int iblock = (int)((blockIdx.x + wa_rot * (blockIdx.z % gridDim.x) + 5u * blockIdx.y) % gridDim.x);
    proteus_we::we_ranked_workgroup(mask, N, z, ytile, iblock);

    const size_t zN = (size_t)z * (size_t)N;
    const float* az = coordsA + zN * 3;
    const float* bz = coordsB + zN * 3;
    const uint8_t* mz = mask ? mask + zN : nullptr;

    // ---- this lane's observer ----
    const int  i    = iblock * 64 + lane;
    const bool i_in = i < N;
    const int  ic   = i_in ? i : N - 1;
    float xi, yi, zi;
    if (layout == PROTEUS_COORDS_SOA) { xi = az[ic]; yi = az[(size_t)N + ic]; zi = az[2 * (size_t)N + ic]; }
    else                              { xi = az[3 * (size_t)ic]; yi = az[3 * (size_t)ic + 1]; zi = az[3 * (size_t)ic + 2]; }
    const bool i_valid   = i_in && !(mz && mz[ic]);
    const bool any_valid = __builtin_amdgcn_ballot_w64(i_valid) != 0;   // uniform over the workgroup

    // ---- this wave's wavenumbers: kr = k/2pi and ck = cb k/2pi, in revolutions per angstrom ----
    const int  k0          = SPLIT ? ytile * KT : (ytile * WA_WAVES + wave) * KT;
    const bool wave_active = k0 < K;
    float kr[KT], ck[KT];
#pragma unroll
    for (int t = 0; t < KT; ++t) {
        const int k = k0 + t;
        const float w = (k < K) ? wavenumbers[k] : 0.0f;
        const float c = (k < K) ? cb_magnitudes[k] : 0.0f;
        kr[t] = sgpr((float)((double)w * 0.15915494309189533577));
        ck[t] = sgpr((float)((double)w * (double)c * 0.15915494309189533577));
    }

    int  j_end = 0;
    bool use_fract = true;
    if (any_valid) {
        // ---- Can any phase of this workgroup leave the range v_sin / v_cos accept?  |phase| <= r kr + |A| ck with
        // r <= the distance from the observer to the farthest corner of the box of the unpadded positions and
        // |A| = |b_j . R| / r <= |b_j|.  One pass over the batch item (a few loads per thread) finds the box, the
        // largest |b_j| and where the unpadded sources end (the blocks behind that are never staged). ----
        {
            float lo[3] = {3.0e38f, 3.0e38f, 3.0e38f}, hi[3] = {-3.0e38f, -3.0e38f, -3.0e38f}, b2max = 0.f;
            int last = 0;
            for (int j = tid; j < N; j += WA_THREADS) {
                if (mz && mz[j]) continue;
                last = j + 1;
                float p[3], q[3];
                if (layout == PROTEUS_COORDS_SOA) {
                    p[0] = az[j]; p[1] = az[(size_t)N + j]; p[2] = az[2 * (size_t)N + j];
                    q[0] = bz[j]; q[1] = bz[(size_t)N + j]; q[2] = bz[2 * (size_t)N + j];
                } else {
                    p[0] = az[3 * (size_t)j]; p[1] = az[3 * (size_t)j + 1]; p[2] = az[3 * (size_t)j + 2];
                    q[0] = bz[3 * (size_t)j]; q[1] = bz[3 * (size_t)j + 1]; q[2] = bz[3 * (size_t)j + 2];
                }
#pragma unroll
                for (int c = 0; c < 3; ++c) { lo[c] = fminf(lo[c], p[c]); hi[c] = fmaxf(hi[c], p[c]); }
                const float b2 = q[0] * q[0] + q[1] * q[1] + q[2] * q[2];
                b2max = (b2 <= b2max) ? b2max : b2;          // (a NaN sticks: the reducing path is taken)
            }
#pragma unroll
            for (int c = 0; c < 3; ++c)
                for (int o = 32; o > 0; o >>= 1) { lo[c] = fminf(lo[c], __shfl_xor(lo[c], o)); hi[c] = fmaxf(hi[c], __shfl_xor(hi[c], o)); }
            for (int o = 32; o > 0; o >>= 1) {
                last = max(last, __shfl_xor(last, o));
                const float other = __shfl_xor(b2max, o);
                b2max = (other <= b2max) ? b2max : other;
            }
            if (lane == 0) {
#pragma unroll
                for (int c = 0; c < 3; ++c) { s_box[wave][c] = lo[c]; s_box[wave][3 + c] = hi[c]; }
                s_box[wave][6] = b2max;
                s_last[wave] = last;
            }
            __syncthreads();
            j_end = max(max(s_last[0], s_last[1]), max(s_last[2], s_last[3]));
#pragma unroll
            for (int c = 0; c < 3; ++c) {
                lo[c] = fminf(fminf(s_box[0][c], s_box[1][c]), fminf(s_box[2][c], s_box[3][c]));
                hi[c] = fmaxf(fmaxf(s_box[0][3 + c], s_box[1][3 + c]), fmaxf(s_box[2][3 + c], s_box[3][3 + c]));
            }
            b2max = s_box[0][6];
#pragma unroll
            for (int w = 1; w < WA_WAVES; ++w) b2max = (s_box[w][6] <= b2max) ? b2max : s_box[w][6];
            float kr_max = 0.f, ck_max = 0.f;
#pragma unroll
            for (int t = 0; t < KT; ++t) { kr_max = fmaxf(kr_max, fabsf(kr[t])); ck_max = fmaxf(ck_max, fabsf(ck[t])); }
            const float fx = fmaxf(fabsf(xi - lo[0]), fabsf(xi - hi[0]));
            const float fy = fmaxf(fabsf(yi - lo[1]), fabsf(yi - hi[1]));
            const float fz = fmaxf(fabsf(zi - lo[2]), fabsf(zi - hi[2]));
            const float rfar = __builtin_sqrtf(fx * fx + fy * fy + fz * fz);
            // NaN-safe: anything that is not provably below the limit takes the reducing path
            // (a padded observer's lane, whose coordinates may hold anything, has no say)
            const bool wave_safe = __builtin_amdgcn_ballot_w64(i_valid && !(rfar * kr_max + __builtin_sqrtf(b2max) * ck_max < WA_MAX_REV)) == 0;
            if (lane == 0) s_wcount[wave] = wave_safe ? 1 : 0;
            __syncthreads();
            use_fract = (s_wcount[0] & s_wcount[1] & s_wcount[2] & s_wcount[3]) == 0;
            __syncthreads();                       // s_wcount is reused by the staging below
        }
    }

    // Everything from here on exists twice, with and without the explicit phase reduction, as two instances of one
    // generic lambda: the running sums live inside it, so the two sets are never alive together.
    auto rest = [&](auto fract_c) {
    constexpr bool FRACT = decltype(fract_c)::value;
    float s1[KT], s2[KT], s3[KT], s4[KT], s5[KT], s6[KT];
#pragma unroll
    for (int t = 0; t < KT; ++t) { s1[t] = 0.f; s2[t] = 0.f; s3[t] = 0.f; s4[t] = 0.f; s5[t] = 0.f; s6[t] = 0.f; }
    float nzero = 0.f;

    if (any_valid) {
        for (int jb = 0; jb < j_end; jb += WA_JB) {
            // -- stage one block of sources, keeping only the unpadded ones --
            const int  j    = jb + tid;
            const bool j_in = j < N;
            const int  jc   = j_in ? j : N - 1;
            float xj, yj, zj, bx, by, bzj;
            if (layout == PROTEUS_COORDS_SOA) {
                xj = az[jc]; yj = az[(size_t)N + jc]; zj = az[2 * (size_t)N + jc];
                bx = bz[jc]; by = bz[(size_t)N + jc]; bzj = bz[2 * (size_t)N + jc];
            } else {
                xj = az[3 * (size_t)jc]; yj = az[3 * (size_t)jc + 1]; zj = az[3 * (size_t)jc + 2];
                bx = bz[3 * (size_t)jc]; by = bz[3 * (size_t)jc + 1]; bzj = bz[3 * (size_t)jc + 2];
            }
            const bool j_valid = j_in && !(mz && mz[jc]);

            const uint64_t bal   = __builtin_amdgcn_ballot_w64(j_valid);
            const int      below = __builtin_popcountll(bal & ((1ull << lane) - 1ull));
            __syncthreads();                       // previous block fully consumed
            if (lane == 0) s_wcount[wave] = __builtin_popcountll(bal);
            __syncthreads();
            int base = 0, nk = 0;
#pragma unroll
            for (int w = 0; w < WA_WAVES; ++w) { const int c = s_wcount[w]; base += (w < wave) ? c : 0; nk += c; }
            if (j_valid) {
                s_ka[base + below] = make_float4(xj, yj, zj, 0.f);
                s_kb[base + below] = make_float4(bx, by, bzj, 0.f);
            }
            __syncthreads();
            nk = __builtin_amdgcn_readfirstlane(nk);

            if (!wave_active) continue;

            // -- stream the staged sources --
            {
                const int first = SPLIT ? wave : 0;
                const int step  = SPLIT ? WA_WAVES : 1;
                float4 anext = s_ka[first], bnext = s_kb[first];
#pragma unroll 1
                for (int jj = first; jj < nk; jj += step) {
                    const float4 a = anext, b = bnext;
                    anext = s_ka[jj + step];
                    bnext = s_kb[jj + step];
                    const float dx = xi - a.x, dy = yi - a.y, dz = zi - a.z;
                    const float r2 = dx * dx + dy * dy + dz * dz;
                    const bool  ok = r2 != 0.0f;
                    const float inv = ok ? __builtin_amdgcn_rsqf(r2) : 0.0f;
                    // one Newton step on r = r2 * rsq(r2): r is then within 1 ulp of sqrt(r2)
                    const float r0 = r2 * inv;
                    const float e  = __builtin_fmaf(-r0, r0, r2);
                    const float r  = __builtin_fmaf(e, 0.5f * inv, r0);
                    const float A  = inv * __builtin_fmaf(b.x, dx, __builtin_fmaf(b.y, dy, b.z * dz));
                    const float v  = inv * A;
                    nzero += ok ? 0.0f : 1.0f;
#pragma unroll
                    for (int t = 0; t < KT; ++t) {
                        float ph = __builtin_fmaf(-A, ck[t], r * kr[t]);
                        if (FRACT) ph = __builtin_amdgcn_fractf(ph);
                        const float s = __builtin_amdgcn_sinf(ph);
                        const float c = __builtin_amdgcn_cosf(ph);
                        s1[t] = __builtin_fmaf(c, inv, s1[t]);
                        s2[t] = __builtin_fmaf(s, inv, s2[t]);
                        if (GRADS) {
                            s3[t] += c;
                            s4[t] += s;
                            s5[t] = __builtin_fmaf(c, v, s5[t]);
                            s6[t] = __builtin_fmaf(s, v, s6[t]);
                        }
                    }
                }
            }
        }
    }

    if (SPLIT) {
        // ---- the four waves' partial sums meet in LDS; wave 0 writes the rows ----
        __syncthreads();
        if (wave > 0) {
            float* q = s_red + (size_t)(wave - 1) * (NS * KT + 1) * 64 + lane;
#pragma unroll
            for (int t = 0; t < KT; ++t) {
                q[(NS * t + 0) * 64] = s1[t]; q[(NS * t + 1) * 64] = s2[t];
                if (GRADS) {
                    q[(NS * t + 2) * 64] = s3[t]; q[(NS * t + 3) * 64] = s4[t]; q[(NS * t + 4) * 64] = s5[t]; q[(NS * t + 5) * 64] = s6[t];
                }
            }
            q[NS * KT * 64] = nzero;
        }
        __syncthreads();
        if (wave > 0) return;
#pragma unroll 1
        for (int w = 0; w < WA_WAVES - 1; ++w) {
            const float* q = s_red + (size_t)w * (NS * KT + 1) * 64 + lane;
#pragma unroll
            for (int t = 0; t < KT; ++t) {
                s1[t] += q[(NS * t + 0) * 64]; s2[t] += q[(NS * t + 1) * 64];
                if (GRADS) {
                    s3[t] += q[(NS * t + 2) * 64]; s4[t] += q[(NS * t + 3) * 64]; s5[t] += q[(NS * t + 4) * 64]; s6[t] += q[(NS * t + 5) * 64];
                }
            }
            nzero += q[NS * KT * 64];
        }
    }

    if (!wave_active || !i_in) return;

    // ---- epilogue: each lane writes its own rows ----
    const size_t row = (zN + (size_t)i) * (size_t)(2 * K) + 2 * (size_t)k0;
    float* po = out  + row;
    float* pc = GRADS ? d_cb + row : nullptr;
    float* pk = GRADS ? d_k  + row : nullptr;
    const bool vec = (k0 + KT <= K) && ((K & 1) == 0) && ((KT & 1) == 0);   // rows and tile start 16-byte aligned
    // The scales are read again here rather than kept from the prologue: held across the main loop they
    // would take 2*KT scalar registers the loop needs for kr[] and ck[].
    const float* wn_e = wavenumbers;
    const float* cb_e = cb_magnitudes;
    asm volatile("" : "+s"(wn_e), "+s"(cb_e));
#pragma unroll
    for (int t = 0; t < KT; t += 2) {
        float o[4], g[4], h[4];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int   k  = k0 + t + u;
            const float wn = (k < K) ? wn_e[k] : 0.0f;
            const float cb = (k < K) ? cb_e[k] : 0.0f;
            // a padded observer's rows are zeros whatever its lane computed
            o[2 * u]     = i_valid ? s1[t + u] : 0.0f;
            o[2 * u + 1] = i_valid ? s2[t + u] : 0.0f;
            h[2 * u]     = i_valid ? __builtin_fmaf(cb, s6[t + u], -s4[t + u]) : 0.0f;
            h[2 * u + 1] = i_valid ? __builtin_fmaf(-cb, s5[t + u], s3[t + u] - nzero) : 0.0f;
            g[2 * u]     = i_valid ? wn * s6[t + u] : 0.0f;
            g[2 * u + 1] = i_valid ? -wn * s5[t + u] : 0.0f;
        }
        if (vec) {
            *reinterpret_cast<float4*>(po + 2 * t) = make_float4(o[0], o[1], o[2], o[3]);
            if (GRADS) {
                *reinterpret_cast<float4*>(pc + 2 * t) = make_float4(g[0], g[1], g[2], g[3]);
                *reinterpret_cast<float4*>(pk + 2 * t) = make_float4(h[0], h[1], h[2], h[3]);
            }
        } else {
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                if (k0 + t + u < K) {
                    po[2 * (t + u)] = o[2 * u]; po[2 * (t + u) + 1] = o[2 * u + 1];
                    if (GRADS) {
                        pc[2 * (t + u)] = g[2 * u]; pc[2 * (t + u) + 1] = g[2 * u + 1];
                        pk[2 * (t + u)] = h[2 * u]; pk[2 * (t + u) + 1] = h[2 * u + 1];
                    }
                }
            }
        }
    }
    };
    if (use_fract) rest(std::true_type{}); else rest(std::false_type{});
}

struct WaVariant { const char* name; int kt; bool split; };
// index 0 is "automatic"; the others force a tile
const WaVariant kVariants[] = {
    {"auto", 0, false},
    {"kt16", 16, false},
    {"kt8", 8, false},
    {"kt16_split", 16, true},
    {"kt8_split", 8, true},
};
constexpr int kNumVariants = (int)(sizeof(kVariants) / sizeof(kVariants[0]));

template <int KT, bool SPLIT, bool GRADS>
int launch(const float* ca, const float* cbv, int layout, const float* cbm, const float* wn, const uint8_t* mask,
           float* out, float* d_cb, float* d_k, int Z, int N, int K, hipStream_t st)
{
    const int iblocks = (N + 63) / 64;
    const int ktiles  = SPLIT ? (K + KT - 1) / KT : (K + KT * WA_WAVES - 1) / (KT * WA_WAVES);
    dim3 grid(iblocks, ktiles, Z);
    hipLaunchKernelGGL((we_aniso_fwd_kernel<KT, SPLIT, GRADS>), grid, dim3(WA_THREADS), 0, st,
                       ca, cbv, layout, cbm, wn, mask, out, d_cb, d_k, N, K);
    return (int)hipGetLastError();
}

}  // namespace

extern "C" int proteus_we_aniso_num_variants(void) { return kNumVariants; }

extern "C" const char* proteus_we_aniso_variant_name(int tuning) {
    return (tuning >= 0 && tuning < kNumVariants) ? kVariants[tuning].name : nullptr;
}

extern "C" int proteus_we_aniso_fwd_check(const float* coordsA, const float* coordsB, int coords_layout,
                                          const float* cb_magnitudes, const float* wavenumbers, const uint8_t* mask,
                                          const float* out, const float* d_cb, const float* d_k,
                                          int Z, int N, int K, int tuning)
{
    (void)mask;
    if (!coordsA || !coordsB || !cb_magnitudes || !wavenumbers || !out) return PROTEUS_ERR_NULL_POINTER;
    if ((d_cb == nullptr) != (d_k == nullptr)) return PROTEUS_ERR_NULL_POINTER;       // both derivatives or neither
    if (Z <= 0 || N <= 0 || K <= 0) return PROTEUS_ERR_BAD_SHAPE;
    if (N > PROTEUS_WE_MAX_N || K > PROTEUS_WE_MAX_K || Z > 65535) return PROTEUS_ERR_BAD_SHAPE;
    if (coords_layout != PROTEUS_COORDS_SOA && coords_layout != PROTEUS_COORDS_AOS) return PROTEUS_ERR_BAD_LAYOUT;
    if (tuning < 0 || tuning >= kNumVariants) return PROTEUS_ERR_BAD_TUNING;
    if (((uintptr_t)out & 15) || ((uintptr_t)d_cb & 15) || ((uintptr_t)d_k & 15)) return PROTEUS_ERR_BAD_ALIGNMENT;   // (NULL passes)
    return PROTEUS_OK;
}

extern "C" int proteus_we_aniso_fwd(const float* coordsA, const float* coordsB, int coords_layout,
                                    const float* cb_magnitudes, const float* wavenumbers, const uint8_t* mask,
                                    float* out, float* d_cb, float* d_k,
                                    int Z, int N, int K, int tuning, void* stream)
{
    const int rc = proteus_we_aniso_fwd_check(coordsA, coordsB, coords_layout, cb_magnitudes, wavenumbers, mask,
                                              out, d_cb, d_k, Z, N, K, tuning);
    if (rc != PROTEUS_OK) return rc;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);

    int kt = kVariants[tuning].kt;
    bool split = kVariants[tuning].split;
    if (tuning == 0) {
        // With the partial derivatives (six sums per wavenumber) eight wavenumbers per wave measured faster than sixteen
        // at every size tried (92 VGPRs, five waves per SIMD, against 155 and three); the embedding alone (two sums)
        // is fastest with sixteen and the source split wherever the split is possible.  The split itself is chosen by
        // the least estimated issue time, instructions per wave x rounds of 1024 waves, with a penalty when a SIMD
        // would hold a single wave; a tie goes to the split kernel (measured 4 % faster at N = 16384 and at 8 x 1024).
        kt = d_cb ? 8 : (N >= 4 * 64 ? 16 : 8);
        const long iblocks = ((long)N + 63) / 64 * Z;
        const long ktiles  = ((long)K + kt - 1) / kt;
        double best = 1e300;
        for (int csp = 1; csp >= 0; --csp) {
            if (csp && N < 2 * WA_WAVES) continue;          // (fewer sources than a split could share out)
            const long nwaves = csp ? iblocks * ktiles * WA_WAVES : iblocks * ((ktiles + WA_WAVES - 1) / WA_WAVES) * WA_WAVES;
            const double keys = csp ? (double)N / WA_WAVES : (double)N;
            const double rounds = (double)((nwaves + 1023) / 1024);
            double est = rounds * keys * ((d_cb ? 13.0 : 9.0) * kt + 22.0);
            if (nwaves < 2048) est *= 1.25;
            if (est < best * 0.999) { best = est; split = csp != 0; }
        }
        if (!d_cb && N >= 4 * 64) split = true;
    }
#define WA_GO(KT_, GR_) (split ? launch<KT_, true, GR_>(coordsA, coordsB, coords_layout, cb_magnitudes, wavenumbers, mask, out, d_cb, d_k, Z, N, K, st) \
                               : launch<KT_, false, GR_>(coordsA, coordsB, coords_layout, cb_magnitudes, wavenumbers, mask, out, d_cb, d_k, Z, N, K, st))
    if (d_cb) {
        if (kt == 16) return WA_GO(16, true);
        return WA_GO(8, true);
    }
    if (kt == 16) return WA_GO(16, false);
    return WA_GO(8, false);
#undef WA_GO
}
