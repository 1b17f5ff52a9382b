// Wavefunction Embedding forward with the reference kernel's in-kernel dropout
// (utils/model_utils/wf_embedding/isotropic/cuda/wf_embedding_kernel.cu:27-46 the hash, :227-232 its use; native
// signature wf_embedding_if.cpp:20-25: dropout_p, rng_seed).
//
// Per (batch item z, observer i, source j, wavenumber k) the reference keeps a term iff
//     float(hash5(z, i, j, k, seed)) / float(UINT32_MAX) >= dropout_p
// and divides what it keeps by 1 - dropout_p; the saved cos / sin sums carry the same mask and factor
// (kernel.cu:234-238 sum the dropped values times r).  hash5 is integer arithmetic, so the mask is reproduced to
// the bit: the three terms of (z, i, j) are xor-ed into the seed once per lane and per source, the term of k is a
// wave-uniform constant per wavenumber, and what remains per unit is the final mix (four shift-xors and two 32-bit
// multiplies) and one unsigned compare against the smallest h that is kept (found on the
// host with the reference's own float expression, which is monotone in h).
//
// The module never asks for dropout (wf_embedding.py:44 passes 0.0), so this is a plain kernel, not a tuned one:
// the mapping of we_fwd.hip without its tile choice (lane = observer, wave = 16 wavenumbers, the four waves of a
// workgroup four tiles of the same observers, sources staged in LDS and compacted to the unpadded ones), phases
// always reduced with v_fract.  About 20 vector instructions per unit against 7 without dropout.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "proteus_hip.h"

namespace {

constexpr int WD_WAVES   = 4;
constexpr int WD_THREADS = WD_WAVES * 64;
constexpr int WD_JB      = 256;   // sources staged per LDS block (one per thread)
constexpr int WD_KT      = 16;    // wavenumbers per wave

__device__ __forceinline__ float wd_sgpr(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, v)));
}

// the last five lines of hash5 (kernel.cu:36-40)
__device__ __forceinline__ unsigned wd_final_mix(unsigned h) {
    h = (h ^ (h >> 16)) * 0x85ebca6bu;
    h ^= (h >> 13);
    h = (h ^ (h >> 16)) * 0xc2b2ae35u;
    h ^= (h >> 16);
    return h;
}

// MAG: the weight m(r) of a source (kernel.cu:192-206): 0: 1, 1: 1/r, 2: 1/log2(r), 3: 1/sqrt(r)
template <int MAG>
__global__ __launch_bounds__(WD_THREADS)
void we_dropout_fwd_kernel(const float* __restrict__ coords, const int layout,
                           const float* __restrict__ wavenumbers, const uint8_t* __restrict__ mask,
                           float* __restrict__ out, float* __restrict__ cos_sums, float* __restrict__ sin_sums,
                           const int N, const int K, const unsigned seed, const unsigned h_keep, const float inv_keep)
{
    __shared__ uint4 s_keys[WD_JB + 1];       // (x, y, z bits, the source's hash term); one entry of padding: read one ahead
    __shared__ int   s_wcount[WD_WAVES];
    const int tid  = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int z    = blockIdx.z;
    const size_t zN = (size_t)z * (size_t)N;
    const float* cz = coords + zN * 3;
    const uint8_t* mz = mask ? mask + zN : nullptr;
    auto position = [&](const int t, float& x, float& y, float& w) {
        if (layout == PROTEUS_COORDS_SOA) { x = cz[t]; y = cz[(size_t)N + t]; w = cz[2 * (size_t)N + t]; }
        else                              { x = cz[3 * (size_t)t]; y = cz[3 * (size_t)t + 1]; w = cz[3 * (size_t)t + 2]; }
    };

    // ---- this lane's observer ----
    const int  i    = blockIdx.x * 64 + lane;
    const bool i_in = i < N;
    const int  ic   = i_in ? i : N - 1;
    float xi, yi, zi;
    position(ic, xi, yi, zi);
    const bool i_valid = i_in && !(mz && mz[ic]);
    // seed and the terms of z and i (kernel.cu:30-32)
    const unsigned h_zi = seed ^ ((unsigned)z * 0x85ebca6bu + 0x9e3779b9u) ^ ((unsigned)i * 0xc2b2ae35u + 0x165667b1u);

    // ---- this wave's wavenumbers (revolutions per angstrom) and their hash terms (kernel.cu:34) ----
    const int  k0 = (blockIdx.y * WD_WAVES + wave) * WD_KT;
    const bool wave_active = k0 < K;
    float kr[WD_KT];
    unsigned hk[WD_KT];
#pragma unroll
    for (int t = 0; t < WD_KT; ++t) {
        const int k = k0 + t;
        const float w = (k < K) ? wavenumbers[k] : 0.0f;
        kr[t] = wd_sgpr((float)((double)w * 0.15915494309189533577));
        hk[t] = (unsigned)__builtin_amdgcn_readfirstlane((int)((unsigned)k * 0x85ebca6bu + 0x1b873593u));
    }

    float acc_oc[WD_KT], acc_os[WD_KT], acc_c[WD_KT], acc_s[WD_KT];
#pragma unroll
    for (int t = 0; t < WD_KT; ++t) { acc_oc[t] = 0.f; acc_os[t] = 0.f; acc_c[t] = 0.f; acc_s[t] = 0.f; }

    for (int jb = 0; jb < N; jb += WD_JB) {
        // -- stage one block of sources, keeping only the unpadded ones; a source brings the term of its index --
        const int  j    = jb + tid;
        const bool j_in = j < N;
        const int  jc   = j_in ? j : N - 1;
        float xj, yj, zj;
        position(jc, xj, yj, zj);
        const bool j_valid = j_in && !(mz && mz[jc]);
        const uint64_t bal   = __builtin_amdgcn_ballot_w64(j_valid);
        const int      below = __builtin_popcountll(bal & ((1ull << lane) - 1ull));
        __syncthreads();                       // previous block fully consumed
        if (lane == 0) s_wcount[wave] = __builtin_popcountll(bal);
        __syncthreads();
        int base = 0, nk = 0;
#pragma unroll
        for (int w = 0; w < WD_WAVES; ++w) { const int c = s_wcount[w]; base += (w < wave) ? c : 0; nk += c; }
        if (j_valid)
            s_keys[base + below] = make_uint4(__builtin_bit_cast(unsigned, xj), __builtin_bit_cast(unsigned, yj),
                                              __builtin_bit_cast(unsigned, zj), (unsigned)j * 0x27d4eb2fu + 0xd6e8feb8u);
        __syncthreads();
        nk = __builtin_amdgcn_readfirstlane(nk);
        if (!wave_active) continue;

        uint4 knext = s_keys[0];
#pragma unroll 1
        for (int jj = 0; jj < nk; ++jj) {
            const uint4 kj = knext;
            knext = s_keys[jj + 1];
            const float dx = xi - __builtin_bit_cast(float, kj.x), dy = yi - __builtin_bit_cast(float, kj.y),
                        dz = zi - __builtin_bit_cast(float, kj.z);
            const float r2 = dx * dx + dy * dy + dz * dz;
            const bool  ok = r2 != 0.0f;
            const float inv = ok ? __builtin_amdgcn_rsqf(r2) : 0.0f;
            // one Newton step on r = r2 * rsq(r2): r is then within 1 ulp of sqrt(r2)
            const float r0 = r2 * inv;
            const float e  = __builtin_fmaf(-r0, r0, r2);
            const float r  = __builtin_fmaf(e, 0.5f * inv, r0);
            // the r = 0 pair (the observer itself, a coincident point) gets weight 0 in both sums
            float m = inv;
            if (MAG == 0) m = ok ? 1.0f : 0.0f;
            if (MAG == 2) m = ok ? __builtin_amdgcn_rcpf(__builtin_amdgcn_logf(r)) : 0.0f;   // v_log_f32 is log2
            if (MAG == 3) m = ok ? __builtin_amdgcn_rsqf(r) : 0.0f;
            const float mr = m * r;
            const unsigned h_zij = h_zi ^ kj.w;
#pragma unroll
            for (int t = 0; t < WD_KT; ++t) {
                const float ph = __builtin_amdgcn_fractf(r * kr[t]);
                const bool keep = wd_final_mix(h_zij ^ hk[t]) >= h_keep;
                const float cs = keep ? __builtin_amdgcn_cosf(ph) : 0.0f;
                const float sn = keep ? __builtin_amdgcn_sinf(ph) : 0.0f;
                acc_oc[t] = __builtin_fmaf(cs, m, acc_oc[t]);
                acc_os[t] = __builtin_fmaf(sn, m, acc_os[t]);
                acc_c[t]  = __builtin_fmaf(cs, mr, acc_c[t]);
                acc_s[t]  = __builtin_fmaf(sn, mr, acc_s[t]);
            }
        }
    }
    if (!wave_active || !i_in) return;

    // ---- epilogue: each lane writes its own rows; what was kept is divided by 1 - dropout_p; a padded observer gets
    //      exact zeros whatever its lane accumulated ----
    const size_t row = zN + (size_t)i;
    float* o  = out + row * (size_t)(2 * K) + 2 * (size_t)k0;
    float* pc = cos_sums + row * (size_t)K + k0;
    float* ps = sin_sums + row * (size_t)K + k0;
#pragma unroll
    for (int t = 0; t < WD_KT; ++t) {
        if (k0 + t < K) {
            o[2 * t]     = i_valid ? acc_oc[t] * inv_keep : 0.0f;
            o[2 * t + 1] = i_valid ? acc_os[t] * inv_keep : 0.0f;
            pc[t] = i_valid ? acc_c[t] * inv_keep : 0.0f;
            ps[t] = i_valid ? acc_s[t] * inv_keep : 0.0f;
        }
    }
}

template <int MAG>
int launch_dropout(const float* coords, int layout, const float* wn, const uint8_t* mask, float* out, float* cs, float* ss,
                   int Z, int N, int K, unsigned seed, unsigned h_keep, float inv_keep, hipStream_t st)
{
    dim3 grid((N + 63) / 64, (K + WD_KT * WD_WAVES - 1) / (WD_KT * WD_WAVES), Z);
    hipLaunchKernelGGL((we_dropout_fwd_kernel<MAG>), grid, dim3(WD_THREADS), 0, st,
                       coords, layout, wn, mask, out, cs, ss, N, K, seed, h_keep, inv_keep);
    return (int)hipGetLastError();
}

// the reference's test (kernel.cu:43-45), on the host
bool kept(uint32_t h, float p) { return (float)h / (float)UINT32_MAX >= p; }

}  // namespace

extern "C" uint32_t proteus_we_dropout_threshold(float dropout_p)
{
    // the smallest h that the reference keeps: its test is monotone in h (the conversion to float rounds
    // monotonically), so a bisection over the 32-bit range finds it
    if (kept(0u, dropout_p)) return 0u;
    uint32_t lo = 0u, hi = UINT32_MAX;          // kept(lo) false, kept(hi) true (checked by the caller for p < 1)
    while (hi - lo > 1u) {
        const uint32_t mid = lo + (hi - lo) / 2u;
        if (kept(mid, dropout_p)) hi = mid; else lo = mid;
    }
    return hi;
}

extern "C" int proteus_we_dropout_fwd_check(const float* coords, int coords_layout,
                                            const float* wavenumbers, const uint8_t* mask,
                                            const float* out, const float* cos_sums, const float* sin_sums,
                                            int Z, int N, int K, int magnitude_type, float dropout_p)
{
    (void)mask;
    if (!coords || !wavenumbers || !out || !cos_sums || !sin_sums) return PROTEUS_ERR_NULL_POINTER;
    if (Z <= 0 || N <= 0 || K <= 0) return PROTEUS_ERR_BAD_SHAPE;
    if (N > PROTEUS_WE_MAX_N || K > PROTEUS_WE_MAX_K || Z > 65535) return PROTEUS_ERR_BAD_SHAPE;
    if (coords_layout != PROTEUS_COORDS_SOA && coords_layout != PROTEUS_COORDS_AOS) return PROTEUS_ERR_BAD_LAYOUT;
    if (magnitude_type < 0 || magnitude_type > 3) return PROTEUS_ERR_UNSUPPORTED;
    // 0 <= p < 1 (NaN fails both comparisons); with p = 1 the reference divides by zero
    if (!(dropout_p >= 0.0f) || !(dropout_p < 1.0f)) return PROTEUS_ERR_BAD_SHAPE;
    return PROTEUS_OK;
}

extern "C" int proteus_we_dropout_fwd(const float* coords, int coords_layout,
                                      const float* wavenumbers, const uint8_t* mask,
                                      float* out, float* cos_sums, float* sin_sums,
                                      int Z, int N, int K, int magnitude_type, float dropout_p, uint32_t rng_seed, void* stream)
{
    const int rc = proteus_we_dropout_fwd_check(coords, coords_layout, wavenumbers, mask, out, cos_sums, sin_sums,
                                                Z, N, K, magnitude_type, dropout_p);
    if (rc != PROTEUS_OK) return rc;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    const uint32_t h_keep = proteus_we_dropout_threshold(dropout_p);
    const float inv_keep = 1.0f / (1.0f - dropout_p);
    switch (magnitude_type) {
        case 0:  return launch_dropout<0>(coords, coords_layout, wavenumbers, mask, out, cos_sums, sin_sums, Z, N, K, rng_seed, h_keep, inv_keep, st);
        case 1:  return launch_dropout<1>(coords, coords_layout, wavenumbers, mask, out, cos_sums, sin_sums, Z, N, K, rng_seed, h_keep, inv_keep, st);
        case 2:  return launch_dropout<2>(coords, coords_layout, wavenumbers, mask, out, cos_sums, sin_sums, Z, N, K, rng_seed, h_keep, inv_keep, st);
        default: return launch_dropout<3>(coords, coords_layout, wavenumbers, mask, out, cos_sums, sin_sums, Z, N, K, rng_seed, h_keep, inv_keep, st);
    }
}
