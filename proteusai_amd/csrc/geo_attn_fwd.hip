// RBF-scaled geometric flash-attention forward for gfx950 (MI355X), d_head = 64.
//
// What it computes (README.md:40 logits on the flash structure of
// old/old_scripts/attn/geometric_attn.py:57-260):
//   s_ij = (q_i . k_j)/sqrt(d) * (1 + exp(-|r_i - r_j|^2 / (2 sigma_h^2))),  -inf for padded keys
//   O_i  = softmax_j(s_ij) V_j,  L_i = logsumexp_j s_ij;  padded/empty rows -> O = 0, L = -inf
//
// Mapping to the machine.  A workgroup is 4 waves; a wave owns 32 queries of one
// (batch, head) and walks the keys in tiles of 64 that the workgroup stages in
// LDS (K row-major, V transposed, key coordinates pre-scaled for the head).
// Both products run on v_mfma_f32_32x32x16_bf16 and are computed TRANSPOSED:
//   S^T (keys x queries)  = K_tile (A, from LDS) x Q^T (B, registers, loaded once)
//   O^T (d x queries)    += V^T_tile (A, from LDS) x P^T (B, registers)
// In the 32x32 accumulator layout a lane holds 16 rows of ONE column, so with
// queries on the columns each lane owns one query: the row maximum, the
// exponentials and the row sum are in-lane except for one exchange between the
// two half-waves, and the S^T accumulator registers are, after conversion to
// bf16, already the B operand of the second product (the contraction index is
// merely visited in the permuted order the accumulator layout dictates, and the
// V^T operand is read from LDS in that same order).
// The geometric multiplier is evaluated per score from the lane's query
// coordinates and broadcast reads of the staged key coordinates; nothing of
// size N x N exists anywhere.

#include <hip/hip_runtime.h>
#include <stdint.h>
#include "proteus_hip.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float  floatx16 __attribute__((ext_vector_type(16)));
typedef float  floatx2 __attribute__((ext_vector_type(2)));

constexpr int GA_WAVES   = 4;
constexpr int GA_THREADS = GA_WAVES * 64;
constexpr int GA_BM      = GA_WAVES * 32;   // queries per workgroup
constexpr int GA_BN      = 64;              // keys per tile
constexpr int GA_D       = 64;              // head dim
constexpr int GA_LDK     = GA_D + 8;        // LDS row stride of the K tile (bf16 elements)
constexpr int GA_LDV     = GA_BN + 8;       // LDS row stride of the V^T tile
constexpr float LOG2E    = 1.4426950408889634f;

struct __align__(16) Smem {
    uint16_t k[GA_BN * GA_LDK];      // K tile   [key][d]
    uint16_t vt[GA_D * GA_LDV];      // V^T tile [d][key]
    float    cx[GA_BN], cy[GA_BN], cz[GA_BN];   // key coordinates * sqrt(log2(e)/(2 sigma^2))
    float    bias[GA_BN];            // 0 for a valid key, -inf for a padded / out-of-range one
    int      flags[2];               // [0] tile has a masked key, [1] tile has a valid key
    int      n_eff;                  // 1 + index of the last valid key of this batch item
};

// Exchange between the two half-waves: lane l and lane l^32 hold the same query.
// v_permlane32_swap exchanges lanes 32..63 of its first register with lanes 0..31
// of its second; starting from two copies of x, the first ends up holding the
// low half's value in every lane and the second the high half's.  (Written as
// inline assembly: the compiler builtin folds the two results of identical
// inputs into one.)
__device__ __forceinline__ void xhalf_both(float x, float& lo, float& hi) {
    lo = x; hi = x;
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(lo), "+v"(hi));
}
__device__ __forceinline__ float xhalf_max(float x) { float a, b; xhalf_both(x, a, b); return fmaxf(a, b); }
__device__ __forceinline__ float xhalf_sum(float x) { float a, b; xhalf_both(x, a, b); return a + b; }

__device__ __forceinline__ unsigned pack_bf16(float a, float b) {
    floatx2 f = {a, b};
    return __builtin_bit_cast(unsigned, __builtin_convertvector(f, bf16x2));
}

__global__ __launch_bounds__(GA_THREADS)
void geo_attn_fwd_kernel(const uint16_t* __restrict__ Q, const uint16_t* __restrict__ K,
                         const uint16_t* __restrict__ V, const float* __restrict__ coords,
                         const float* __restrict__ sigma, const uint8_t* __restrict__ key_pad,
                         float* __restrict__ O, float* __restrict__ L,
                         const int H, const int N)
{
    __shared__ Smem sm;

    const int tid  = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int half = lane >> 5;          // which 4-row group of every 8 accumulator rows
    const int col  = lane & 31;          // accumulator column = query within the wave

    const int zh = blockIdx.y;
    const int z  = zh / H;
    const int h  = zh - z * H;
    const size_t head_off = (size_t)zh * (size_t)N * GA_D;
    const uint16_t* Qh = Q + head_off;
    const uint16_t* Kh = K + head_off;
    const uint16_t* Vh = V + head_off;
    const float*    cz = coords + (size_t)z * N * 3;
    const uint8_t*  mz = key_pad ? key_pad + (size_t)z * N : nullptr;

    const float sg = sigma[h];
    // exp(-d^2/(2 sg^2)) = exp2(-(d*cs)^2) with cs = sqrt(log2(e)/2)/sg
    const float cscale = 0.84932180028801907f / sg;

    // ---- 1 + index of the last unpadded key: trailing padded tiles are never visited ----
    if (tid == 0) sm.n_eff = mz ? 0 : N;
    __syncthreads();
    if (mz) {
        int last = 0;
        for (int j = tid; j < N; j += GA_THREADS) if (!mz[j]) last = j + 1;
        // wave maximum, then one LDS atomic per wave
        for (int o = 32; o > 0; o >>= 1) last = max(last, __shfl_xor(last, o));
        if (lane == 0) atomicMax(&sm.n_eff, last);
    }
    __syncthreads();
    const int n_eff = sm.n_eff;

    // ---- this lane's query ----
    const int  q      = blockIdx.x * GA_BM + wave * 32 + col;
    const bool q_in   = q < N;
    const int  qc     = q_in ? q : N - 1;
    const bool q_ok   = q_in && !(mz && mz[qc]);
    const float qx = cz[3 * qc] * cscale, qy = cz[3 * qc + 1] * cscale, qz = cz[3 * qc + 2] * cscale;

    // Q^T as the B operand: lane (half, col) holds d = 16*ks + 8*half + 0..7 of its query,
    // pre-multiplied by 1/sqrt(64) = 2^-3 (exact in bf16)
    bf16x8 qreg[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
        const uint4 raw = *reinterpret_cast<const uint4*>(Qh + (size_t)qc * GA_D + ks * 16 + half * 8);
        bf16x8 v = __builtin_bit_cast(bf16x8, raw);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = (__bf16)((float)v[e] * 0.125f);
        qreg[ks] = v;
    }

    floatx16 oacc[2];
#pragma unroll
    for (int dt = 0; dt < 2; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[dt][r] = 0.f;
    float m_run = -INFINITY;     // running maximum of s (natural units), same in both half-waves
    float l_run = 0.f;           // this half-wave's part of the running sum

    // staging roles
    const int kp   = tid & 31;   // V: key pair
    const int vdc  = tid >> 5;   // V: 8-wide d chunk
    const int krow = tid >> 3;   // K: key row (0..31, +32 on the second pass)
    const int kdc  = tid & 7;    // K: 8-wide d chunk

    for (int j0 = 0; j0 < n_eff; j0 += GA_BN) {
        // ---- global -> registers ----
        uint4 kreg[2], vreg[2];
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            const int j = j0 + krow + 32 * p;
            kreg[p] = (j < N) ? *reinterpret_cast<const uint4*>(Kh + (size_t)j * GA_D + kdc * 8) : make_uint4(0, 0, 0, 0);
            const int jv = j0 + 2 * kp + p;
            vreg[p] = (jv < N) ? *reinterpret_cast<const uint4*>(Vh + (size_t)jv * GA_D + vdc * 8) : make_uint4(0, 0, 0, 0);
        }
        float kcx = 0.f, kcy = 0.f, kcz = 0.f, kb = 0.f;
        bool kvalid = false;
        if (tid < GA_BN) {
            const int j = j0 + tid;
            if (j < N) {
                kcx = cz[3 * j] * cscale; kcy = cz[3 * j + 1] * cscale; kcz = cz[3 * j + 2] * cscale;
                kvalid = !(mz && mz[j]);
            }
            kb = kvalid ? 0.f : -INFINITY;
        }

        __syncthreads();      // previous tile fully consumed
        // ---- registers -> LDS ----
#pragma unroll
        for (int p = 0; p < 2; ++p)
            *reinterpret_cast<uint4*>(&sm.k[(krow + 32 * p) * GA_LDK + kdc * 8]) = kreg[p];
        {
            const uint16_t* v0 = reinterpret_cast<const uint16_t*>(&vreg[0]);
            const uint16_t* v1 = reinterpret_cast<const uint16_t*>(&vreg[1]);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const unsigned pr = (unsigned)v0[e] | ((unsigned)v1[e] << 16);
                *reinterpret_cast<unsigned*>(&sm.vt[(vdc * 8 + e) * GA_LDV + 2 * kp]) = pr;
            }
        }
        if (tid < GA_BN) {
            sm.cx[tid] = kcx; sm.cy[tid] = kcy; sm.cz[tid] = kcz; sm.bias[tid] = kb;
            const uint64_t bal = __builtin_amdgcn_ballot_w64(kvalid);
            if (tid == 0) { sm.flags[0] = (bal != ~0ull); sm.flags[1] = (bal != 0ull); }
        }
        __syncthreads();
        const bool has_masked = sm.flags[0] != 0;
        const bool has_valid  = sm.flags[1] != 0;
        if (!has_valid) continue;

        // ---- S^T = K_tile x Q^T : two 32-key blocks ----
        floatx16 sacc[2];
#pragma unroll
        for (int mt = 0; mt < 2; ++mt) {
#pragma unroll
            for (int r = 0; r < 16; ++r) sacc[mt][r] = 0.f;
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) {
                const uint4 raw = *reinterpret_cast<const uint4*>(&sm.k[(mt * 32 + col) * GA_LDK + ks * 16 + half * 8]);
                sacc[mt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, raw), qreg[ks], sacc[mt], 0, 0, 0);
            }
        }

        // ---- geometric multiplier, mask, tile maximum ----
        // accumulator register r of block mt is key  mt*32 + 8*(r/4) + 4*half + (r%4)
        float tmax = -INFINITY;
#pragma unroll
        for (int mt = 0; mt < 2; ++mt) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int kb0 = mt * 32 + 8 * g + 4 * half;
                const float4 kx = *reinterpret_cast<const float4*>(&sm.cx[kb0]);
                const float4 ky = *reinterpret_cast<const float4*>(&sm.cy[kb0]);
                const float4 kz = *reinterpret_cast<const float4*>(&sm.cz[kb0]);
                const float kxs[4] = {kx.x, kx.y, kx.z, kx.w};
                const float kys[4] = {ky.x, ky.y, ky.z, ky.w};
                const float kzs[4] = {kz.x, kz.y, kz.z, kz.w};
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const float dx = qx - kxs[v], dy = qy - kys[v], dz = qz - kzs[v];
                    const float d2 = dx * dx + dy * dy + dz * dz;
                    const float rbf = __builtin_amdgcn_exp2f(-d2);
                    const float s = sacc[mt][4 * g + v];
                    sacc[mt][4 * g + v] = __builtin_fmaf(s, rbf, s);
                }
                if (has_masked) {
                    const float4 b = *reinterpret_cast<const float4*>(&sm.bias[kb0]);
                    sacc[mt][4 * g + 0] += b.x; sacc[mt][4 * g + 1] += b.y;
                    sacc[mt][4 * g + 2] += b.z; sacc[mt][4 * g + 3] += b.w;
                }
#pragma unroll
                for (int v = 0; v < 4; ++v) tmax = fmaxf(tmax, sacc[mt][4 * g + v]);
            }
        }
        tmax = xhalf_max(tmax);

        // ---- online softmax: rescale only when some query's maximum moved ----
        const float m_new = fmaxf(m_run, tmax);
        if (__builtin_amdgcn_ballot_w64(m_new > m_run) != 0) {
            const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
            const float alpha = __builtin_amdgcn_exp2f((m_run - m_use) * LOG2E);   // m_run = -inf -> 0
#pragma unroll
            for (int dt = 0; dt < 2; ++dt)
#pragma unroll
                for (int r = 0; r < 16; ++r) oacc[dt][r] *= alpha;
            l_run *= alpha;
            m_run = m_new;
        }
        const float mneg = -((m_run == -INFINITY) ? 0.f : m_run) * LOG2E;

        // ---- P^T (bf16) and O^T += V^T_tile x P^T ----
#pragma unroll
        for (int mt = 0; mt < 2; ++mt) {
            float p[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                p[r] = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[mt][r], LOG2E, mneg));
                l_run += p[r];
            }
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                // contraction slot e of this half-wave is key mt*32 + 16*t + 8*(e/4) + 4*half + (e%4)
                uint4 pb;
                pb.x = pack_bf16(p[8 * t + 0], p[8 * t + 1]);
                pb.y = pack_bf16(p[8 * t + 2], p[8 * t + 3]);
                pb.z = pack_bf16(p[8 * t + 4], p[8 * t + 5]);
                pb.w = pack_bf16(p[8 * t + 6], p[8 * t + 7]);
                const int key0 = mt * 32 + 16 * t + 4 * half;
#pragma unroll
                for (int dt = 0; dt < 2; ++dt) {
                    const uint16_t* row = &sm.vt[(dt * 32 + col) * GA_LDV + key0];
                    const uint2 a0 = *reinterpret_cast<const uint2*>(row);
                    const uint2 a1 = *reinterpret_cast<const uint2*>(row + 8);
                    const uint4 a = make_uint4(a0.x, a0.y, a1.x, a1.y);
                    oacc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, pb), oacc[dt], 0, 0, 0);
                }
            }
        }
    }

    // ---- epilogue ----
    const float l_tot = xhalf_sum(l_run);
    const bool  row_ok = q_ok && l_tot > 0.f;
    const float inv_l = row_ok ? 1.0f / l_tot : 0.f;
    if (q_in) {
        float* orow = O + head_off + (size_t)q * GA_D;
#pragma unroll
        for (int dt = 0; dt < 2; ++dt)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                float4 v = make_float4(oacc[dt][4 * g] * inv_l, oacc[dt][4 * g + 1] * inv_l,
                                       oacc[dt][4 * g + 2] * inv_l, oacc[dt][4 * g + 3] * inv_l);
                *reinterpret_cast<float4*>(orow + dt * 32 + 8 * g + 4 * half) = v;
            }
        if (L && half == 0) L[(size_t)zh * N + q] = row_ok ? m_run + __logf(l_tot) : -INFINITY;
    }
}

struct GaVariant { const char* name; };
const GaVariant kVariants[] = { {"auto"}, {"w4_q32_k64"} };
constexpr int kNumVariants = (int)(sizeof(kVariants) / sizeof(kVariants[0]));

}  // namespace

extern "C" int proteus_geo_attn_num_variants(void) { return kNumVariants; }

extern "C" const char* proteus_geo_attn_variant_name(int tuning) {
    return (tuning >= 0 && tuning < kNumVariants) ? kVariants[tuning].name : nullptr;
}

extern "C" int proteus_geo_attn_fwd_check(const uint16_t* Q, const uint16_t* K, const uint16_t* V,
                                          const float* coords, const float* sigma,
                                          const uint8_t* key_pad_mask,
                                          const float* O, const float* L,
                                          int Z, int H, int N, int d_head, int tuning)
{
    (void)key_pad_mask; (void)L;
    if (!Q || !K || !V || !coords || !sigma || !O) return PROTEUS_ERR_NULL_POINTER;
    if (Z <= 0 || H <= 0 || N <= 0) return PROTEUS_ERR_BAD_SHAPE;
    if (N > PROTEUS_ATTN_MAX_N || (long)Z * H > 65535) return PROTEUS_ERR_BAD_SHAPE;
    if (d_head != GA_D) return PROTEUS_ERR_BAD_HEAD_DIM;
    if (tuning < 0 || tuning >= kNumVariants) return PROTEUS_ERR_BAD_TUNING;
    if (((uintptr_t)Q & 15) || ((uintptr_t)K & 15) || ((uintptr_t)V & 15) || ((uintptr_t)O & 15)) return PROTEUS_ERR_BAD_ALIGNMENT;
    return PROTEUS_OK;
}

extern "C" int proteus_geo_attn_fwd(const uint16_t* Q, const uint16_t* K, const uint16_t* V,
                                    const float* coords, const float* sigma,
                                    const uint8_t* key_pad_mask,
                                    float* O, float* L,
                                    int Z, int H, int N, int d_head, int tuning, void* stream)
{
    const int rc = proteus_geo_attn_fwd_check(Q, K, V, coords, sigma, key_pad_mask, O, L, Z, H, N, d_head, tuning);
    if (rc != PROTEUS_OK) return rc;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    dim3 grid((N + GA_BM - 1) / GA_BM, Z * H, 1);
    hipLaunchKernelGGL(geo_attn_fwd_kernel, grid, dim3(GA_THREADS), 0, st,
                       Q, K, V, coords, sigma, key_pad_mask, O, L, H, N);
    return (int)hipGetLastError();
}
