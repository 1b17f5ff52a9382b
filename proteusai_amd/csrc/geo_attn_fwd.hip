// RBF-scaled geometric flash-attention forward for gfx950 (MI355X), d_head = 32, 64 or 128 (this file: 64 and the C ABI).
//
// What it computes (README.md:40 logits on the flash structure of
// old/old_scripts/attn/geometric_attn.py:57-260):
//   s_ij = (q_i . k_j)/sqrt(d) * (1 + exp(-|r_i - r_j|^2 / (2 sigma_h^2))),  -inf for padded keys
//   O_i  = softmax_j(s_ij) V_j,  L_i = logsumexp_j s_ij;  padded/empty rows -> O = 0, L = -inf
//
// Mapping to the machine.  A workgroup is 4 waves; a wave owns 64 queries of one
// (batch, head) as two blocks of 32 (one block where the grid would otherwise leave
// half of the wave slots empty) and walks the keys in tiles of 64 that the
// workgroup stages in LDS (K row-major, V transposed, key geometry), two tiles
// deep: tile t is consumed while tile t+1 travels global -> registers -> LDS.
// All products run on the matrix cores and are computed TRANSPOSED:
//   S^T (keys x queries)  = K_tile (A, from LDS) x Q^T (B, registers, loaded once)
//   D^T (keys x queries)  = G_tile (A, from LDS) x G_q^T (B, registers)     [geometry, see below]
//   O^T (d x queries)    += V^T_tile (A, from LDS) x P^T (B, registers)
// In the 32x32 accumulator layout a lane holds 16 rows of ONE column, so with
// queries on the columns each lane owns one query per block: the exponentials
// and the row sum are in-lane (the two half-waves of a query meet only when its
// softmax reference is re-based and at the end), and the S^T accumulator registers are, after conversion
// to bf16, already the B operand of the last product (the contraction index is
// merely visited in the permuted order the accumulator layout dictates, and the
// V^T operand is read from LDS in that same order).  Every A fragment read from
// LDS serves both query blocks.  The softmax keeps a lazy reference instead of a
// running maximum, and for blocks whose multiplier is 1 that reference is carried
// into the score product as one more contraction slot (see the key loop).
//
// Geometry on the matrix cores.  With x' = (x - c) * sqrt(log2(e)/2)/sigma_h (c = a
// point near the workgroup's queries) the multiplier is 1 + exp2(D),
//   D = -|x'_k - x'_q|^2 = -|x'_k|^2 + 2 x'_k . x'_q - |x'_q|^2 .
// Every fp32 scalar is split exactly into three bf16 pieces (8+8+8 mantissa
// bits), and D becomes a 24-term bf16 contraction whose products are exact in
// the fp32 accumulator: per coordinate the pieces hh, hm, mh, mm, hl, lh (the
// dropped ml, lm, ll are below 2^-24 of the product), plus the two squared
// norms against ones.  One 32x32x16 and one 32x32x8 MFMA per 32 keys replace six
// vector-ALU instructions per score.  The cancellation error is about
// 2^-20 (|x'_k|^2 + |x'_q|^2); it only matters where the multiplier differs from
// 1, i.e. for keys within ~6 sigma of the query, so with the origin near the
// queries it is below 3e-3 in D as long as the workgroup's queries lie within
// GA_MFMA_DIST_MAX_RHO2 of that origin.  A workgroup whose queries are spread
// wider evaluates the distances directly on the vector ALU instead.
// Nothing of size N x N exists anywhere.


#include <hip/hip_runtime.h>
#include <atomic>
#include <stdint.h>
#include <type_traits>
#include "proteus_hip.h"
#include "geo_attn_ops.h"
#include "geo_attn_internal.h"

namespace {

#include "geo_attn_fwd_body.inc"
#include "geo_attn_fwd_pipe.inc"

// The pipelined body over the first half of a doubled grid, the direct-distance body (for workgroups whose
// queries are spread too widely for the matrix-core distances) over the second; take_all: the pipelined body alone.
__global__ __launch_bounds__(GA_THREADS, 2)
void geo_attn_fwd_pipe_kernel(const uint16_t* __restrict__ Q, const uint16_t* __restrict__ K,
                              const uint16_t* __restrict__ V, const float* __restrict__ coords,
                              const float* __restrict__ sigma, const uint8_t* __restrict__ key_pad,
                              float* __restrict__ O, float* __restrict__ L,
                              const int H, const int N, const int ZH, const int n_qtiles, const int n_wgs, const int take_all,
                              const GaStrides st)
{
    extern __shared__ __align__(16) unsigned char ga_dyn_smem[];
    const int id = (int)blockIdx.x;
    if (id < n_wgs)
        geo_attn_fwd_pipe_body(*reinterpret_cast<PipeSmem*>(ga_dyn_smem), id, Q, K, V, coords, sigma, key_pad, O, L,
                               H, N, ZH, n_qtiles, take_all, st);
    else
        geo_attn_fwd_body<true, false, 2>(*reinterpret_cast<Smem*>(ga_dyn_smem), id - n_wgs, Q, K, V, coords, sigma, key_pad, O, L,
                                          H, N, ZH, n_qtiles, 0, nullptr, 0.f, 1.f, st);
}
constexpr size_t GA_PIPE_LDS = sizeof(PipeSmem) > sizeof(Smem) ? sizeof(PipeSmem) : sizeof(Smem);
static_assert(GA_PIPE_LDS <= 80 * 1024, "two workgroups per compute unit");

struct GaVariant { const char* name; };
const GaVariant kVariants[] = { {"auto"}, {"dist_mfma"}, {"dist_valu"}, {"one_block_per_wave"}, {"two_blocks_per_wave"},
                                {"pipelined"}, {"pipelined_dist_mfma"}, {"split_keys"} };
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
    if (d_head != 32 && d_head != 64 && d_head != 128) return PROTEUS_ERR_BAD_HEAD_DIM;
    if (tuning < 0 || tuning >= kNumVariants) return PROTEUS_ERR_BAD_TUNING;
    if (((uintptr_t)Q & 15) || ((uintptr_t)K & 15) || ((uintptr_t)V & 15) || ((uintptr_t)O & 15)) return PROTEUS_ERR_BAD_ALIGNMENT;
    return PROTEUS_OK;
}

namespace {
int launch_attn_pipe(const uint16_t* Q, const uint16_t* K, const uint16_t* V, const float* coords, const float* sigma,
                     const uint8_t* key_pad_mask, float* O, float* L, int Z, int H, int N, bool take_all,
                     const GaStrides& gs, hipStream_t st)
{
    // more than 64 KB of dynamic LDS must be allowed once per device (remembered for the first 64 devices)
    static std::atomic<unsigned long long> allowed{0ull};
    int dev = 0;
    const hipError_t got = hipGetDevice(&dev);
    if (got != hipSuccess) return (int)got;
    if (dev < 0 || dev >= 64 || !((allowed.load(std::memory_order_relaxed) >> dev) & 1ull)) {
        const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(geo_attn_fwd_pipe_kernel),
                                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)GA_PIPE_LDS);
        if (attr != hipSuccess) return (int)attr;
        if (dev >= 0 && dev < 64) allowed.fetch_or(1ull << dev, std::memory_order_relaxed);
    }
    constexpr int BM = GA_WAVES * 64;
    const int n_qtiles = (N + BM - 1) / BM;
    const int ZH = Z * H;
    const unsigned n_wgs = (unsigned)n_qtiles * (unsigned)ZH;
    hipLaunchKernelGGL(geo_attn_fwd_pipe_kernel, dim3(take_all ? n_wgs : 2 * n_wgs), dim3(GA_THREADS), GA_PIPE_LDS, st,
                       Q, K, V, coords, sigma, key_pad_mask, O, L, H, N, ZH, n_qtiles, (int)n_wgs, take_all ? 1 : 0, gs);
    return (int)hipGetLastError();
}

// d_head and operand type to the kernels.  With two query blocks per wave, d = 64, bf16 operands and the README logits
// the software-pipelined kernel runs (automatically for large grids of long sequences, or when the tuning asks).
int launch_attn(bool legacy, bool f16, int d_head, const uint16_t* Q, const uint16_t* K, const uint16_t* V, const float* coords,
                const float* sigma, const uint8_t* key_pad_mask, float* O, float* L, int Z, int H, int N, int tuning,
                const float* beta, float min_rbf, float max_rbf, const GaStrides& gs, hipStream_t st)
{
    if (d_head == 32)
        return proteus_internal::attn_fwd_d32(legacy, f16, Q, K, V, coords, sigma, key_pad_mask, O, L, Z, H, N, (tuning == 5 || tuning == 6) ? 0 : tuning,
                                              beta, min_rbf, max_rbf, gs, st);
    if (d_head == 128)
        return proteus_internal::attn_fwd_d128(legacy, f16, Q, K, V, coords, sigma, key_pad_mask, O, L, Z, H, N, (tuning == 5 || tuning == 6) ? 0 : tuning,
                                               beta, min_rbf, max_rbf, gs, st);
    // The pipelined kernel pays a longer prologue back from about 16 key tiles per workgroup on, and only where its
    // 256-query workgroups fill the chip twice: measured against the templated body it wins from 512 workgroups and
    // N = 1024 on (3-11 %), loses below (7-9 % at 256 workgroups of N = 1024, 6-10 % at N = 256 and 512).  A batch that
    // comes with a padding mask is taken to be ragged: up to N = 1024 such a batch runs 12-17 % faster on the body's
    // 128-query workgroups (twice as many, half as long: they even out), so it goes there.
    const long wgs2 = (long)((N + GA_WAVES * 64 - 1) / (GA_WAVES * 64)) * Z * H;
    const bool small_ragged = key_pad_mask != nullptr && N <= 1024 && wgs2 <= 1024;
    if (!legacy && (tuning == 5 || tuning == 6 || (tuning == 0 && wgs2 >= 512 && N >= 1024 && !small_ragged)))
        return launch_attn_pipe(Q, K, V, coords, sigma, key_pad_mask, O, L, Z, H, N, tuning == 6, gs, st);
    return launch_attn_dh<64>(legacy, f16, Q, K, V, coords, sigma, key_pad_mask, O, L, Z, H, N, (tuning == 5 || tuning == 6) ? 4 : tuning,
                              beta, min_rbf, max_rbf, gs, st);
}
// contiguous [Z,H,N,d] tensors
GaStrides contiguous_strides(int H, int N, int d) {
    GaStrides gs;
    const long t[3] = {(long)H * N * d, (long)N * d, (long)d};
    for (int i = 0; i < 3; ++i) { gs.q[i] = t[i]; gs.k[i] = t[i]; gs.v[i] = t[i]; gs.o[i] = t[i]; }
    return gs;
}

// strides[12]: (batch, head, token) element strides of Q, K, V, O in this order
int strides_from(const int64_t* strides, int Z, int H, int N, int d, GaStrides& gs) {
    if (!strides) return PROTEUS_ERR_NULL_POINTER;
    long* dst[4] = {gs.q, gs.k, gs.v, gs.o};
    for (int t = 0; t < 4; ++t) {
        const int64_t sz = strides[3 * t], sh = strides[3 * t + 1], sn = strides[3 * t + 2];
        // rows of d contiguous elements that do not overlap and stay 16-byte aligned; a sequence's byte
        // offsets fit the 31 bits of a buffer-load offset
        if (sz < 0 || sh < 0 || sn < d) return PROTEUS_ERR_BAD_LAYOUT;
        const int align = (t == 3) ? 4 : 8;
        if ((sz % align) || (sh % align) || (sn % align)) return PROTEUS_ERR_BAD_ALIGNMENT;
        if ((Z > 1 && sz == 0) || (H > 1 && sh == 0)) return PROTEUS_ERR_BAD_LAYOUT;
        if ((long)N * sn * (t == 3 ? 4 : 2) >= (1L << 31)) return PROTEUS_ERR_BAD_SHAPE;
        dst[t][0] = (long)sz; dst[t][1] = (long)sh; dst[t][2] = (long)sn;
    }
    return PROTEUS_OK;
}
}  // namespace

extern "C" int proteus_geo_attn_fwd_strided_check(const uint16_t* Q, const uint16_t* K, const uint16_t* V,
                                                  const int64_t* strides,
                                                  const float* coords, const float* sigma, const uint8_t* key_pad_mask,
                                                  const float* O, const float* L,
                                                  int Z, int H, int N, int d_head, int tuning)
{
    const int rc = proteus_geo_attn_fwd_check(Q, K, V, coords, sigma, key_pad_mask, O, L, Z, H, N, d_head, tuning);
    if (rc != PROTEUS_OK) return rc;
    GaStrides gs;
    return strides_from(strides, Z, H, N, d_head, gs);
}

extern "C" int proteus_geo_attn_fwd_strided(const uint16_t* Q, const uint16_t* K, const uint16_t* V,
                                            const int64_t* strides,
                                            const float* coords, const float* sigma, const uint8_t* key_pad_mask,
                                            float* O, float* L,
                                            int Z, int H, int N, int d_head, int tuning, void* stream)
{
    int rc = proteus_geo_attn_fwd_check(Q, K, V, coords, sigma, key_pad_mask, O, L, Z, H, N, d_head, tuning);
    if (rc != PROTEUS_OK) return rc;
    GaStrides gs;
    rc = strides_from(strides, Z, H, N, d_head, gs);
    if (rc != PROTEUS_OK) return rc;
    return launch_attn(false, false, d_head, Q, K, V, coords, sigma, key_pad_mask, O, L, Z, H, N, tuning, nullptr, 0.f, 1.f, gs,
                       reinterpret_cast<hipStream_t>(stream));
}

extern "C" int proteus_geo_attn_fwd(const uint16_t* Q, const uint16_t* K, const uint16_t* V,
                                    const float* coords, const float* sigma,
                                    const uint8_t* key_pad_mask,
                                    float* O, float* L,
                                    int Z, int H, int N, int d_head, int tuning, void* stream)
{
    const int rc = proteus_geo_attn_fwd_check(Q, K, V, coords, sigma, key_pad_mask, O, L, Z, H, N, d_head, tuning);
    if (rc != PROTEUS_OK) return rc;
    return launch_attn(false, false, d_head, Q, K, V, coords, sigma, key_pad_mask, O, L, Z, H, N, tuning, nullptr, 0.f, 1.f,
                       contiguous_strides(H, N, d_head), reinterpret_cast<hipStream_t>(stream));
}

namespace {
int legacy_args_check(const float* beta, float min_rbf, float max_rbf, int operand_type) {
    if (!beta) return PROTEUS_ERR_NULL_POINTER;
    if (!(max_rbf > min_rbf)) return PROTEUS_ERR_BAD_SHAPE;
    if (operand_type != PROTEUS_OPERAND_BF16 && operand_type != PROTEUS_OPERAND_F16) return PROTEUS_ERR_BAD_OPERAND_TYPE;
    return PROTEUS_OK;
}
}  // namespace

extern "C" int proteus_geo_attn_legacy_fwd(const uint16_t* Q, const uint16_t* K, const uint16_t* V,
                                           const float* coords, const float* sigma, const float* beta,
                                           const uint8_t* key_pad_mask,
                                           float* O, float* L,
                                           int Z, int H, int N, int d_head,
                                           float min_rbf, float max_rbf, int operand_type, int tuning, void* stream)
{
    int rc = proteus_geo_attn_fwd_check(Q, K, V, coords, sigma, key_pad_mask, O, L, Z, H, N, d_head, tuning);
    if (rc != PROTEUS_OK) return rc;
    rc = legacy_args_check(beta, min_rbf, max_rbf, operand_type);
    if (rc != PROTEUS_OK) return rc;
    // a pair mask makes the result sensitive to the last bits of the rbf: use direct distances then
    if ((tuning == 0 || tuning >= 3) && (min_rbf > 0.f || max_rbf < 1.f)) tuning = 2;
    return launch_attn(true, operand_type == PROTEUS_OPERAND_F16, d_head, Q, K, V, coords, sigma, key_pad_mask, O, L, Z, H, N, tuning,
                       beta, min_rbf, max_rbf, contiguous_strides(H, N, d_head), reinterpret_cast<hipStream_t>(stream));
}

extern "C" int proteus_geo_attn_legacy_fwd_strided(const uint16_t* Q, const uint16_t* K, const uint16_t* V,
                                                   const int64_t* strides,
                                                   const float* coords, const float* sigma, const float* beta,
                                                   const uint8_t* key_pad_mask,
                                                   float* O, float* L,
                                                   int Z, int H, int N, int d_head,
                                                   float min_rbf, float max_rbf, int operand_type, int tuning, void* stream)
{
    int rc = proteus_geo_attn_fwd_check(Q, K, V, coords, sigma, key_pad_mask, O, L, Z, H, N, d_head, tuning);
    if (rc != PROTEUS_OK) return rc;
    rc = legacy_args_check(beta, min_rbf, max_rbf, operand_type);
    if (rc != PROTEUS_OK) return rc;
    GaStrides gs;
    rc = strides_from(strides, Z, H, N, d_head, gs);
    if (rc != PROTEUS_OK) return rc;
    if ((tuning == 0 || tuning >= 3) && (min_rbf > 0.f || max_rbf < 1.f)) tuning = 2;
    return launch_attn(true, operand_type == PROTEUS_OPERAND_F16, d_head, Q, K, V, coords, sigma, key_pad_mask, O, L, Z, H, N, tuning,
                       beta, min_rbf, max_rbf, gs, reinterpret_cast<hipStream_t>(stream));
}
