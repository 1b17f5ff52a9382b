// RBF-scaled geometric attention backward for gfx950 (MI355X): dQ, dK, dV, d sigma (and d beta); d_head = 32, 64 or 128
// (this file: 64 and the C ABI).
//
// What it computes (reference: old/old_scripts/attn/geometric_attn.py:262-543, wrapper :609-660), with
// S = q.k/sqrt(d), rbf = exp(-|r_i - r_j|^2/(2 sigma_h^2)) and the logits t(S, rbf) of the forward kernel:
//     P    = exp(t - L_i)                 (L: the forward's logsumexp; 0 for a masked pair)      :453
//     dV_j = sum_i P_ij dO_i                                                                      :459
//     dP   = dO_i . V_j ;  dt = P (dP - D_i),  D_i = sum_d O_id dO_id                             :462-465
//     dS   = dt * dt/dS ;  dQ_i = sum_j dS_ij K_j / sqrt(d) ;  dK_j = sum_i dS_ij Q_i / sqrt(d)   :468,500-505
//     d sigma_h = sum dt * dt/drbf * rbf * |r_i - r_j|^2 / sigma_h^3                              :473,494-497
//   README logits  t = S (1 + rbf):             dt/dS = 1 + rbf,              dt/drbf = S
//   LEGACY logits  t = S + beta Rn |S|, Rn = 2 (rbf - min)/(max - min) - 1   (:448-449):
//                  dt/dS = 1 + beta Rn sign(S), dt/drbf = 2 beta |S|/(max - min), d beta_h = sum dt Rn |S|  (:468-479)
//
// Two passes instead of the reference's one kernel with atomic adds into dQ (:501-503), run by the two
// halves of one launch:
//   OWN_Q = false  a wave owns 32 keys, streams the queries, accumulates dK, dV (and d sigma, d beta);
//   OWN_Q = true   a wave owns 32 queries, streams the keys, accumulates dQ.
// Both are the same code.  Scores are computed with the rows of the streamed ("other") tokens in the
// accumulator rows and the wave's own token in the accumulator column (lane % 32), so a lane owns one own
// token: S = other . own^T and dP likewise on v_mfma_f32_32x32x16_bf16 with the own side held in registers
// as the B operand for the whole kernel.  P and dS are, after bf16 conversion, directly the B operands of
// the accumulating products (dV^T += dO^T P, dK^T += Q^T dS; dQ^T += K^T dS) whose A operands are the
// streamed tiles transposed, read in the accumulator's row order: the tiles travel global -> LDS directly
// and are transposed by the LDS read (ds_read_b64_tr_b16).  No atomics except the one per-wave add into
// d sigma / d beta; dQ, dK, dV are deterministic.

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>
#include "proteus_hip.h"
#include "geo_attn_ops.h"
#include "geo_attn_internal.h"

namespace {

#include "geo_attn_bwd_body.inc"

int launch_bwd_any(bool legacy, bool f16, int d_head, const uint16_t* Q, const uint16_t* K, const uint16_t* V, const uint16_t* dO,
                   const float* coords, const float* sigma, const float* beta, const uint8_t* mask,
                   const float* L, const float* D, float* dQ, float* dK, float* dV, float* d_sigma, float* d_beta,
                   int Z, int H, int N, float min_rbf, float max_rbf, const GbStrides& gs, hipStream_t st)
{
    if (d_head == 32)
        return proteus_internal::attn_bwd_d32(legacy, f16, Q, K, V, dO, coords, sigma, beta, mask, L, D, dQ, dK, dV, d_sigma, d_beta,
                                              Z, H, N, min_rbf, max_rbf, gs, st);
    if (d_head == 128)
        return proteus_internal::attn_bwd_d128(legacy, f16, Q, K, V, dO, coords, sigma, beta, mask, L, D, dQ, dK, dV, d_sigma, d_beta,
                                               Z, H, N, min_rbf, max_rbf, gs, st);
    return launch_bwd_dh<64>(legacy, f16, Q, K, V, dO, coords, sigma, beta, mask, L, D, dQ, dK, dV, d_sigma, d_beta,
                             Z, H, N, min_rbf, max_rbf, gs, st);
}

GbStrides contiguous_strides(int H, int N, int d) {
    GbStrides gs;
    const long t[3] = {(long)H * N * d, (long)N * d, (long)d};
    long* all[7] = {gs.q, gs.k, gs.v, gs.g, gs.dq, gs.dk, gs.dv};
    for (int a = 0; a < 7; ++a) for (int i = 0; i < 3; ++i) all[a][i] = t[i];
    return gs;
}

// strides[21]: (batch, head, token) element strides of Q, K, V, dO, dQ, dK, dV in this order
int strides_from(const int64_t* strides, int Z, int H, int N, int d, GbStrides& gs) {
    if (!strides) return PROTEUS_ERR_NULL_POINTER;
    long* dst[7] = {gs.q, gs.k, gs.v, gs.g, gs.dq, gs.dk, gs.dv};
    for (int t = 0; t < 7; ++t) {
        const int64_t sz = strides[3 * t], sh = strides[3 * t + 1], sn = strides[3 * t + 2];
        if (sz < 0 || sh < 0 || sn < d) return PROTEUS_ERR_BAD_LAYOUT;
        const int align = (t >= 4) ? 4 : 8;            // 16-byte rows: f32 outputs, bf16 inputs
        if ((sz % align) || (sh % align) || (sn % align)) return PROTEUS_ERR_BAD_ALIGNMENT;
        if ((Z > 1 && sz == 0) || (H > 1 && sh == 0)) return PROTEUS_ERR_BAD_LAYOUT;
        if ((long)N * sn >= (1L << 30)) return PROTEUS_ERR_BAD_SHAPE;
        dst[t][0] = (long)sz; dst[t][1] = (long)sh; dst[t][2] = (long)sn;
    }
    return PROTEUS_OK;
}

}  // namespace

extern "C" int proteus_geo_attn_bwd_check(const uint16_t* Q, const uint16_t* K, const uint16_t* V, const uint16_t* dO,
                                          const float* coords, const float* sigma, const float* beta,
                                          const uint8_t* key_pad_mask, const float* L, const float* D,
                                          const float* dQ, const float* dK, const float* dV,
                                          const float* d_sigma, const float* d_beta,
                                          int Z, int H, int N, int d_head, float min_rbf, float max_rbf, int operand_type)
{
    (void)key_pad_mask; (void)d_sigma; (void)d_beta;
    if (!Q || !K || !V || !dO || !coords || !sigma || !L || !D || !dQ || !dK || !dV) return PROTEUS_ERR_NULL_POINTER;
    if (Z <= 0 || H <= 0 || N <= 0) return PROTEUS_ERR_BAD_SHAPE;
    if (N > PROTEUS_ATTN_MAX_N || (long)Z * H > 65535) return PROTEUS_ERR_BAD_SHAPE;
    if (d_head != 32 && d_head != 64 && d_head != 128) return PROTEUS_ERR_BAD_HEAD_DIM;
    if (beta && !(max_rbf > min_rbf)) return PROTEUS_ERR_BAD_SHAPE;
    // fp16 operands go with the reference kernel's logits only
    if (operand_type != PROTEUS_OPERAND_BF16 && !(operand_type == PROTEUS_OPERAND_F16 && beta)) return PROTEUS_ERR_BAD_OPERAND_TYPE;
    if (((uintptr_t)Q & 15) || ((uintptr_t)K & 15) || ((uintptr_t)V & 15) || ((uintptr_t)dO & 15) ||
        ((uintptr_t)dQ & 15) || ((uintptr_t)dK & 15) || ((uintptr_t)dV & 15)) return PROTEUS_ERR_BAD_ALIGNMENT;
    return PROTEUS_OK;
}

extern "C" int proteus_geo_attn_bwd(const uint16_t* Q, const uint16_t* K, const uint16_t* V, const uint16_t* dO,
                                    const float* coords, const float* sigma, const float* beta,
                                    const uint8_t* key_pad_mask, const float* L, const float* D,
                                    float* dQ, float* dK, float* dV, float* d_sigma, float* d_beta,
                                    int Z, int H, int N, int d_head, float min_rbf, float max_rbf, int operand_type, void* stream)
{
    const int rc = proteus_geo_attn_bwd_check(Q, K, V, dO, coords, sigma, beta, key_pad_mask, L, D, dQ, dK, dV,
                                              d_sigma, d_beta, Z, H, N, d_head, min_rbf, max_rbf, operand_type);
    if (rc != PROTEUS_OK) return rc;
    return launch_bwd_any(beta != nullptr, operand_type == PROTEUS_OPERAND_F16, d_head, Q, K, V, dO, coords, sigma, beta, key_pad_mask,
                          L, D, dQ, dK, dV, d_sigma, d_beta, Z, H, N, min_rbf, max_rbf, contiguous_strides(H, N, d_head),
                          reinterpret_cast<hipStream_t>(stream));
}

extern "C" int proteus_geo_attn_bwd_strided_check(const uint16_t* Q, const uint16_t* K, const uint16_t* V, const uint16_t* dO,
                                                  const int64_t* strides,
                                                  const float* coords, const float* sigma, const float* beta,
                                                  const uint8_t* key_pad_mask, const float* L, const float* D,
                                                  const float* dQ, const float* dK, const float* dV,
                                                  const float* d_sigma, const float* d_beta,
                                                  int Z, int H, int N, int d_head, float min_rbf, float max_rbf, int operand_type)
{
    const int rc = proteus_geo_attn_bwd_check(Q, K, V, dO, coords, sigma, beta, key_pad_mask, L, D, dQ, dK, dV,
                                              d_sigma, d_beta, Z, H, N, d_head, min_rbf, max_rbf, operand_type);
    if (rc != PROTEUS_OK) return rc;
    GbStrides gs;
    return strides_from(strides, Z, H, N, d_head, gs);
}

extern "C" int proteus_geo_attn_bwd_strided(const uint16_t* Q, const uint16_t* K, const uint16_t* V, const uint16_t* dO,
                                            const int64_t* strides,
                                            const float* coords, const float* sigma, const float* beta,
                                            const uint8_t* key_pad_mask, const float* L, const float* D,
                                            float* dQ, float* dK, float* dV, float* d_sigma, float* d_beta,
                                            int Z, int H, int N, int d_head, float min_rbf, float max_rbf, int operand_type, void* stream)
{
    int rc = proteus_geo_attn_bwd_check(Q, K, V, dO, coords, sigma, beta, key_pad_mask, L, D, dQ, dK, dV,
                                        d_sigma, d_beta, Z, H, N, d_head, min_rbf, max_rbf, operand_type);
    if (rc != PROTEUS_OK) return rc;
    GbStrides gs;
    rc = strides_from(strides, Z, H, N, d_head, gs);
    if (rc != PROTEUS_OK) return rc;
    return launch_bwd_any(beta != nullptr, operand_type == PROTEUS_OPERAND_F16, d_head, Q, K, V, dO, coords, sigma, beta, key_pad_mask,
                          L, D, dQ, dK, dV, d_sigma, d_beta, Z, H, N, min_rbf, max_rbf, gs, reinterpret_cast<hipStream_t>(stream));
}
