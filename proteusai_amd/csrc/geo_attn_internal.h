// What the translation units of the attention kernels share: stride records and the per-head-dimension launchers
// (one translation unit per head dimension keeps the compile parallel).  Nothing here is part of the C ABI.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace proteus_internal {

// Element strides (batch, head, token) of Q, K, V (16-bit) and O (f32); the head dimension is contiguous.
struct GaStrides { long q[3], k[3], v[3], o[3]; };
// ... of Q, K, V, dO (16-bit) and dQ, dK, dV (f32)
struct GbStrides { long q[3], k[3], v[3], g[3], dq[3], dk[3], dv[3]; };

#define PROTEUS_HIDDEN __attribute__((visibility("hidden")))

// forward, head dimension 32 / 128 (64 lives with the ABI): legacy = the reference kernel's logits (beta, rbf range),
// f16 = fp16 operands.  Returns a hipError_t as int.
PROTEUS_HIDDEN int attn_fwd_d32(bool legacy, bool f16, const uint16_t* Q, const uint16_t* K, const uint16_t* V, const float* coords,
                                const float* sigma, const uint8_t* key_pad_mask, float* O, float* L, int Z, int H, int N, int tuning,
                                const float* beta, float min_rbf, float max_rbf, const GaStrides& gs, hipStream_t st);
PROTEUS_HIDDEN int attn_fwd_d128(bool legacy, bool f16, const uint16_t* Q, const uint16_t* K, const uint16_t* V, const float* coords,
                                 const float* sigma, const uint8_t* key_pad_mask, float* O, float* L, int Z, int H, int N, int tuning,
                                 const float* beta, float min_rbf, float max_rbf, const GaStrides& gs, hipStream_t st);

// backward, head dimension 32 / 128
PROTEUS_HIDDEN int attn_bwd_d32(bool legacy, bool f16, const uint16_t* Q, const uint16_t* K, const uint16_t* V, const uint16_t* dO,
                                const float* coords, const float* sigma, const float* beta, const uint8_t* mask,
                                const float* L, const float* D, float* dQ, float* dK, float* dV, float* d_sigma, float* d_beta,
                                int Z, int H, int N, float min_rbf, float max_rbf, const GbStrides& gs, hipStream_t st);
PROTEUS_HIDDEN int attn_bwd_d128(bool legacy, bool f16, const uint16_t* Q, const uint16_t* K, const uint16_t* V, const uint16_t* dO,
                                 const float* coords, const float* sigma, const float* beta, const uint8_t* mask,
                                 const float* L, const float* D, float* dQ, float* dK, float* dV, float* d_sigma, float* d_beta,
                                 int Z, int H, int N, float min_rbf, float max_rbf, const GbStrides& gs, hipStream_t st);

}  // namespace proteus_internal
