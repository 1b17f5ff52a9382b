// Geometric attention backward, head dimension 128: the instantiations of the templated body (see geo_attn_bwd.hip for
// what the kernel computes and how it maps to the machine).
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>
#include "proteus_hip.h"
#include "geo_attn_ops.h"
#include "geo_attn_internal.h"

namespace {
#include "geo_attn_bwd_body.inc"
}  // namespace

int proteus_internal::attn_bwd_d128(bool legacy, bool f16, const uint16_t* Q, const uint16_t* K, const uint16_t* V, const uint16_t* dO,
                                    const float* coords, const float* sigma, const float* beta, const uint8_t* mask,
                                    const float* L, const float* D, float* dQ, float* dK, float* dV, float* d_sigma, float* d_beta,
                                    int Z, int H, int N, float min_rbf, float max_rbf, const GbStrides& gs, hipStream_t st)
{
    return launch_bwd_dh<128>(legacy, f16, Q, K, V, dO, coords, sigma, beta, mask, L, D, dQ, dK, dV, d_sigma, d_beta,
                              Z, H, N, min_rbf, max_rbf, gs, st);
}
