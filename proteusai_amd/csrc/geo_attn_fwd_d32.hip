// Geometric attention forward, head dimension 32: the instantiations of the templated body (see geo_attn_fwd.hip for
// what the kernel computes and how it maps to the machine).
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>
#include "proteus_hip.h"
#include "geo_attn_ops.h"
#include "geo_attn_internal.h"

namespace {
#include "geo_attn_fwd_body.inc"
}  // namespace

int proteus_internal::attn_fwd_d32(bool legacy, bool f16, const uint16_t* Q, const uint16_t* K, const uint16_t* V, const float* coords,
                                   const float* sigma, const uint8_t* key_pad_mask, float* O, float* L, int Z, int H, int N, int tuning,
                                   const float* beta, float min_rbf, float max_rbf, const GaStrides& gs, hipStream_t st)
{
    return launch_attn_dh<32>(legacy, f16, Q, K, V, coords, sigma, key_pad_mask, O, L, Z, H, N, tuning, beta, min_rbf, max_rbf, gs, st);
}
