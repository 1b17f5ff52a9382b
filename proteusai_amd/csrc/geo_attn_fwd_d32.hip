// Geometric attention forward, head dimension 32: the instantiations of the templated body and of the software-pipelined
// one (see geo_attn_fwd.hip for what the kernels compute and how they map to the machine).
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>
#include "proteus_hip.h"
#include "geo_attn_ops.h"
#include "geo_attn_internal.h"

namespace {
#include "geo_attn_fwd_body.inc"
#include "geo_attn_fwd_pipe.inc"

int launch_attn_pipe_d32(const uint16_t* Q, const uint16_t* K, const uint16_t* V, const float* coords, const float* sigma,
                         const uint8_t* key_pad_mask, float* O, float* L, int Z, int H, int N, bool take_all,
                         const GaStrides& gs, hipStream_t st)
{
    constexpr int BM = GA_WAVES * 64;
    const int n_qtiles = (N + BM - 1) / BM;
    const int ZH = Z * H;
    const unsigned n_wgs = (unsigned)n_qtiles * (unsigned)ZH;
    hipLaunchKernelGGL(geo_attn_fwd_pipe_kernel<32>, dim3(take_all ? n_wgs : 2 * n_wgs), dim3(GA_THREADS), ga_pipe_lds<32>(), st,
                       Q, K, V, coords, sigma, key_pad_mask, O, L, H, N, ZH, n_qtiles, (int)n_wgs, take_all ? 1 : 0, gs);
    return (int)hipGetLastError();
}
}  // namespace

int proteus_internal::attn_fwd_d32(bool legacy, bool f16, const uint16_t* Q, const uint16_t* K, const uint16_t* V, const float* coords,
                                   const float* sigma, const uint8_t* key_pad_mask, float* O, float* L, int Z, int H, int N, int tuning,
                                   const float* beta, float min_rbf, float max_rbf, const GaStrides& gs, hipStream_t st)
{
    // tuning 5 / 6: the software-pipelined kernel (6: without the direct-distance workgroups); 0 takes it by the rule of
    // d = 64 (see launch_attn): above 384 workgroups of 256 queries, from N = 1024 on, short ragged batches excepted
    const long wgs2 = (long)((N + GA_WAVES * 64 - 1) / (GA_WAVES * 64)) * Z * H;
    const bool small_ragged = key_pad_mask != nullptr && N <= 1024 && wgs2 <= 1024;
    if (!legacy && (tuning == 5 || tuning == 6 || (tuning == 0 && wgs2 > 384 && N >= 1024 && !small_ragged)))
        return launch_attn_pipe_d32(Q, K, V, coords, sigma, key_pad_mask, O, L, Z, H, N, tuning == 6, gs, st);
    return launch_attn_dh<32>(legacy, f16, Q, K, V, coords, sigma, key_pad_mask, O, L, Z, H, N, (tuning == 5 || tuning == 6) ? 4 : tuning,
                              beta, min_rbf, max_rbf, gs, st);
}
