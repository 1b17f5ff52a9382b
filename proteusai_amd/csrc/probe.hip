// Instruction-rate and accuracy probes (not on the product path): they state, from measurement, the denominators
// the WE roofline model uses and the error of the hardware sin/cos/rsq path.

#include <hip/hip_runtime.h>
#include <stdint.h>
#include "proteus_hip.h"

namespace {

template <int OP>
__device__ __forceinline__ float step(float x, float a, float b) {
    if (OP == 0) return __builtin_fmaf(x, a, b);
    if (OP == 1) return x * a;
    if (OP == 2) return x + b;
    if (OP == 3) return __builtin_amdgcn_sinf(x);
    if (OP == 4) return __builtin_amdgcn_cosf(x);
    if (OP == 5) return __builtin_amdgcn_exp2f(x);
    if (OP == 6) return __builtin_amdgcn_rsqf(x);
    return __builtin_amdgcn_fractf(x);
}

// 64 independent dependency chains per lane, `iters` links each.
template <int OP>
__global__ __launch_bounds__(256)
void valu_rate_kernel(float* sink, int iters, float a, float b) {
    float x[64];
#pragma unroll
    for (int c = 0; c < 64; ++c) x[c] = 0.001f * (float)(threadIdx.x + c) + 0.25f;
#pragma unroll 1
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int c = 0; c < 64; ++c) x[c] = step<OP>(x[c], a, b);
    }
    float s = 0.f;
#pragma unroll
    for (int c = 0; c < 64; ++c) s += x[c];
    sink[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = s;
}

// 64 independent accumulations per lane and link with VECTOR operands only (the rate kernels above feed
// the scalars a and b): FORM 0: x = fma(x, u, v); 1: x = fma(u, v, x) (v_fmac_f32); 2: x += u; 3: x *= u.
template <int FORM>
__global__ __launch_bounds__(256)
void valu_vector_operand_kernel(float* sink, int iters, float a, float b) {
    float x[64];
#pragma unroll
    for (int c = 0; c < 64; ++c) x[c] = 0.001f * (float)(threadIdx.x + c) + 0.25f;
    float u = a + 1e-9f * (float)threadIdx.x, v = b + 1e-12f * (float)threadIdx.x;
    if (FORM == 1) { u = 1e-3f * u; }
    if (FORM == 2) { u = v; }
#pragma unroll 1
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int c = 0; c < 64; ++c) {
            if (FORM == 0) x[c] = __builtin_fmaf(x[c], u, v);
            if (FORM == 1) x[c] = __builtin_fmaf(u, v, x[c]);
            if (FORM == 2) x[c] += u;
            if (FORM == 3) x[c] *= u;
        }
        asm volatile("" : "+v"(u), "+v"(v));      // keeps u and v in vector registers, opaque to the optimiser
    }
    float s = 0.f;
#pragma unroll
    for (int c = 0; c < 64; ++c) s += x[c];
    sink[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = s;
}

__global__ void sincos_probe_kernel(const float* x, float* s, float* c, float* q, int n, int use_fract) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float v  = x[i];
    const float ph = use_fract ? __builtin_amdgcn_fractf(v) : v;
    s[i] = __builtin_amdgcn_sinf(ph);
    c[i] = __builtin_amdgcn_cosf(ph);
    const float r2 = v;
    const bool  ok = r2 != 0.0f;
    const float inv = ok ? __builtin_amdgcn_rsqf(r2) : 0.0f;
    const float r0 = r2 * inv;
    const float e  = __builtin_fmaf(-r0, r0, r2);
    q[i] = __builtin_fmaf(e, 0.5f * inv, r0);
}

}  // namespace

extern "C" int proteus_probe_valu_rate(int op, int blocks, int iters, float* sink, void* stream) {
    if (!sink) return PROTEUS_ERR_NULL_POINTER;
    if (blocks <= 0 || iters <= 0 || blocks > (1 << 20)) return PROTEUS_ERR_BAD_SHAPE;
    if (op < 0 || op > 9) return PROTEUS_ERR_BAD_TUNING;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    // a, b chosen so that the chains stay finite and are not constant-folded
    const float a = 0.999999f, b = 1e-7f;
#define GO(OP_) hipLaunchKernelGGL((valu_rate_kernel<OP_>), dim3(blocks), dim3(256), 0, st, sink, iters, a, b)
    switch (op) {
        case 8: hipLaunchKernelGGL((valu_vector_operand_kernel<1>), dim3(blocks), dim3(256), 0, st, sink, iters, a, b); break;
        case 9: hipLaunchKernelGGL((valu_vector_operand_kernel<2>), dim3(blocks), dim3(256), 0, st, sink, iters, a, b); break;
        case 0: GO(0); break; case 1: GO(1); break; case 2: GO(2); break; case 3: GO(3); break;
        case 4: GO(4); break; case 5: GO(5); break; case 6: GO(6); break; default: GO(7); break;
    }
#undef GO
    return (int)hipGetLastError();
}

extern "C" int proteus_probe_sincos(const float* x, float* s, float* c, float* q, int n, int use_fract, void* stream) {
    if (!x || !s || !c || !q) return PROTEUS_ERR_NULL_POINTER;
    if (n <= 0) return PROTEUS_ERR_BAD_SHAPE;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(sincos_probe_kernel, dim3((n + 255) / 256), dim3(256), 0, st, x, s, c, q, n, use_fract);
    return (int)hipGetLastError();
}
