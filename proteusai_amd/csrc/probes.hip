// Instruction-rate and accuracy probes (not on the product path): they state, from measurement, the denominators
// the WE roofline model uses, the error of the hardware sin/cos/rsq path, and how far one matrix product and the
// softmax work that goes with it overlap on a SIMD (the issue model of the attention kernel).

#include <hip/hip_runtime.h>
#include <stdint.h>
#include "proteus_hip.h"      // return codes
#include "proteus_probes.h"

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

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float  floatx16 __attribute__((ext_vector_type(16)));
typedef float  floatx2 __attribute__((ext_vector_type(2)));

// One "slot" of the attention forward's inner loop: a 32x32x16 bf16 matrix product and the softmax work of two scores
// (two fused multiply-adds, two exp2, one pack to bf16, one packed row-sum add).  MODE 0: the products only;
// 1: the vector work only; 2: both, in the order the kernel issues them.  Eight slots per loop trip.
// VEC picks the vector work of a slot: 0 the softmax work; 1 twelve ordinary fused multiply-adds (about as long);
// 2 four exp2 and nothing else.  The two last ones tell which kind of vector instruction runs beside a product.
template <int MODE, int VEC>
__global__ __launch_bounds__(256)
void mfma_softmax_slot_kernel(float* sink, int iters) {
    floatx16 acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.f;
    bf16x8 a, b;
#pragma unroll
    for (int e = 0; e < 8; ++e) { a[e] = (__bf16)(0.001f * (float)(threadIdx.x + e)); b[e] = (__bf16)(0.002f * (float)(e + 1)); }
    float s0 = 0.001f * (float)threadIdx.x, s1 = 0.5f - s0, lsum = 0.f;
    float log2e = 1.4426950408889634f, mneg = -0.25f;
    asm volatile("" : "+v"(log2e), "+v"(mneg));
#pragma unroll 1
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            if (MODE != 1) acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc, 0, 0, 0);
            if (MODE != 0) {
                asm volatile("" : "+v"(s0), "+v"(s1));          // opaque: nothing of the step is hoisted out of the loop
                if (VEC == 1) {
#pragma unroll
                    for (int q = 0; q < 6; ++q) { s0 = __builtin_fmaf(s0, log2e, mneg); s1 = __builtin_fmaf(s1, log2e, mneg); }
                    __builtin_amdgcn_sched_barrier(0);
                    continue;
                }
                if (VEC == 2) {
                    const float y0 = __builtin_amdgcn_exp2f(s0), y1 = __builtin_amdgcn_exp2f(s1);
                    const float y2 = __builtin_amdgcn_exp2f(mneg), y3 = __builtin_amdgcn_exp2f(log2e);
                    asm volatile("" :: "v"(y0), "v"(y1), "v"(y2), "v"(y3));
                    __builtin_amdgcn_sched_barrier(0);
                    continue;
                }
                const float x0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s0, log2e, mneg));
                const float x1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s1, log2e, mneg));
                const floatx2 f = {x0, x1};
                const bf16x2 pk = __builtin_convertvector(f, bf16x2);
                lsum = __builtin_amdgcn_fdot2_f32_bf16(pk, __builtin_bit_cast(bf16x2, 0x3f803f80u), lsum, false);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    float s = lsum + s0 + s1;
#pragma unroll
    for (int r = 0; r < 16; ++r) s += acc[r];
    sink[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = s;
}

// Do transcendental and ordinary vector instructions of DIFFERENT waves of one SIMD overlap?  One workgroup of
// 4 * WPS waves per compute unit (its LDS request keeps a second one away), WPS waves on every SIMD.  Each wave reads
// the SIMD it runs on from the hardware-id register and draws a ticket among the waves of its workgroup on that SIMD:
// the first `k_trans` tickets run `iters_trans` links of 64 independent v_sin_f32 chains, the others `iters_valu`
// links of 64 independent v_fmac_f32 chains with vector-register operands only.  census[workgroup * 4 + simd] receives
// (waves seen << 16) | waves that took the transcendental role, so the host can check the placement it relies on.
__global__ __launch_bounds__(1024)
void trans_valu_mix_kernel(float* sink, unsigned* census, int k_trans, int iters_trans, int iters_valu, float a, float b) {
    extern __shared__ unsigned mix_lds[];            // [0..3]: tickets per SIMD, [4..7]: transcendental waves per SIMD
    if (threadIdx.x < 8) mix_lds[threadIdx.x] = 0u;
    __syncthreads();
    // HW_REG_HW_ID (register 4), bits 5:4 = SIMD_ID
    const unsigned simd = __builtin_amdgcn_s_getreg((1 << 11) | (4 << 6) | 4) & 3u;
    unsigned ticket = 0;
    if ((threadIdx.x & 63) == 0) ticket = atomicAdd(&mix_lds[simd], 1u);
    ticket = (unsigned)__builtin_amdgcn_readfirstlane((int)ticket);
    const bool trans = (int)ticket < k_trans;
    if (trans && (threadIdx.x & 63) == 0) atomicAdd(&mix_lds[4 + simd], 1u);
    float x[64];
#pragma unroll
    for (int c = 0; c < 64; ++c) x[c] = 0.001f * (float)((threadIdx.x & 63) + c) + 0.25f;
    float u = 1e-3f * (a + 1e-9f * (float)threadIdx.x), v = b + 1e-12f * (float)threadIdx.x;
    if (trans) {
#pragma unroll 1
        for (int it = 0; it < iters_trans; ++it) {
#pragma unroll
            for (int c = 0; c < 64; ++c) x[c] = __builtin_amdgcn_sinf(x[c]);
        }
    } else {
#pragma unroll 1
        for (int it = 0; it < iters_valu; ++it) {
#pragma unroll
            for (int c = 0; c < 64; ++c) x[c] = __builtin_fmaf(u, v, x[c]);
            asm volatile("" : "+v"(u), "+v"(v));
        }
    }
    float s = 0.f;
#pragma unroll
    for (int c = 0; c < 64; ++c) s += x[c];
    sink[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = s;
    __syncthreads();
    if (threadIdx.x < 4) census[blockIdx.x * 4 + threadIdx.x] = (mix_lds[threadIdx.x] << 16) | mix_lds[4 + threadIdx.x];
}

}  // namespace

extern "C" int proteus_probe_trans_valu_mix(int waves_per_simd, int k_trans, int blocks, int iters_trans, int iters_valu,
                                            float* sink, unsigned* census, void* stream) {
    if (!sink || !census) return PROTEUS_ERR_NULL_POINTER;
    if (blocks <= 0 || blocks > (1 << 20) || iters_trans < 0 || iters_valu < 0) return PROTEUS_ERR_BAD_SHAPE;
    if (waves_per_simd < 1 || waves_per_simd > 4 || k_trans < 0 || k_trans > waves_per_simd) return PROTEUS_ERR_BAD_TUNING;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    // 96 KB of LDS per workgroup: one workgroup per compute unit (160 KB each)
    static bool allowed = false;
    if (!allowed) {
        const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(trans_valu_mix_kernel),
                                                    hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024);
        if (attr != hipSuccess) return (int)attr;
        allowed = true;
    }
    hipLaunchKernelGGL(trans_valu_mix_kernel, dim3(blocks), dim3(256 * waves_per_simd), 96 * 1024, st,
                       sink, census, k_trans, iters_trans, iters_valu, 0.999999f, 1e-7f);
    return (int)hipGetLastError();
}

extern "C" int proteus_probe_mfma_softmax_slot(int mode, int blocks, int iters, float* sink, void* stream) {
    if (!sink) return PROTEUS_ERR_NULL_POINTER;
    if (blocks <= 0 || iters <= 0 || blocks > (1 << 20)) return PROTEUS_ERR_BAD_SHAPE;
    if (mode < 0 || mode > 6) return PROTEUS_ERR_BAD_TUNING;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
#define PROTEUS_SLOT(M_, V_) hipLaunchKernelGGL((mfma_softmax_slot_kernel<M_, V_>), dim3(blocks), dim3(256), 0, st, sink, iters)
    switch (mode) {
        case 0: PROTEUS_SLOT(0, 0); break;
        case 1: PROTEUS_SLOT(1, 0); break;
        case 2: PROTEUS_SLOT(2, 0); break;
        case 3: PROTEUS_SLOT(1, 1); break;
        case 4: PROTEUS_SLOT(2, 1); break;
        case 5: PROTEUS_SLOT(1, 2); break;
        default: PROTEUS_SLOT(2, 2); break;
    }
#undef PROTEUS_SLOT
    return (int)hipGetLastError();
}

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
