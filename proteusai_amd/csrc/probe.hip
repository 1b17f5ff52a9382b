// Instruction-rate and accuracy probes (not on the product path): they state,
// from measurement, the denominators the WE roofline model uses and the error
// of the hardware sin/cos/rsq path.  Also home of the error-code text.

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

// NT chains of v_sin_f32 and NF chains of v_fma_f32 per lane in one instruction stream: tells whether
// the transcendental and the ordinary fp32 pipelines of a SIMD overlap, within a wave or across waves.
template <int NT, int NF>
__global__ __launch_bounds__(256)
void valu_mix_kernel(float* sink, int iters, float a, float b) {
    float x[NT], y[NF];
#pragma unroll
    for (int c = 0; c < NT; ++c) x[c] = 0.001f * (float)(threadIdx.x + c) + 0.25f;
#pragma unroll
    for (int c = 0; c < NF; ++c) y[c] = 0.002f * (float)(threadIdx.x + c) + 0.5f;
#pragma unroll 1
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int c = 0; c < (NT > NF ? NT : NF); ++c) {
            if (c < NT) x[c] = __builtin_amdgcn_sinf(x[c]);
#pragma unroll
            for (int f = c * NF / NT; f < (c + 1) * NF / NT && c < NT; ++f) y[f] = __builtin_fmaf(y[f], a, b);
        }
    }
    float s = 0.f;
#pragma unroll
    for (int c = 0; c < NT; ++c) s += x[c];
#pragma unroll
    for (int c = 0; c < NF; ++c) s += y[c];
    sink[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = s;
}

// Whole waves of one kind: the first four waves of a 512-thread workgroup run v_sin_f32 chains, the
// last four v_fma_f32 chains, so that a SIMD holds waves of both kinds: do the two pipelines overlap
// ACROSS waves?
__global__ __launch_bounds__(512)
void valu_split_mix_kernel(float* sink, int iters, float a, float b) {
    float x[64];
#pragma unroll
    for (int c = 0; c < 64; ++c) x[c] = 0.001f * (float)(threadIdx.x + c) + 0.25f;
    if (threadIdx.x >= 256) {
        float u = 1e-3f * a + 1e-9f * (float)threadIdx.x, v = b + 1e-12f * (float)threadIdx.x;
#pragma unroll 1
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int c = 0; c < 64; ++c) x[c] = __builtin_fmaf(u, v, x[c]);      // v_fmac_f32, vector operands
            asm volatile("" : "+v"(u), "+v"(v));
        }
    } else {
#pragma unroll 1
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int c = 0; c < 64; ++c) x[c] = __builtin_amdgcn_sinf(x[c]);
        }
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

// 64 chains of v_mul_f32 whose first source goes through DPP (quad broadcast of one lane of a vector
// register): a way to feed a wave-uniform factor without a scalar-register operand.
__global__ __launch_bounds__(256)
void valu_dpp_mul_kernel(float* sink, int iters, float a, float b) {
    float x[64];
#pragma unroll
    for (int c = 0; c < 64; ++c) x[c] = 0.001f * (float)(threadIdx.x + c) + 0.25f;
    float u = a + 1e-9f * (float)(threadIdx.x & 3) + b;
#pragma unroll 1
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int c = 0; c < 64; c += 4) {
            asm volatile("v_mul_f32_dpp %0, %1, %0 quad_perm:[0,0,0,0] row_mask:0xf bank_mask:0xf" : "+v"(x[c]) : "v"(u));
            asm volatile("v_mul_f32_dpp %0, %1, %0 quad_perm:[1,1,1,1] row_mask:0xf bank_mask:0xf" : "+v"(x[c + 1]) : "v"(u));
            asm volatile("v_mul_f32_dpp %0, %1, %0 quad_perm:[2,2,2,2] row_mask:0xf bank_mask:0xf" : "+v"(x[c + 2]) : "v"(u));
            asm volatile("v_mul_f32_dpp %0, %1, %0 quad_perm:[3,3,3,3] row_mask:0xf bank_mask:0xf" : "+v"(x[c + 3]) : "v"(u));
        }
    }
    float s = 0.f;
#pragma unroll
    for (int c = 0; c < 64; ++c) s += x[c];
    sink[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = s;
}

// The embedding kernel's inner step on register data: per wavenumber one v_mul_f32 with a scalar operand,
// (TRANS: v_sin_f32 + v_cos_f32, else two more v_mul_f32), two v_fmac_f32 and two v_add_f32 on vector
// operands, KT wavenumbers per step.  Instructions issued per lane and step: 7*KT.
template <int KT, bool TRANS>
__global__ __launch_bounds__(256)
void valu_we_step_kernel(float* sink, int iters, float a, float b) {
    float kr[KT], s1[KT], s2[KT], s3[KT], s4[KT];
#pragma unroll
    for (int t = 0; t < KT; ++t) {
        kr[t] = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, a * (float)(t + 1) * 0.01f)));
        s1[t] = 0.f; s2[t] = 0.f; s3[t] = 0.f; s4[t] = 0.f;
    }
    float r = 1.0f + 0.01f * (float)threadIdx.x, inv = 1.0f / r;
#pragma unroll 1
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int t = 0; t < KT; ++t) {
            const float ph = r * kr[t];
            const float s = TRANS ? __builtin_amdgcn_sinf(ph) : ph * inv;
            const float c = TRANS ? __builtin_amdgcn_cosf(ph) : ph * r;
            s1[t] = __builtin_fmaf(c, inv, s1[t]);
            s2[t] = __builtin_fmaf(s, inv, s2[t]);
            s3[t] += c;
            s4[t] += s;
        }
        r += b;
        inv -= b;
    }
    float acc = 0.f;
#pragma unroll
    for (int t = 0; t < KT; ++t) acc += s1[t] + s2[t] + s3[t] + s4[t];
    sink[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = acc;
}

// Matrix-core accumulation beside the transcendental pipeline.  MODE 0: 16 independent
// v_mfma_f32_4x4x1_16B_f32 accumulators per lane and link; 1: 16 v_sin_f32 chains; 2: both in one
// instruction stream, one v_sin_f32 after each MFMA; 3: waves 0-3 of a 512-thread workgroup run the
// MFMAs, waves 4-7 the v_sin_f32 chains.
typedef float f32x4 __attribute__((ext_vector_type(4)));
template <int MODE>
__global__ __launch_bounds__(512)
void mfma_sin_mix_kernel(float* sink, int iters, float a, float b) {
    f32x4 d[16];
    float x[16];
#pragma unroll
    for (int c = 0; c < 16; ++c) { d[c] = f32x4{0.f, 0.f, 0.f, 0.f}; x[c] = 0.001f * (float)(threadIdx.x + c) + 0.25f; }
    float u = 1e-3f * a + 1e-9f * (float)threadIdx.x, v = b + 1e-12f * (float)threadIdx.x;
    const bool do_mfma = MODE == 0 || MODE == 2 || (MODE == 3 && threadIdx.x < 256);
    const bool do_sin  = MODE == 1 || MODE == 2 || (MODE == 3 && threadIdx.x >= 256);
#pragma unroll 1
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int c = 0; c < 16; ++c) {
            if (do_mfma) d[c] = __builtin_amdgcn_mfma_f32_4x4x1f32(u, v, d[c], 0, 0, 0);
            if (do_sin)  x[c] = __builtin_amdgcn_sinf(x[c]);
        }
        asm volatile("" : "+v"(u), "+v"(v));
    }
    float s = 0.f;
#pragma unroll
    for (int c = 0; c < 16; ++c) s += x[c] + d[c][0] + d[c][1] + d[c][2] + d[c][3];
    sink[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = s;
}

// The attention kernel's matrix instruction beside ordinary vector work.  Per link: MODE 0: four independent
// v_mfma_f32_32x32x16_bf16; 1: 32 v_fmac_f32 on vector operands; 2: both in one instruction stream (eight
// v_fmac_f32 after each MFMA); 3: as 2 with v_exp_f32 chains in place of the v_fmac_f32.
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
template <int MODE>
__global__ __launch_bounds__(256)
void mfma_valu_mix_kernel(float* sink, int iters, float a, float b) {
    f32x16 d[4];
    float x[32];
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
        for (int e = 0; e < 16; ++e) d[c][e] = 0.f;
#pragma unroll
    for (int c = 0; c < 32; ++c) x[c] = 0.001f * (float)(threadIdx.x + c) + 0.25f;
    float u = 1e-3f * a + 1e-9f * (float)threadIdx.x, v = b + 1e-12f * (float)threadIdx.x;
    bf16x8_t pa, pb;
#pragma unroll
    for (int e = 0; e < 8; ++e) { pa[e] = (__bf16)(0.01f * (float)(threadIdx.x & 7)); pb[e] = (__bf16)(0.02f * (float)e); }
#pragma unroll 1
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            if (MODE != 1) d[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(pa, pb, d[c], 0, 0, 0);
#pragma unroll
            for (int f = 0; f < 8; ++f) {
                if (MODE == 1 || MODE == 2) x[8 * c + f] = __builtin_fmaf(u, v, x[8 * c + f]);
                if (MODE == 3) x[8 * c + f] = __builtin_amdgcn_exp2f(x[8 * c + f]);
            }
        }
        asm volatile("" : "+v"(u), "+v"(v));
    }
    float s = 0.f;
#pragma unroll
    for (int c = 0; c < 32; ++c) s += x[c];
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
        for (int e = 0; e < 16; ++e) s += d[c][e];
    sink[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = s;
}

// Matrix and vector work in DIFFERENT waves of one SIMD: workgroups of 8 waves, waves 0-3 run
// v_mfma_f32_32x32x16_bf16 only (MODE 0 and 2), waves 4-7 alternate 8 v_exp_f32 with 8 v_fmac_f32 on vector
// operands (MODE 1 and 2).  Per link: 4 MFMAs in the one kind of wave, 16 + 16 vector instructions in the other.
template <int MODE>
__global__ __launch_bounds__(512)
void mfma_cross_wave_kernel(float* sink, int iters, float a, float b) {
    float s = 0.f;
    if (threadIdx.x < 256) {
        if (MODE == 1) return;
        f32x16 d[4];
#pragma unroll
        for (int c = 0; c < 4; ++c)
#pragma unroll
            for (int e = 0; e < 16; ++e) d[c][e] = 0.f;
        bf16x8_t pa, pb;
#pragma unroll
        for (int e = 0; e < 8; ++e) { pa[e] = (__bf16)(0.01f * (float)(threadIdx.x & 7)); pb[e] = (__bf16)(0.02f * (float)e); }
#pragma unroll 1
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int c = 0; c < 4; ++c) d[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(pa, pb, d[c], 0, 0, 0);
        }
#pragma unroll
        for (int c = 0; c < 4; ++c)
#pragma unroll
            for (int e = 0; e < 16; ++e) s += d[c][e];
    } else {
        if (MODE == 0) return;
        float x[16], y[16];
#pragma unroll
        for (int c = 0; c < 16; ++c) { x[c] = 0.001f * (float)(threadIdx.x + c) - 0.75f; y[c] = 0.5f + 0.01f * (float)c; }
        float u = 1e-3f * a + 1e-9f * (float)threadIdx.x, v = b + 1e-12f * (float)threadIdx.x;
#pragma unroll 1
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
#pragma unroll
                for (int c = 0; c < 8; ++c) x[8 * h + c] = __builtin_amdgcn_exp2f(x[8 * h + c] - 1.0f);
#pragma unroll
                for (int c = 0; c < 8; ++c) y[8 * h + c] = __builtin_fmaf(u, v, y[8 * h + c]);
            }
            asm volatile("" : "+v"(u), "+v"(v));
        }
#pragma unroll
        for (int c = 0; c < 16; ++c) s += x[c] + y[c];
    }
    sink[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = s;
}

// The same mix in a fixed program order: every v_sin_f32 is followed by NF_PER ordinary instructions
// before the next one (the compiler, left alone, tends to group the transcendentals).
template <int NF_PER>
__global__ __launch_bounds__(256)
void valu_ordered_mix_kernel(float* sink, int iters, float a, float b) {
    float x[16], y[16 * NF_PER];
    float u = 1e-3f * a + 1e-9f * (float)threadIdx.x, v = b + 1e-12f * (float)threadIdx.x;
#pragma unroll
    for (int c = 0; c < 16; ++c) x[c] = 0.001f * (float)(threadIdx.x + c) + 0.25f;
#pragma unroll
    for (int c = 0; c < 16 * NF_PER; ++c) y[c] = 0.002f * (float)(threadIdx.x + c) + 0.5f;
#pragma unroll 1
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int c = 0; c < 16; ++c) {
            asm volatile("v_sin_f32 %0, %0" : "+v"(x[c]));
#pragma unroll
            for (int f = 0; f < NF_PER; ++f)
                asm volatile("v_fmac_f32 %0, %1, %2" : "+v"(y[c * NF_PER + f]) : "v"(u), "v"(v));
        }
    }
    float s = 0.f;
#pragma unroll
    for (int c = 0; c < 16; ++c) s += x[c];
#pragma unroll
    for (int c = 0; c < 16 * NF_PER; ++c) s += y[c];
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

extern "C" int proteus_version(void) { return 100; }

extern "C" const char* proteus_strerror(int code) {
    switch (code) {
        case PROTEUS_OK:                return "ok";
        case PROTEUS_ERR_NULL_POINTER:  return "a required pointer is NULL";
        case PROTEUS_ERR_BAD_SHAPE:     return "a dimension is not positive or exceeds the supported maximum";
        case PROTEUS_ERR_BAD_HEAD_DIM:  return "d_head must be 64";
        case PROTEUS_ERR_BAD_LAYOUT:    return "unknown coords_layout";
        case PROTEUS_ERR_BAD_ALIGNMENT: return "a pointer is not 16-byte aligned";
        case PROTEUS_ERR_BAD_TUNING:    return "unknown tuning selector";
        case PROTEUS_ERR_UNSUPPORTED:   return "option not implemented";
        case PROTEUS_ERR_TOO_LARGE:     return "size beyond the fixed capacity of this entry point";
        default: break;
    }
    if (code > 0) return hipGetErrorString((hipError_t)code);
    return "unknown error code";
}

extern "C" int proteus_probe_valu_rate(int op, int blocks, int iters, float* sink, void* stream) {
    if (!sink) return PROTEUS_ERR_NULL_POINTER;
    if (blocks <= 0 || iters <= 0 || blocks > (1 << 20)) return PROTEUS_ERR_BAD_SHAPE;
    if (op < 0 || op > 34) return PROTEUS_ERR_BAD_TUNING;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    // a, b chosen so that the chains stay finite and are not constant-folded
    const float a = 0.999999f, b = 1e-7f;
#define GO(OP_) hipLaunchKernelGGL((valu_rate_kernel<OP_>), dim3(blocks), dim3(256), 0, st, sink, iters, a, b)
#define MIX(NT_, NF_) hipLaunchKernelGGL((valu_mix_kernel<NT_, NF_>), dim3(blocks), dim3(256), 0, st, sink, iters, a, b)
    switch (op) {
        case 34: hipLaunchKernelGGL(valu_dpp_mul_kernel, dim3(blocks), dim3(256), 0, st, sink, iters, a, b); break;
        case 31: hipLaunchKernelGGL((mfma_cross_wave_kernel<0>), dim3((blocks + 1) / 2), dim3(512), 0, st, sink, iters, a, b); break;
        case 32: hipLaunchKernelGGL((mfma_cross_wave_kernel<1>), dim3((blocks + 1) / 2), dim3(512), 0, st, sink, iters, a, b); break;
        case 33: hipLaunchKernelGGL((mfma_cross_wave_kernel<2>), dim3((blocks + 1) / 2), dim3(512), 0, st, sink, iters, a, b); break;
        case 27: hipLaunchKernelGGL((mfma_valu_mix_kernel<0>), dim3(blocks), dim3(256), 0, st, sink, iters, a, b); break;
        case 28: hipLaunchKernelGGL((mfma_valu_mix_kernel<1>), dim3(blocks), dim3(256), 0, st, sink, iters, a, b); break;
        case 29: hipLaunchKernelGGL((mfma_valu_mix_kernel<2>), dim3(blocks), dim3(256), 0, st, sink, iters, a, b); break;
        case 30: hipLaunchKernelGGL((mfma_valu_mix_kernel<3>), dim3(blocks), dim3(256), 0, st, sink, iters, a, b); break;
        case 23: hipLaunchKernelGGL((mfma_sin_mix_kernel<0>), dim3((blocks + 1) / 2), dim3(512), 0, st, sink, iters, a, b); break;
        case 24: hipLaunchKernelGGL((mfma_sin_mix_kernel<1>), dim3((blocks + 1) / 2), dim3(512), 0, st, sink, iters, a, b); break;
        case 25: hipLaunchKernelGGL((mfma_sin_mix_kernel<2>), dim3((blocks + 1) / 2), dim3(512), 0, st, sink, iters, a, b); break;
        case 26: hipLaunchKernelGGL((mfma_sin_mix_kernel<3>), dim3((blocks + 1) / 2), dim3(512), 0, st, sink, iters, a, b); break;
        case 19: hipLaunchKernelGGL((valu_vector_operand_kernel<0>), dim3(blocks), dim3(256), 0, st, sink, iters, a, b); break;
        case 20: hipLaunchKernelGGL((valu_vector_operand_kernel<1>), dim3(blocks), dim3(256), 0, st, sink, iters, a, b); break;
        case 21: hipLaunchKernelGGL((valu_vector_operand_kernel<2>), dim3(blocks), dim3(256), 0, st, sink, iters, a, b); break;
        case 22: hipLaunchKernelGGL((valu_vector_operand_kernel<3>), dim3(blocks), dim3(256), 0, st, sink, iters, a, b); break;
        case 15: hipLaunchKernelGGL((valu_we_step_kernel<8, true>), dim3(blocks), dim3(256), 0, st, sink, iters, a, b); break;
        case 16: hipLaunchKernelGGL((valu_we_step_kernel<8, false>), dim3(blocks), dim3(256), 0, st, sink, iters, a, b); break;
        case 17: hipLaunchKernelGGL((valu_we_step_kernel<32, true>), dim3(blocks), dim3(256), 0, st, sink, iters, a, b); break;
        case 18: hipLaunchKernelGGL((valu_we_step_kernel<32, false>), dim3(blocks), dim3(256), 0, st, sink, iters, a, b); break;
        case 14: hipLaunchKernelGGL(valu_split_mix_kernel, dim3((blocks + 1) / 2), dim3(512), 0, st, sink, iters, a, b); break;
        case 11: hipLaunchKernelGGL((valu_ordered_mix_kernel<1>), dim3(blocks), dim3(256), 0, st, sink, iters, a, b); break;
        case 12: hipLaunchKernelGGL((valu_ordered_mix_kernel<2>), dim3(blocks), dim3(256), 0, st, sink, iters, a, b); break;
        case 13: hipLaunchKernelGGL((valu_ordered_mix_kernel<3>), dim3(blocks), dim3(256), 0, st, sink, iters, a, b); break;
        case 8: MIX(16, 16); break; case 9: MIX(16, 32); break; case 10: MIX(16, 48); break;
        case 0: GO(0); break; case 1: GO(1); break; case 2: GO(2); break; case 3: GO(3); break;
        case 4: GO(4); break; case 5: GO(5); break; case 6: GO(6); break; default: GO(7); break;
    }
#undef GO
#undef MIX
    return (int)hipGetLastError();
}

extern "C" int proteus_probe_sincos(const float* x, float* s, float* c, float* q, int n, int use_fract, void* stream) {
    if (!x || !s || !c || !q) return PROTEUS_ERR_NULL_POINTER;
    if (n <= 0) return PROTEUS_ERR_BAD_SHAPE;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(sincos_probe_kernel, dim3((n + 255) / 256), dim3(256), 0, st, x, s, c, q, n, use_fract);
    return (int)hipGetLastError();
}
