// Residual add + LayerNorm of the post-LN encoder layer for gfx950 (inference forward).
//
// What it computes: out = LayerNorm(x + res) * gamma + beta over the last dimension, i.e. the two lines
//   q = self.attn_norm(q + self.dropout(self.attn(...)))  and  q = self.ffn_norm(q + self.dropout(self.ffn(q)))
// of old/old_scripts/encoder.py:36-39 with dropout inactive, as torch evaluates them: the sum is rounded to the
// tensors' type first (a bf16 sum is a bf16 tensor), mean and biased variance are taken in fp32, eps is added under
// the square root, and the result is rounded to the tensors' type.
//
// Pure streaming work, bound by HBM: 3 x sizeof(T) bytes per element.  A wave owns a row; every lane moves 16 bytes
// per chunk of the row and keeps its share of the row in registers, so x and res are read once; the two reductions
// (sum, then sum of squared deviations: the two-pass variance) run over the wave with cross-lane shuffles.

#include <hip/hip_runtime.h>
#include <stdint.h>
#include "proteus_hip.h"

namespace {

constexpr int AL_WAVES  = 4;            // rows per workgroup
constexpr int AL_MAX_CH = 8;            // 16-byte chunks per lane and row

__device__ __forceinline__ float bf16_to_f32(const uint16_t h) { return __builtin_bit_cast(float, (uint32_t)h << 16); }
// round to nearest even; NaN stays NaN
__device__ __forceinline__ uint16_t f32_to_bf16(const float f) {
    const uint32_t u = __builtin_bit_cast(uint32_t, f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}

template <typename T> struct Elem;
template <> struct Elem<float> {
    static constexpr int VEC = 4;
    static __device__ __forceinline__ void load(const float* p, float (&v)[4]) {
        const float4 t = *reinterpret_cast<const float4*>(p);
        v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
    }
    static __device__ __forceinline__ void store(float* p, const float (&v)[4]) {
        *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
    }
    static __device__ __forceinline__ float round(const float v) { return v; }
};
template <> struct Elem<uint16_t> {          // bf16
    static constexpr int VEC = 8;
    static __device__ __forceinline__ void load(const uint16_t* p, float (&v)[8]) {
        const uint4 t = *reinterpret_cast<const uint4*>(p);
        const uint32_t w[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            v[2 * e]     = __builtin_bit_cast(float, w[e] << 16);
            v[2 * e + 1] = __builtin_bit_cast(float, w[e] & 0xffff0000u);
        }
    }
    static __device__ __forceinline__ void store(uint16_t* p, const float (&v)[8]) {
        uint32_t w[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) w[e] = (uint32_t)f32_to_bf16(v[2 * e]) | ((uint32_t)f32_to_bf16(v[2 * e + 1]) << 16);
        *reinterpret_cast<uint4*>(p) = make_uint4(w[0], w[1], w[2], w[3]);
    }
    static __device__ __forceinline__ float round(const float v) { return bf16_to_f32(f32_to_bf16(v)); }
};

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    return v;
}

// CH = chunks of 64 * VEC elements that cover a row (the last one may be partial; D is a multiple of VEC)
template <typename T, int CH>
__global__ __launch_bounds__(AL_WAVES * 64)
void add_layernorm_kernel(const T* x, const T* res, const T* __restrict__ gamma, const T* __restrict__ beta,
                          T* out, const long rows, const int D, const float eps)
{
    constexpr int VEC = Elem<T>::VEC;
    const int lane = threadIdx.x & 63;
    const long row = (long)blockIdx.x * AL_WAVES + (threadIdx.x >> 6);
    if (row >= rows) return;                       // (whole waves leave: no barrier follows)
    const T* xr = x + (size_t)row * D;
    const T* rr = res ? res + (size_t)row * D : nullptr;
    float y[CH][VEC];
    float sum = 0.f;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int e0 = (c * 64 + lane) * VEC;
        if (e0 < D) {
            Elem<T>::load(xr + e0, y[c]);
            if (rr) {
                float r[VEC];
                Elem<T>::load(rr + e0, r);
#pragma unroll
                for (int e = 0; e < VEC; ++e) y[c][e] = Elem<T>::round(y[c][e] + r[e]);
            }
#pragma unroll
            for (int e = 0; e < VEC; ++e) sum += y[c][e];
        } else {
#pragma unroll
            for (int e = 0; e < VEC; ++e) y[c][e] = 0.f;
        }
    }
    const float mean = wave_sum(sum) / (float)D;
    float sq = 0.f;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int e0 = (c * 64 + lane) * VEC;
        if (e0 < D) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) { const float dlt = y[c][e] - mean; sq = __builtin_fmaf(dlt, dlt, sq); }
        }
    }
    const float rstd = 1.0f / __builtin_sqrtf(wave_sum(sq) / (float)D + eps);
    T* orow = out + (size_t)row * D;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int e0 = (c * 64 + lane) * VEC;
        if (e0 < D) {
            float g[VEC], b[VEC], o[VEC];
            if (gamma) Elem<T>::load(gamma + e0, g);
            if (beta)  Elem<T>::load(beta + e0, b);
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                const float n = (y[c][e] - mean) * rstd;
                o[e] = gamma ? (beta ? __builtin_fmaf(n, g[e], b[e]) : n * g[e]) : (beta ? n + b[e] : n);
            }
            Elem<T>::store(orow + e0, o);
        }
    }
}

template <typename T>
int launch(const void* x, const void* res, const void* gamma, const void* beta, void* out,
           const long rows, const int D, const float eps, hipStream_t st)
{
    constexpr int VEC = Elem<T>::VEC;
    const int ch = (D + 64 * VEC - 1) / (64 * VEC);
    const dim3 grid((unsigned)((rows + AL_WAVES - 1) / AL_WAVES)), block(AL_WAVES * 64);
#define AL_GO(CH_) hipLaunchKernelGGL((add_layernorm_kernel<T, CH_>), grid, block, 0, st, (const T*)x, (const T*)res, \
                                      (const T*)gamma, (const T*)beta, (T*)out, rows, D, eps)
    switch (ch) {
        case 1: AL_GO(1); break;
        case 2: AL_GO(2); break;
        case 3: case 4: AL_GO(4); break;
        default: AL_GO(8); break;
    }
#undef AL_GO
    return (int)hipGetLastError();
}

}  // namespace

extern "C" int proteus_add_layernorm_fwd_check(const void* x, const void* res, const void* gamma, const void* beta, const void* out,
                                               long rows, int D, float eps, int dtype)
{
    if (!x || !out) return PROTEUS_ERR_NULL_POINTER;
    if (dtype != PROTEUS_DTYPE_F32 && dtype != PROTEUS_DTYPE_BF16) return PROTEUS_ERR_BAD_OPERAND_TYPE;
    const int vec = dtype == PROTEUS_DTYPE_F32 ? 4 : 8;
    if (rows <= 0 || D <= 0 || rows > ((1L << 31) - 1) * AL_WAVES) return PROTEUS_ERR_BAD_SHAPE;      // grid.x below 2^31
    if (D % vec != 0 || D > 64 * vec * AL_MAX_CH) return PROTEUS_ERR_BAD_SHAPE;
    if (!(eps >= 0.0f)) return PROTEUS_ERR_BAD_SHAPE;
    const uintptr_t all = (uintptr_t)x | (uintptr_t)res | (uintptr_t)gamma | (uintptr_t)beta | (uintptr_t)out;
    if (all & 15) return PROTEUS_ERR_BAD_ALIGNMENT;
    return PROTEUS_OK;
}

extern "C" int proteus_add_layernorm_fwd(const void* x, const void* res, const void* gamma, const void* beta, void* out,
                                         long rows, int D, float eps, int dtype, void* stream)
{
    const int rc = proteus_add_layernorm_fwd_check(x, res, gamma, beta, out, rows, D, eps, dtype);
    if (rc != PROTEUS_OK) return rc;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    return dtype == PROTEUS_DTYPE_F32 ? launch<float>(x, res, gamma, beta, out, rows, D, eps, st)
                                      : launch<uint16_t>(x, res, gamma, beta, out, rows, D, eps, st);
}
