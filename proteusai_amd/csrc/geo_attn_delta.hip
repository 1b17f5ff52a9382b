// D = rowsum(O * dO) for the attention backward, gfx950.
//
// The reference's backward wrapper takes it with torch before its kernel runs (old/old_scripts/attn/geometric_attn.py:618:
// `D = torch.sum(O*dO, dim=3)`); the backward kernels subtract it from dP.  Here: one pass over O (fp32) and dO (fp32,
// bf16 or fp16, as autograd hands it over), products and sum in fp32, D [Z,H,N] fp32.  HBM-bound streaming work:
// (4 + sizeof(dO element)) bytes per element read, 4 bytes per row written.  d / 4 lanes share a row, every lane
// loads 4 consecutive elements of both tensors (16 / 8 bytes), the lanes of a row meet by shuffles.

#include <hip/hip_runtime.h>
#include <stdint.h>
#include "proteus_hip.h"

namespace {

constexpr int GD_THREADS = 256;

struct GdStrides { long o[3], g[3]; };      // (batch, head, token) element strides of O and dO

template <int DTYPE> struct Grad;
template <> struct Grad<PROTEUS_DTYPE_F32> {
    typedef float T;
    static __device__ __forceinline__ void load(const float* p, float (&v)[4]) {
        const float4 t = *reinterpret_cast<const float4*>(p);
        v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
    }
};
template <> struct Grad<PROTEUS_DTYPE_BF16> {
    typedef uint16_t T;
    static __device__ __forceinline__ void load(const uint16_t* p, float (&v)[4]) {
        const uint2 t = *reinterpret_cast<const uint2*>(p);
        v[0] = __builtin_bit_cast(float, t.x << 16); v[1] = __builtin_bit_cast(float, t.x & 0xffff0000u);
        v[2] = __builtin_bit_cast(float, t.y << 16); v[3] = __builtin_bit_cast(float, t.y & 0xffff0000u);
    }
};
template <> struct Grad<PROTEUS_DTYPE_F16> {
    typedef uint16_t T;
    static __device__ __forceinline__ void load(const uint16_t* p, float (&v)[4]) {
        typedef _Float16 half2v __attribute__((ext_vector_type(2)));
        const uint2 t = *reinterpret_cast<const uint2*>(p);
        const half2v a = __builtin_bit_cast(half2v, t.x), b = __builtin_bit_cast(half2v, t.y);
        v[0] = (float)a[0]; v[1] = (float)a[1]; v[2] = (float)b[0]; v[3] = (float)b[1];
    }
};

// LPR = d / 4 lanes per row (8, 16, 32)
template <int DTYPE, int LPR>
__global__ __launch_bounds__(GD_THREADS)
void geo_attn_delta_kernel(const float* __restrict__ O, const typename Grad<DTYPE>::T* __restrict__ dO, float* __restrict__ D,
                           const long rows, const int H, const int N, const GdStrides st)
{
    constexpr int RPW = GD_THREADS / LPR;                    // rows per workgroup
    const int  sub = threadIdx.x % LPR;
    const long row = (long)blockIdx.x * RPW + threadIdx.x / LPR;
    float s = 0.f;
    if (row < rows) {
        const long n = row % N, zh = row / N;
        const long h = zh % H, z = zh / H;
        float a[4], b[4];
        const float* po = O + z * st.o[0] + h * st.o[1] + n * st.o[2] + 4 * sub;
        Grad<DTYPE>::load(dO + z * st.g[0] + h * st.g[1] + n * st.g[2] + 4 * sub, b);
        const float4 t = *reinterpret_cast<const float4*>(po);
        a[0] = t.x; a[1] = t.y; a[2] = t.z; a[3] = t.w;
#pragma unroll
        for (int e = 0; e < 4; ++e) s = __builtin_fmaf(a[e], b[e], s);
    }
    // (rows of a wave all take part: a row past the end adds zeros among its own lanes)
#pragma unroll
    for (int o = LPR / 2; o > 0; o >>= 1) s += __shfl_xor(s, o);
    if (row < rows && sub == 0) D[row] = s;
}

template <int DTYPE>
int launch(const float* O, const void* dO, float* D, int Z, int H, int N, int d, const GdStrides& st, hipStream_t stream)
{
    typedef typename Grad<DTYPE>::T T;
    const long rows = (long)Z * H * N;
    const int  lpr = d / 4;
    const dim3 grid((unsigned)((rows + GD_THREADS / lpr - 1) / (GD_THREADS / lpr)));
    if (lpr == 8)       hipLaunchKernelGGL((geo_attn_delta_kernel<DTYPE, 8>), grid, dim3(GD_THREADS), 0, stream, O, (const T*)dO, D, rows, H, N, st);
    else if (lpr == 16) hipLaunchKernelGGL((geo_attn_delta_kernel<DTYPE, 16>), grid, dim3(GD_THREADS), 0, stream, O, (const T*)dO, D, rows, H, N, st);
    else                hipLaunchKernelGGL((geo_attn_delta_kernel<DTYPE, 32>), grid, dim3(GD_THREADS), 0, stream, O, (const T*)dO, D, rows, H, N, st);
    return (int)hipGetLastError();
}

int check(const float* O, const void* dO, const int64_t* strides, const float* D, int Z, int H, int N, int d_head, int dtype, GdStrides& st)
{
    if (!O || !dO || !D) return PROTEUS_ERR_NULL_POINTER;
    if (d_head != 32 && d_head != 64 && d_head != 128) return PROTEUS_ERR_BAD_HEAD_DIM;
    if (dtype != PROTEUS_DTYPE_F32 && dtype != PROTEUS_DTYPE_BF16 && dtype != PROTEUS_DTYPE_F16) return PROTEUS_ERR_BAD_OPERAND_TYPE;
    if (Z <= 0 || H <= 0 || N <= 0 || N > PROTEUS_ATTN_MAX_N || (long)Z * H > 65535) return PROTEUS_ERR_BAD_SHAPE;
    if ((long)Z * H * N / (GD_THREADS / (d_head / 4)) >= (1L << 31) - 1) return PROTEUS_ERR_BAD_SHAPE;      // grid.x below 2^31
    const int gbytes = dtype == PROTEUS_DTYPE_F32 ? 4 : 2;
    if (((uintptr_t)O & 15) || ((uintptr_t)dO & (uintptr_t)(4 * gbytes - 1)) || ((uintptr_t)D & 3)) return PROTEUS_ERR_BAD_ALIGNMENT;
    if (!strides) {
        st.o[0] = st.g[0] = (long)H * N * d_head; st.o[1] = st.g[1] = (long)N * d_head; st.o[2] = st.g[2] = d_head;
        return PROTEUS_OK;
    }
    for (int i = 0; i < 3; ++i) { st.o[i] = (long)strides[i]; st.g[i] = (long)strides[3 + i]; }
    for (int i = 0; i < 3; ++i) {
        // rows of d elements must not overlap and every row must start on a 16-byte (O) / 4-element (dO) boundary
        if (st.o[i] < 0 || st.g[i] < 0) return PROTEUS_ERR_BAD_LAYOUT;
        if ((st.o[i] & 3) || (st.g[i] & 3)) return PROTEUS_ERR_BAD_ALIGNMENT;
    }
    if (st.o[2] < d_head || st.g[2] < d_head) return PROTEUS_ERR_BAD_LAYOUT;
    return PROTEUS_OK;
}

}  // namespace

extern "C" int proteus_geo_attn_delta_check(const float* O, const void* dO, const int64_t* strides, const float* D,
                                            int Z, int H, int N, int d_head, int dO_dtype)
{
    GdStrides st;
    return check(O, dO, strides, D, Z, H, N, d_head, dO_dtype, st);
}

extern "C" int proteus_geo_attn_delta(const float* O, const void* dO, const int64_t* strides, float* D,
                                      int Z, int H, int N, int d_head, int dO_dtype, void* stream)
{
    GdStrides st;
    const int rc = check(O, dO, strides, D, Z, H, N, d_head, dO_dtype, st);
    if (rc != PROTEUS_OK) return rc;
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    if (dO_dtype == PROTEUS_DTYPE_F32)  return launch<PROTEUS_DTYPE_F32>(O, dO, D, Z, H, N, d_head, st, s);
    if (dO_dtype == PROTEUS_DTYPE_BF16) return launch<PROTEUS_DTYPE_BF16>(O, dO, D, Z, H, N, d_head, st, s);
    return launch<PROTEUS_DTYPE_F16>(O, dO, D, Z, H, N, d_head, st, s);
}
