// Backward of the wavefunction embedding for gfx950: the contraction of dO with what the forward kept.
//
// Isotropic (isotropic/cuda/wf_embedding.py:64-83):
//   d_wavenumbers[k] = sum_{z,n} dO[z,n,2k+1] * cos_sums[z,n,k] - dO[z,n,2k] * sin_sums[z,n,k]
// Anisotropic (anisotropic/cb_scaling/learnable_wavenumbers/cuda/wf_embedding.py:65-79):
//   g_cb[k] = sum_{z,n} dO[z,n,2k] * d_cb[z,n,2k] + dO[z,n,2k+1] * d_cb[z,n,2k+1]      (and the same with d_k)
//
// Pure streaming work, bound by HBM: 16 (isotropic) or 24 (anisotropic) bytes per (token, wavenumber).
// Two launches, no atomics, deterministic: every workgroup reduces a contiguous slab of token rows into
// one row of partial sums in the caller's workspace (a lane owns one wavenumber, so every load is a
// coalesced 4- or 8-byte-per-lane row segment), then one small kernel adds the slabs in a fixed order.

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <mutex>
#include "proteus_hip.h"

// Partial sums of proteus_we_bwd_static: one row of PROTEUS_WE_BWD_STATIC_MAX_K floats per slab (2 MiB).  Every
// GPU the library runs on holds its own copy at its own address until the process ends.  In host code this
// name is only a handle for hipGetSymbolAddress; kernels are given the address that call returns.
static __device__ __align__(256) float scratch[1024 * PROTEUS_WE_BWD_STATIC_MAX_K];

namespace {

constexpr int WB_THREADS   = 256;
constexpr int WB_MAX_SLABS = 1024;     // rows of partial sums in the workspace
constexpr int WB_MIN_ROWS  = 8;        // a slab is not made smaller than this
constexpr int WB_UNROLL    = 4;        // token rows in flight per lane
static_assert(sizeof(scratch) == (size_t)WB_MAX_SLABS * PROTEUS_WE_BWD_STATIC_MAX_K * sizeof(float), "scratch holds one row per slab");

__host__ __device__ inline int slabs_for(long rows) {
    long g = (rows + WB_MIN_ROWS - 1) / WB_MIN_ROWS;
    if (g > WB_MAX_SLABS) g = WB_MAX_SLABS;
    if (g < 1) g = 1;
    return (int)g;
}

// ANISO = false: a0 = cos_sums, a1 = sin_sums ([R,K]); one output.
// ANISO = true : a0 = d_cb, a1 = d_k ([R,2K]); two outputs (either may be skipped with a NULL pointer).
// grid = (slabs, ceil(K/256)); partial[(slab * n_out + o) * K + k]
template <bool ANISO>
__global__ __launch_bounds__(WB_THREADS)
void we_bwd_partial_kernel(const float* __restrict__ d_out, const float* __restrict__ a0, const float* __restrict__ a1,
                           float* __restrict__ partial, const long rows, const int K, const int n_out)
{
    __shared__ float red[2][WB_THREADS];
    const int tid = threadIdx.x;
    const int kc0 = blockIdx.y * WB_THREADS;
    const int kc  = min(K - kc0, WB_THREADS);          // wavenumbers of this chunk
    int kp = 1;
    while (kp < kc) kp <<= 1;                          // lanes per token row (power of two <= 256)
    const int rp  = WB_THREADS / kp;                   // token rows handled side by side
    const int kl  = tid & (kp - 1);
    const int sub = tid / kp;
    const bool k_ok = kl < kc;
    const int k = kc0 + (k_ok ? kl : 0);

    const long per = (rows + gridDim.x - 1) / gridDim.x;
    const long r0 = (long)blockIdx.x * per;
    const long r1 = (r0 + per < rows) ? r0 + per : rows;

    float s0 = 0.f, s1 = 0.f;
    const size_t ld2 = (size_t)2 * K;
    long r = r0 + sub;
    for (; r + (long)(WB_UNROLL - 1) * rp < r1; r += (long)WB_UNROLL * rp) {
        float2 g[WB_UNROLL], p[WB_UNROLL], q[WB_UNROLL];
#pragma unroll
        for (int u = 0; u < WB_UNROLL; ++u) {
            const size_t row = (size_t)(r + (long)u * rp);
            g[u] = *reinterpret_cast<const float2*>(d_out + row * ld2 + 2 * k);
            if (ANISO) {
                p[u] = a0 ? *reinterpret_cast<const float2*>(a0 + row * ld2 + 2 * k) : make_float2(0.f, 0.f);
                q[u] = a1 ? *reinterpret_cast<const float2*>(a1 + row * ld2 + 2 * k) : make_float2(0.f, 0.f);
            } else {
                p[u] = make_float2(a0[row * K + k], a1[row * K + k]);
            }
        }
#pragma unroll
        for (int u = 0; u < WB_UNROLL; ++u) {
            if (ANISO) {
                s0 = __builtin_fmaf(g[u].x, p[u].x, __builtin_fmaf(g[u].y, p[u].y, s0));
                s1 = __builtin_fmaf(g[u].x, q[u].x, __builtin_fmaf(g[u].y, q[u].y, s1));
            } else {
                s0 = __builtin_fmaf(g[u].y, p[u].x, __builtin_fmaf(-g[u].x, p[u].y, s0));
            }
        }
    }
    for (; r < r1; r += rp) {
        const size_t row = (size_t)r;
        const float2 g = *reinterpret_cast<const float2*>(d_out + row * ld2 + 2 * k);
        if (ANISO) {
            if (a0) { const float2 p = *reinterpret_cast<const float2*>(a0 + row * ld2 + 2 * k); s0 = __builtin_fmaf(g.x, p.x, __builtin_fmaf(g.y, p.y, s0)); }
            if (a1) { const float2 q = *reinterpret_cast<const float2*>(a1 + row * ld2 + 2 * k); s1 = __builtin_fmaf(g.x, q.x, __builtin_fmaf(g.y, q.y, s1)); }
        } else {
            s0 = __builtin_fmaf(g.y, a0[row * K + k], __builtin_fmaf(-g.x, a1[row * K + k], s0));
        }
    }
    // the rp side-by-side rows of a wavenumber meet in LDS, added in a fixed order
    red[0][tid] = s0;
    red[1][tid] = s1;
    __syncthreads();
    if (sub == 0 && k_ok) {
        float t0 = 0.f, t1 = 0.f;
        for (int j = 0; j < rp; ++j) { t0 += red[0][j * kp + kl]; t1 += red[1][j * kp + kl]; }
        float* dst = partial + (size_t)blockIdx.x * n_out * K;
        dst[k] = t0;
        if (ANISO) dst[K + k] = t1;
    }
}

// out_o[k] = sum over the slabs.  A workgroup takes WB_FK wavenumbers (few of them: many small workgroups are done
// sooner than few large ones); WB_THREADS / WB_FK lanes share each wavenumber's slabs (lane j takes slabs j,
// j + lanes, ...: independent loads, many in flight) and their partial sums meet in LDS in a fixed order.
constexpr int WB_FK = 4;
__global__ __launch_bounds__(WB_THREADS)
void we_bwd_final_kernel(const float* __restrict__ partial, float* __restrict__ out0, float* __restrict__ out1,
                         const int slabs, const int K, const int n_out)
{
    __shared__ float red[2][WB_THREADS];
    constexpr int LANES = WB_THREADS / WB_FK;
    const int kl = threadIdx.x % WB_FK, sl = threadIdx.x / WB_FK;
    const int k = blockIdx.x * WB_FK + kl;
    float t0 = 0.f, t1 = 0.f;
    if (k < K) {
#pragma unroll 8
        for (int g = sl; g < slabs; g += LANES) {
            t0 += partial[(size_t)g * n_out * K + k];
            if (n_out == 2) t1 += partial[(size_t)g * n_out * K + K + k];
        }
    }
    red[0][threadIdx.x] = t0;
    red[1][threadIdx.x] = t1;
    __syncthreads();
    if (sl == 0 && k < K) {
        float u0 = 0.f, u1 = 0.f;
        for (int j = 0; j < LANES; ++j) { u0 += red[0][j * WB_FK + kl]; u1 += red[1][j * WB_FK + kl]; }
        if (out0) out0[k] = u0;
        if (n_out == 2 && out1) out1[k] = u1;
    }
}

}  // namespace

extern "C" size_t proteus_we_bwd_workspace_bytes(int Z, int N, int K) {
    if (Z <= 0 || N <= 0 || K <= 0) return 0;
    return (size_t)slabs_for((long)Z * N) * 2 * K * sizeof(float);
}

namespace {

int check_common(const void* d_out, const void* workspace, size_t workspace_bytes, int Z, int N, int K, int n_out) {
    if (!d_out || !workspace) return PROTEUS_ERR_NULL_POINTER;
    if (Z <= 0 || N <= 0 || K <= 0 || N > PROTEUS_WE_MAX_N || K > PROTEUS_WE_MAX_K) return PROTEUS_ERR_BAD_SHAPE;
    if (((uintptr_t)d_out & 7) || ((uintptr_t)workspace & 3)) return PROTEUS_ERR_BAD_ALIGNMENT;
    (void)n_out;
    if (workspace_bytes < proteus_we_bwd_workspace_bytes(Z, N, K)) return PROTEUS_ERR_BAD_SHAPE;
    return PROTEUS_OK;
}

}  // namespace

extern "C" int proteus_we_bwd_check(const float* d_out, const float* cos_sums, const float* sin_sums,
                                    const float* d_wavenumbers, const float* workspace, size_t workspace_bytes,
                                    int Z, int N, int K)
{
    if (!cos_sums || !sin_sums || !d_wavenumbers) return PROTEUS_ERR_NULL_POINTER;
    return check_common(d_out, workspace, workspace_bytes, Z, N, K, 1);
}

extern "C" int proteus_we_bwd(const float* d_out, const float* cos_sums, const float* sin_sums,
                              float* d_wavenumbers, float* workspace, size_t workspace_bytes,
                              int Z, int N, int K, void* stream)
{
    const int rc = proteus_we_bwd_check(d_out, cos_sums, sin_sums, d_wavenumbers, workspace, workspace_bytes, Z, N, K);
    if (rc != PROTEUS_OK) return rc;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    const long rows = (long)Z * N;
    const int slabs = slabs_for(rows);
    const int kchunks = (K + WB_THREADS - 1) / WB_THREADS;
    hipLaunchKernelGGL((we_bwd_partial_kernel<false>), dim3(slabs, kchunks), dim3(WB_THREADS), 0, st,
                       d_out, cos_sums, sin_sums, workspace, rows, K, 1);
    hipLaunchKernelGGL(we_bwd_final_kernel, dim3((K + WB_FK - 1) / WB_FK), dim3(WB_THREADS), 0, st,
                       (const float*)workspace, d_wavenumbers, (float*)nullptr, slabs, K, 1);
    return (int)hipGetLastError();
}

namespace {

// Device address of `scratch` on each GPU, looked up on the first call made with that GPU current.
constexpr int WB_MAX_DEVICES = 64;
std::mutex g_scratch_mutex;
float*     g_scratch_ptr[WB_MAX_DEVICES] = {};

int scratch_for_current_device(float** ptr) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= WB_MAX_DEVICES) return (int)hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        if (!p) return (int)hipErrorInvalidSymbol;
        g_scratch_ptr[dev] = static_cast<float*>(p);
    }
    *ptr = g_scratch_ptr[dev];
    return PROTEUS_OK;
}

}  // namespace

extern "C" int proteus_we_bwd_static(const float* d_out, const float* cos_sums, const float* sin_sums,
                                     float* d_wavenumbers, int Z, int N, int K, void* stream)
{
    if (!d_out || !cos_sums || !sin_sums || !d_wavenumbers) return PROTEUS_ERR_NULL_POINTER;
    if (Z <= 0 || N <= 0 || K <= 0 || N > PROTEUS_WE_MAX_N) return PROTEUS_ERR_BAD_SHAPE;
    if (K > PROTEUS_WE_BWD_STATIC_MAX_K) return PROTEUS_ERR_TOO_LARGE;
    if ((uintptr_t)d_out & 7) return PROTEUS_ERR_BAD_ALIGNMENT;
    float* partial = nullptr;
    const int rc = scratch_for_current_device(&partial);
    if (rc != PROTEUS_OK) return rc;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    const long rows = (long)Z * N;
    const int slabs = slabs_for(rows);
    const int kchunks = (K + WB_THREADS - 1) / WB_THREADS;
    // the first kernel overwrites every partial sum the second one reads: nothing has to start at zero
    hipLaunchKernelGGL((we_bwd_partial_kernel<false>), dim3(slabs, kchunks), dim3(WB_THREADS), 0, st,
                       d_out, cos_sums, sin_sums, partial, rows, K, 1);
    hipLaunchKernelGGL(we_bwd_final_kernel, dim3((K + WB_FK - 1) / WB_FK), dim3(WB_THREADS), 0, st,
                       (const float*)partial, d_wavenumbers, (float*)nullptr, slabs, K, 1);
    return (int)hipGetLastError();
}

extern "C" int proteus_we_aniso_bwd_check(const float* d_out, const float* d_cb, const float* d_k,
                                          const float* g_cb, const float* g_k,
                                          const float* workspace, size_t workspace_bytes, int Z, int N, int K)
{
    // a gradient that is not wanted is skipped by passing NULL for both its partials and its output
    if ((d_cb == nullptr) != (g_cb == nullptr) || (d_k == nullptr) != (g_k == nullptr)) return PROTEUS_ERR_NULL_POINTER;
    if (!g_cb && !g_k) return PROTEUS_ERR_NULL_POINTER;
    if (((uintptr_t)d_cb & 7) || ((uintptr_t)d_k & 7)) return PROTEUS_ERR_BAD_ALIGNMENT;
    return check_common(d_out, workspace, workspace_bytes, Z, N, K, 2);
}

extern "C" int proteus_we_aniso_bwd(const float* d_out, const float* d_cb, const float* d_k,
                                    float* g_cb, float* g_k, float* workspace, size_t workspace_bytes,
                                    int Z, int N, int K, void* stream)
{
    const int rc = proteus_we_aniso_bwd_check(d_out, d_cb, d_k, g_cb, g_k, workspace, workspace_bytes, Z, N, K);
    if (rc != PROTEUS_OK) return rc;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    const long rows = (long)Z * N;
    const int slabs = slabs_for(rows);
    const int kchunks = (K + WB_THREADS - 1) / WB_THREADS;
    hipLaunchKernelGGL((we_bwd_partial_kernel<true>), dim3(slabs, kchunks), dim3(WB_THREADS), 0, st,
                       d_out, d_cb, d_k, workspace, rows, K, 2);
    hipLaunchKernelGGL(we_bwd_final_kernel, dim3((K + WB_FK - 1) / WB_FK), dim3(WB_THREADS), 0, st,
                       (const float*)workspace, g_cb, g_k, slabs, K, 2);
    return (int)hipGetLastError();
}
