// The order in which the workgroups of a Wavefunction Embedding forward launch take their (batch item, observer block,
// wavenumber tile) when the batch is padded: shared by the isotropic and the anisotropic kernel.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace proteus_we {

// Padded batches of up to WE_RANK_MAX_Z items of at least WE_RANK_MIN_N tokens, whose mask has at most WE_RANK_MAX_BYTES
// and whose launch at most WE_RANK_MAX_WGS workgroups, are handed out by the number of sources of their items;
// WE_RANK_ROW = compute units of the chip.  Measured against the rotated order (isotropic kernel), lengths drawn from
// [N/8, N]: 8 x 1024 (six draws) -4 ... -27 %, 16 x 512 -21 %, 2 x 8192 -45 %, 8 x 2048 -14 %, 32 x 512 -9 %, 16 x 1024 -6 %,
// 4 x 4096 -1 %; beyond the limits the scan (paid by the workgroups of padded blocks too, which otherwise leave at once)
// costs more than the order gains: 64 x 256 +17 %, 64 x 512 (8192 workgroups, 8 rounds) +5 %, 64 x 1024 +3 %.
#ifndef WE_RANKED
#define WE_RANKED 1
#endif
constexpr int WE_RANK_MAX_Z = 64, WE_RANK_MAX_BYTES = 64 * 1024, WE_RANK_ROW = 256, WE_RANK_MAX_WGS = 4096;
#ifndef WE_RANK_MIN_N
#define WE_RANK_MIN_N 512
#endif
constexpr int WE_RANK_WAVES = 4, WE_RANK_THREADS = 256;      // the workgroup shape of the kernels that call this

// A padded batch of a few items: the time of a workgroup follows the number of unpadded sources of its item, and
// the launch is about one round of the chip, so it lasts as long as the compute unit whose workgroups have the
// most to do.  Every workgroup scans the whole mask (a few KB), ranks the items by their number of sources and
// takes its place in the list "live workgroups of the item with the most sources, ..., of the one with the fewest,
// then the workgroups of the blocks behind every item's last unpadded token".  The dispatcher gives every compute
// unit one workgroup before any gets its next, so workgroups b, b + 256, b + 512 ... share a unit: the list is laid
// over the launch as a snake (every second row of 256 reversed), which gives every unit a long, a short, a
// middling ... workgroup.
// Called by every thread of a workgroup of a launch over (observer blocks, wavenumber tiles, batch items), before any
// divergence; leaves z, ytile and iblock alone and returns false where the launch keeps its own order.
__device__ __forceinline__ bool we_ranked_workgroup(const uint8_t* __restrict__ mask, const int N, int& z, int& ytile, int& iblock)
{
#if WE_RANKED
    const int tid  = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int Zb = (int)gridDim.z;
    if (mask && Zb > 1 && Zb <= WE_RANK_MAX_Z && N >= WE_RANK_MIN_N && (size_t)Zb * (size_t)N <= (size_t)WE_RANK_MAX_BYTES &&
        (long)gridDim.x * gridDim.y * Zb <= WE_RANK_MAX_WGS) {
        __shared__ int s_rlast[WE_RANK_MAX_Z], s_rcnt[WE_RANK_MAX_Z], s_rord[WE_RANK_MAX_Z];
        if (tid < Zb) { s_rlast[tid] = 0; s_rcnt[tid] = 0; }
        __syncthreads();
        if ((N & 15) == 0 && ((uintptr_t)mask & 15) == 0) {
            // the mask as one array of 16-byte pieces, each inside one item: all loads of a thread in flight together
            const int per_item = N >> 4, pieces = Zb * per_item;
            for (int p = tid; p < pieces; p += WE_RANK_THREADS) {
                const uint4 m16 = *reinterpret_cast<const uint4*>(mask + (size_t)p * 16);
                const unsigned w[4] = {m16.x, m16.y, m16.z, m16.w};
                int last = 0, cnt = 0;
#pragma unroll
                for (int e = 0; e < 4; ++e)
#pragma unroll
                    for (int q = 0; q < 4; ++q)
                        if (((w[e] >> (8 * q)) & 0xffu) == 0u) { last = 4 * e + q + 1; ++cnt; }
                if (cnt) {
                    const int zz = p / per_item;
                    atomicAdd(&s_rcnt[zz], cnt);
                    atomicMax(&s_rlast[zz], (p - zz * per_item) * 16 + last);
                }
            }
        } else {
            for (int zz = wave; zz < Zb; zz += WE_RANK_WAVES) {
                const uint8_t* m = mask + (size_t)zz * (size_t)N;
                int last = 0, cnt = 0;
                for (int j = lane; j < N; j += 64) if (!m[j]) { last = j + 1; ++cnt; }
                for (int o = 32; o > 0; o >>= 1) { last = max(last, __shfl_xor(last, o)); cnt += __shfl_xor(cnt, o); }
                if (lane == 0) { s_rlast[zz] = last; s_rcnt[zz] = cnt; }
            }
        }
        __syncthreads();
        if (tid < Zb) {
            const int mine = s_rcnt[tid];
            int r = 0;
            for (int u = 0; u < Zb; ++u) { const int o = s_rcnt[u]; r += (o > mine || (o == mine && u < tid)) ? 1 : 0; }
            s_rord[r] = tid;
        }
        __syncthreads();
        const int gx = (int)gridDim.x, gy = (int)gridDim.y;
        const long total = (long)gx * gy * Zb;
        const long b = (long)blockIdx.x + (long)gx * ((long)blockIdx.y + (long)gy * (long)blockIdx.z);
        const long row0 = b - b % WE_RANK_ROW;
        const long rowlen = (total - row0 < WE_RANK_ROW) ? total - row0 : (long)WE_RANK_ROW;
        long rem = ((b / WE_RANK_ROW) & 1) ? row0 + (rowlen - 1 - (b - row0)) : b;
        int zsel = -1, first = 0;
        for (int r = 0; r < Zb && zsel < 0; ++r) {            // the live workgroups
            const int zz = s_rord[r];
            const long cnt = (long)((s_rlast[zz] + 63) / 64) * gy;
            if (rem < cnt) zsel = zz; else rem -= cnt;
        }
        for (int r = 0; r < Zb && zsel < 0; ++r) {            // those of the blocks behind the last unpadded token
            const int zz = s_rord[r];
            const int live = (s_rlast[zz] + 63) / 64;
            const long cnt = (long)(gx - live) * gy;
            if (rem < cnt) { zsel = zz; first = live; } else rem -= cnt;
        }
        z      = __builtin_amdgcn_readfirstlane(zsel);
        ytile  = __builtin_amdgcn_readfirstlane((int)(rem % gy));
        iblock = __builtin_amdgcn_readfirstlane(first + (int)(rem / gy));
        return true;
    }
#endif
    return false;
}

}  // namespace proteus_we
