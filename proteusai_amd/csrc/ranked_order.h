// Handing out the workgroups of a padded batch by the length of their batch items (the Wavefunction Embedding forward
// kernels, through we_ranked.h).
//
// The launch of a padded batch of a few items is one or two rounds of the chip, so it lasts as long as the compute unit
// whose workgroups have the most to do, and a workgroup's time follows the length of its item.  Every workgroup scans
// the whole mask (a few KB: 16-byte pieces, all loads of a thread in flight together), ranks the items and takes its
// place in the list "live workgroups of the longest item, ..., of the shortest, then the workgroups whose tokens are
// all behind their item's last unpadded one".  The dispatcher gives every compute unit one workgroup before any gets
// its next, so workgroups b, b + 256, b + 512 ... share a unit: the list is laid over the launch as a snake (every
// second row of 256 reversed), which gives every unit a long, a short, a middling ... workgroup.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace proteus_ranked {

constexpr int MAX_Z     = 64;            // items that are ranked (their tables live in LDS)
constexpr int MAX_BYTES = 64 * 1024;     // largest mask that every workgroup scans
constexpr int ROW       = 256;           // compute units of the chip
constexpr int THREADS   = 256;           // the workgroup shape of the kernels that call this

struct Tables { int last[MAX_Z], cnt[MAX_Z], ord[MAX_Z]; };

// last[z] = 1 + index of the last unpadded token of item z, cnt[z] = number of unpadded tokens, ord[r] = the item of
// rank r (by cnt if by_count, else by last; ties by index).  Called by all THREADS threads; ends with a barrier.
__device__ __forceinline__ void scan_and_rank(const uint8_t* __restrict__ mask, const int N, const int Zb, const bool by_count, Tables& t)
{
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if (tid < Zb) { t.last[tid] = 0; t.cnt[tid] = 0; }
    __syncthreads();
    if ((N & 15) == 0 && ((uintptr_t)mask & 15) == 0) {
        const int per_item = N >> 4, pieces = Zb * per_item;       // (a piece lies inside one item)
        for (int p = tid; p < pieces; p += THREADS) {
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
                atomicAdd(&t.cnt[zz], cnt);
                atomicMax(&t.last[zz], (p - zz * per_item) * 16 + last);
            }
        }
    } else {
        for (int zz = wave; zz < Zb; zz += THREADS / 64) {
            const uint8_t* m = mask + (size_t)zz * (size_t)N;
            int last = 0, cnt = 0;
            for (int j = lane; j < N; j += 64) if (!m[j]) { last = j + 1; ++cnt; }
            for (int o = 32; o > 0; o >>= 1) { last = max(last, __shfl_xor(last, o)); cnt += __shfl_xor(cnt, o); }
            if (lane == 0) { t.last[zz] = last; t.cnt[zz] = cnt; }
        }
    }
    __syncthreads();
    if (tid < Zb) {
        const int mine = by_count ? t.cnt[tid] : t.last[tid];
        int r = 0;
        for (int u = 0; u < Zb; ++u) { const int o = by_count ? t.cnt[u] : t.last[u]; r += (o > mine || (o == mine && u < tid)) ? 1 : 0; }
        t.ord[r] = tid;
    }
    __syncthreads();
}

// The place of workgroup b of a launch of total = Zb x rows x cols workgroups: item z, row (a block of `block` tokens,
// live while it starts before last[z]) and column.  Workgroup-uniform.
__device__ __forceinline__ void place(const long b, const int Zb, const int rows, const int cols, const int block, const Tables& t,
                                      int& z, int& row, int& col)
{
    const long total = (long)Zb * rows * cols;
    const long row0 = b - b % ROW;
    const long rowlen = (total - row0 < ROW) ? total - row0 : (long)ROW;
    long rem = ((b / ROW) & 1) ? row0 + (rowlen - 1 - (b - row0)) : b;
    int zsel = -1, first = 0;
    for (int r = 0; r < Zb && zsel < 0; ++r) {            // the live workgroups
        const int zz = t.ord[r];
        const long n = (long)((t.last[zz] + block - 1) / block) * cols;
        if (rem < n) zsel = zz; else rem -= n;
    }
    for (int r = 0; r < Zb && zsel < 0; ++r) {            // those behind the last unpadded token
        const int zz = t.ord[r];
        const int live = (t.last[zz] + block - 1) / block;
        const long n = (long)(rows - live) * cols;
        if (rem < n) { zsel = zz; first = live; } else rem -= n;
    }
    z   = __builtin_amdgcn_readfirstlane(zsel);
    col = __builtin_amdgcn_readfirstlane((int)(rem % cols));
    row = __builtin_amdgcn_readfirstlane(first + (int)(rem / cols));
}

}  // namespace proteus_ranked
