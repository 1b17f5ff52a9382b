// The order in which the workgroups of a Wavefunction Embedding forward launch take their (batch item, observer block,
// wavenumber tile) when the batch is padded: shared by the isotropic and the anisotropic kernel.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "ranked_order.h"

namespace proteus_we {

// Padded batches of up to proteus_ranked::MAX_Z items of at least WE_RANK_MIN_N tokens, whose mask has at most
// proteus_ranked::MAX_BYTES and whose launch at most WE_RANK_MAX_WGS workgroups, are handed out by the number of sources of
// their items (ranked_order.h says how).  Measured against the rotated order (isotropic kernel), lengths drawn from
// [N/8, N]: 8 x 1024 (six draws) -4 ... -27 %, 16 x 512 -21 %, 2 x 8192 -45 %, 8 x 2048 -14 %, 32 x 512 -9 %, 16 x 1024 -6 %,
// 4 x 4096 -1 %; beyond the limits the scan (paid by the workgroups of padded blocks too, which otherwise leave at once)
// costs more than the order gains: 64 x 256 +17 %, 64 x 512 (8192 workgroups, 8 rounds) +5 %, 64 x 1024 +3 %.
constexpr int WE_RANK_MAX_WGS = 4096, WE_RANK_MIN_N = 512;

// Called by every thread of a workgroup (256 threads) of a launch over (observer blocks, wavenumber tiles, batch items),
// before any divergence; leaves z, ytile and iblock alone and returns false where the launch keeps its own order.
__device__ __forceinline__ bool we_ranked_workgroup(const uint8_t* __restrict__ mask, const int N, int& z, int& ytile, int& iblock)
{
    const int Zb = (int)gridDim.z;
    if (mask && Zb > 1 && Zb <= proteus_ranked::MAX_Z && N >= WE_RANK_MIN_N && (size_t)Zb * (size_t)N <= (size_t)proteus_ranked::MAX_BYTES &&
        (long)gridDim.x * gridDim.y * Zb <= WE_RANK_MAX_WGS) {
        __shared__ proteus_ranked::Tables tables;
        proteus_ranked::scan_and_rank(mask, N, Zb, true, tables);
        const long b = (long)blockIdx.x + (long)gridDim.x * ((long)blockIdx.y + (long)gridDim.y * (long)blockIdx.z);
        proteus_ranked::place(b, Zb, (int)gridDim.x, (int)gridDim.y, 64, tables, z, iblock, ytile);
        return true;
    }
    return false;
}

}  // namespace proteus_we
