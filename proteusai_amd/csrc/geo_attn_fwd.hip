// RBF-scaled geometric flash-attention forward for gfx950 (MI355X), d_head = 32, 64 or 128 (this file: 64 and the C ABI).
//
// What it computes (README.md:40 logits on the flash structure of
// old/old_scripts/attn/geometric_attn.py:57-260):
//   s_ij = (q_i . k_j)/sqrt(d) * (1 + exp(-|r_i - r_j|^2 / (2 sigma_h^2))),  -inf for padded keys
//   O_i  = softmax_j(s_ij) V_j,  L_i = logsumexp_j s_ij;  padded/empty rows -> O = 0, L = -inf
//
// Mapping to the machine.  A workgroup is 4 waves; a wave owns 64 queries of one
// (batch, head) as two blocks of 32 (one block where the grid would otherwise leave
// half of the wave slots empty) and walks the keys in tiles of 64 that the
// workgroup stages in LDS (K row-major, V transposed, key geometry), two tiles
// deep: tile t is consumed while tile t+1 travels global -> registers -> LDS.
// All products run on the matrix cores and are computed TRANSPOSED:
//   S^T (keys x queries)  = K_tile (A, from LDS) x Q^T (B, registers, loaded once)
//   D^T (keys x queries)  = G_tile (A, from LDS) x G_q^T (B, registers)     [geometry, see below]
//   O^T (d x queries)    += V^T_tile (A, from LDS) x P^T (B, registers)
// In the 32x32 accumulator layout a lane holds 16 rows of ONE column, so with
// queries on the columns each lane owns one query per block: the exponentials
// and the row sum are in-lane (the two half-waves of a query meet only when its
// softmax reference is re-based and at the end), and the S^T accumulator registers are, after conversion
// to bf16, already the B operand of the last product (the contraction index is
// merely visited in the permuted order the accumulator layout dictates, and the
// V^T operand is read from LDS in that same order).  Every A fragment read from
// LDS serves both query blocks.  The softmax keeps a lazy reference instead of a
// running maximum, and for blocks whose multiplier is 1 that reference is carried
// into the score product as one more contraction slot (see the key loop).
//
// Geometry on the matrix cores.  With x' = (x - c) * sqrt(log2(e)/2)/sigma_h (c = a
// point near the workgroup's queries) the multiplier is 1 + exp2(D),
//   D = -|x'_k - x'_q|^2 = -|x'_k|^2 + 2 x'_k . x'_q - |x'_q|^2 .
// Every fp32 scalar is split exactly into three bf16 pieces (8+8+8 mantissa
// bits), and D becomes a 24-term bf16 contraction whose products are exact in
// the fp32 accumulator: per coordinate the pieces hh, hm, mh, mm, hl, lh (the
// dropped ml, lm, ll are below 2^-24 of the product), plus the two squared
// norms against ones.  One 32x32x16 and one 32x32x8 MFMA per 32 keys replace six
// vector-ALU instructions per score.  The cancellation error is about
// 2^-20 (|x'_k|^2 + |x'_q|^2); it only matters where the multiplier differs from
// 1, i.e. for keys within ~6 sigma of the query, so with the origin near the
// queries it is below 3e-3 in D as long as the workgroup's queries lie within
// GA_MFMA_DIST_MAX_RHO2 of that origin.  A workgroup whose queries are spread
// wider evaluates the distances directly on the vector ALU instead.
// Nothing of size N x N exists anywhere.


#include <hip/hip_runtime.h>
#include <atomic>
#include <stdint.h>
#include <type_traits>
#include "proteus_hip.h"
#include "geo_attn_ops.h"
#include "geo_attn_internal.h"

namespace {

#include "geo_attn_fwd_body.inc"
#include "geo_attn_fwd_pipe.inc"

// True if the plan of a padded batch (see geo_attn_plan_kernel) marks a query tile whose tokens spread too far for
// the matrix-core distances: then the balanced kernel runs the direct-distance body instead.
// (`any_wide`: an int of the workgroup's LDS, free at that point)
__device__ __forceinline__ bool ga_plan_has_wide_tile(const int* __restrict__ wide, const int n, int& any_wide) {
    if (threadIdx.x == 0) any_wide = 0;
    __syncthreads();
    int w = 0;
    for (int i = threadIdx.x; i < n; i += GA_THREADS) w |= wide[i];
    if (w) any_wide = 1;
    __syncthreads();
    const bool r = any_wide != 0;
    __syncthreads();
    return r;
}

constexpr size_t GA_PIPE_LDS = ga_pipe_lds<64>();

// ---------------- padded batches: a balanced schedule over a persistent grid ----------------
//
// With a padding mask the plain grid gives every (batch, head, 256-query tile) one workgroup, whose key loop is as
// long as its sequence: when the grid is about one round of the chip, the launch lasts as long as the longest
// sequence's workgroups while the others' slots idle.  Here the work is laid out as one line of steps (a step = one
// key tile of one item; items ordered batch, head, query tile; only query tiles and key tiles up to the last unpadded
// token count) and cut into G equal shares, one per persistent workgroup.  A share is a few parts: the tail of one
// item, whole items, the head of another.  Every part leaves its unnormalised state in the caller's workspace; the
// last of an item's parts to finish (a counter per item says which) adds them up and writes O and L.  No workgroup
// ever waits for another.  The plan that all workgroups derive the same shares from (last unpadded token per query
// tile) is made by a small kernel launched before this one.

constexpr int    GB_MAX_WGS     = 512;                       // persistent workgroups: two per compute unit of a 256-CU chip
constexpr int    GB_MAX_Z       = 256;                       // batch items (their lengths and prefix sums live in LDS)
constexpr size_t GB_PART_FLOATS = (size_t)GP_PART_FLOATS;   // one part: the O^T accumulators of 256 queries, (reference, row sum) per query

struct BalSmem {
    PipeSmem pipe;
    int n_eff[GB_MAX_Z];             // 1 + index of the last unpadded token of a batch item
    int prefix[GB_MAX_Z + 1];        // steps before batch item z
    int flag;
};
static_assert(sizeof(BalSmem) <= 80 * 1024, "two workgroups per compute unit");

// Ints of the plan at the head of the workspace: tile_last [Z * nqt], wide [Z * nqt], counters [Z * nqt * H].
__host__ __device__ inline size_t gb_plan_ints(const int Z, const int H, const int nqt) { return (size_t)Z * nqt * (2 + (size_t)H); }
__host__ __device__ inline size_t gb_parts_offset(const int Z, const int H, const int nqt) {
    return (gb_plan_ints(Z, H, nqt) * sizeof(int) + 255) / 256 * 256;
}

// One workgroup per (query tile, batch item): 1 + index of its last unpadded token, whether its unpadded tokens lie
// too far apart for the matrix-core distances of the pipelined body at the smallest sigma (same origin as the body:
// midway between the first and the last unpadded token of the tile), and zeroed part counters of its H items.
__global__ __launch_bounds__(GA_THREADS)
void geo_attn_plan_kernel(const float* __restrict__ coords, const float* __restrict__ sigma, const uint8_t* __restrict__ key_pad,
                          int* __restrict__ plan, const int Z, const int H, const int N, const int nqt)
{
    __shared__ int s_lo, s_hi;
    __shared__ unsigned s_rho2;
    const int qt = (int)blockIdx.x, z = (int)blockIdx.y, tid = (int)threadIdx.x;
    int* tile_last = plan;
    int* wide      = plan + (size_t)Z * nqt;
    int* counters  = plan + (size_t)2 * Z * nqt;
    if (tid == 0) { s_lo = 0x7fffffff; s_hi = -1; s_rho2 = 0u; }
    __syncthreads();
    const int q = qt * GA_THREADS + tid;
    const bool valid = q < N && !(key_pad && key_pad[(size_t)z * N + q]);
    const float* cz = coords + (size_t)z * N * 3;
    float cx = 0.f, cy = 0.f, cw = 0.f;
    if (valid) { cx = cz[3 * q]; cy = cz[3 * q + 1]; cw = cz[3 * q + 2]; }
    {
        // first and last unpadded token of the wave from one ballot; one LDS atomic per wave
        const uint64_t bal = __builtin_amdgcn_ballot_w64(valid);
        if ((tid & 63) == 0 && bal != 0) {
            const int base = qt * GA_THREADS + (tid & ~63);
            atomicMin(&s_lo, base + __builtin_ctzll(bal));
            atomicMax(&s_hi, base + 63 - __builtin_clzll(bal));
        }
    }
    __syncthreads();
    const int lo = s_lo, hi = s_hi;
    if (hi >= 0) {
        const float ox = 0.5f * (cz[3 * lo] + cz[3 * hi]), oy = 0.5f * (cz[3 * lo + 1] + cz[3 * hi + 1]), oz = 0.5f * (cz[3 * lo + 2] + cz[3 * hi + 2]);
        const float dx = cx - ox, dy = cy - oy, dz = cw - oz;
        float r2 = valid ? dx * dx + dy * dy + dz * dz : 0.f;
        for (int o = 32; o > 0; o >>= 1) r2 = fmaxf(r2, __shfl_xor(r2, o));
        if ((tid & 63) == 0) atomicMax(&s_rho2, __builtin_bit_cast(unsigned, r2));
    }
    __syncthreads();
    const size_t t = (size_t)z * nqt + qt;
    if (tid == 0) {
        float cs_max = 0.f;
        for (int h = 0; h < H; ++h) cs_max = fmaxf(cs_max, 0.84932180028801907f / sigma[h]);
        tile_last[t] = hi + 1;
        // (a sigma that is not a positive number gives garbage either way; NaN compares false: the plain grid's
        // behaviour is kept by calling the tile wide)
        const float rho2 = __builtin_bit_cast(float, s_rho2) * cs_max * cs_max;
        wide[t] = (hi >= 0 && !(rho2 <= GA_MFMA_DIST_MAX_RHO2)) ? 1 : 0;
    }
    for (int h = tid; h < H; h += GA_THREADS) counters[t * H + h] = 0;
}


// The last part of an item to finish adds the parts up, in the registers' layout and in part order:
// O = sum_p 2^(m_p - M) O_p / sum_p 2^(m_p - M) l_p with M the largest reference among the parts that saw a key, kept as a
// running maximum (what has been added is rescaled when it grows).  The parts are taken two at a time, all loads of
// a pair issued together: one round trip to memory per pair and query block.  slot_of(j): where part j lies.
template <typename SlotOf>
__device__ __forceinline__ void gb_merge_parts(const SlotOf& slot_of, const int first_g, const int last_g,
                                   float* __restrict__ O, float* __restrict__ L, const uint8_t* __restrict__ key_pad,
                                   const int z, const int h, const int zh, const int qt, const int N, const GaStrides& st)
{
    const int tid = (int)threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63, half = lane >> 5, col = lane & 31;
    float* Oh = O + (size_t)z * st.o[0] + (size_t)h * st.o[1];
    const uint8_t* mz = key_pad ? key_pad + (size_t)z * N : nullptr;
#pragma unroll 1
    for (int bq = 0; bq < 2; ++bq) {
        const int mlo = gp_part_ml_offset(wave, bq, col);
        float M = -INFINITY, l = 0.f;
        float acc[32];
#pragma unroll
        for (int r = 0; r < 32; ++r) acc[r] = 0.f;
#pragma unroll 1
        for (int j = first_g; j <= last_g; j += 2) {
            const bool two = j + 1 <= last_g;
            const __amdgpu_buffer_rsrc_t rpa = gp_part_rsrc(slot_of(j));
            const __amdgpu_buffer_rsrc_t rpb = gp_part_rsrc(slot_of(two ? j + 1 : j));
            const gp_uint2v rmla = __builtin_amdgcn_raw_buffer_load_b64(rpa, mlo, 0, GP_SC1);
            const gp_uint2v rmlb = __builtin_amdgcn_raw_buffer_load_b64(rpb, mlo, 0, GP_SC1);
            uint4v rawa[8], rawb[8];
#pragma unroll
            for (int q4 = 0; q4 < 8; ++q4) {
                const int off = gp_part_o_offset(wave, bq, q4 >> 2, q4 & 3, lane);
                rawa[q4] = __builtin_amdgcn_raw_buffer_load_b128(rpa, off, 0, GP_SC1);
                rawb[q4] = __builtin_amdgcn_raw_buffer_load_b128(rpb, off, 0, GP_SC1);
            }
            const floatx2 mla = __builtin_bit_cast(floatx2, rmla), mlb = __builtin_bit_cast(floatx2, rmlb);
            const bool ua = mla[1] > 0.f, ub = two && mlb[1] > 0.f;          // the part saw a key of this query
            const float Mn = fmaxf(M, fmaxf(ua ? mla[0] : -INFINITY, ub ? mlb[0] : -INFINITY));
            const float sc = (M > -INFINITY) ? __builtin_amdgcn_exp2f(M - Mn) : 0.f;
            const float wa = ua ? __builtin_amdgcn_exp2f(mla[0] - Mn) : 0.f;
            const float wb = ub ? __builtin_amdgcn_exp2f(mlb[0] - Mn) : 0.f;
            l = __builtin_fmaf(wb, mlb[1], __builtin_fmaf(wa, mla[1], l * sc));
#pragma unroll
            for (int q4 = 0; q4 < 8; ++q4) {
                const floatx4 va = __builtin_bit_cast(floatx4, rawa[q4]), vb = __builtin_bit_cast(floatx4, rawb[q4]);
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    acc[4 * q4 + e] = __builtin_fmaf(wb, vb[e], __builtin_fmaf(wa, va[e], acc[4 * q4 + e] * sc));
            }
            M = Mn;
        }
        const int qi = qt * (GA_WAVES * 64) + wave * 64 + 32 * bq + col;
        if (qi < N) {
            const bool row_ok = l > 0.f && !(mz && mz[qi]);
            const float inv_l = row_ok ? 1.0f / l : 0.f;
            float* orow = Oh + (size_t)qi * (size_t)st.o[2];
#pragma unroll
            for (int dt = 0; dt < 2; ++dt)
#pragma unroll
                for (int gq = 0; gq < 4; ++gq)
                    *reinterpret_cast<float4*>(orow + dt * 32 + 8 * gq + 4 * half) =
                        make_float4(acc[dt * 16 + 4 * gq] * inv_l, acc[dt * 16 + 4 * gq + 1] * inv_l,
                                    acc[dt * 16 + 4 * gq + 2] * inv_l, acc[dt * 16 + 4 * gq + 3] * inv_l);
            if (L && half == 0) L[(size_t)zh * N + qi] = row_ok ? (M + __log2f(l)) * 0.69314718055994531f : -INFINITY;
        }
    }
}

__global__ __launch_bounds__(GA_THREADS, 2)
void geo_attn_fwd_balanced_kernel(const uint16_t* __restrict__ Q, const uint16_t* __restrict__ K,
                                  const uint16_t* __restrict__ V, const float* __restrict__ coords,
                                  const float* __restrict__ sigma, const uint8_t* __restrict__ key_pad,
                                  float* __restrict__ O, float* __restrict__ L,
                                  int* __restrict__ plan, float* __restrict__ parts,
                                  const int Z, const int H, const int N, const int nqt, const GaStrides st)
{
    extern __shared__ __align__(16) unsigned char ga_dyn_smem[];
    BalSmem& bs = *reinterpret_cast<BalSmem*>(ga_dyn_smem);
    const int tid = (int)threadIdx.x;
    const int G = (int)gridDim.x;
    const int* tile_last = plan;
    const int* wide      = plan + (size_t)Z * nqt;
    int*       counters  = plan + (size_t)2 * Z * nqt;

    // ---- the plan every workgroup derives: lengths, steps before each batch item ----
    if (ga_plan_has_wide_tile(wide, Z * nqt, bs.flag)) {
        // A query tile whose tokens lie too far apart for the matrix-core distances of the pipelined body (an extended
        // chain): this batch is done with the direct-distance body instead, whole items in turn, no parts.
        static_assert(sizeof(Smem) <= sizeof(BalSmem), "the direct-distance body's LDS fits");
        for (int item = (int)blockIdx.x; item < Z * H * nqt; item += G) {
            __syncthreads();
            geo_attn_fwd_body<true, false, 2>(*reinterpret_cast<Smem*>(ga_dyn_smem), item, Q, K, V, coords, sigma, key_pad, O, L,
                                              H, N, Z * H, nqt, 1, nullptr, 0.f, 1.f, st);
        }
        return;
    }
    for (int z = tid; z < Z; z += GA_THREADS) {
        int last = 0;
        for (int qt = 0; qt < nqt; ++qt) last = max(last, tile_last[(size_t)z * nqt + qt]);
        bs.n_eff[z] = last;
    }
    __syncthreads();
    if (tid == 0) {
        int run = 0;
        for (int z = 0; z < Z; ++z) {
            bs.prefix[z] = run;
            const int ne = bs.n_eff[z];
            run += H * ((ne + GA_THREADS - 1) / GA_THREADS) * ((ne + GA_BN - 1) / GA_BN);
        }
        bs.prefix[Z] = run;
    }
    __syncthreads();
    const int total = bs.prefix[Z];
    const int share = max((total + G - 1) / G, 1);
    // consecutive workgroup numbers go to different XCDs: XCD x takes the x-th eighth of the line, so that the
    // workgroups that share an L2 work on neighbouring items (the same K and V)
    const int g = ((int)blockIdx.x & 7) * (G >> 3) + ((int)blockIdx.x >> 3);

    int a = min(g * share, total);
    const int b = min(a + share, total);
    while (a < b) {
        int z = 0;
        while (bs.prefix[z + 1] <= a) ++z;                      // (uniform: a few scalar steps)
        z = __builtin_amdgcn_readfirstlane(z);
        const int ne = bs.n_eff[z];
        const int nq = (ne + GA_THREADS - 1) / GA_THREADS, c = (ne + GA_BN - 1) / GA_BN;
        const int r = a - bs.prefix[z];
        const int item = r / c, k0 = r - item * c;
        const int h = item / nq, qt = item - h * nq;
        const int zh = z * H + h;
        const int start = a - k0;                               // first step of the item on the line
        const int k1 = min(c, k0 + (b - a));
        // the workgroups that hold parts of this item, and where each left (or will leave) its part: a workgroup's
        // slot 0 takes the item its share begins with, slot 1 an item that begins inside its share and ends beyond it
        const int first_g = start / share, last_g = (start + c - 1) / share;
        const int nparts = last_g - first_g + 1;
        auto slot_of = [&](const int j) -> float* {
            const int second = (j == first_g && start > j * share) ? 1 : 0;
            return parts + ((size_t)2 * j + second) * GB_PART_FLOATS;
        };
        float* mine = slot_of(g);
        const int rc = geo_attn_fwd_pipe_part<true>(bs.pipe, zh, qt, k0, k1, ne, mine,
                                                    Q, K, V, coords, sigma, key_pad, O, L, H, N, 1, st);
        if (rc == 0) {
            // The part was written with device-scope stores: once they have completed it is in memory for every
            // workgroup of the chip, and only then may the item's counter say so.
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
            if (tid == 0) bs.flag = (nparts == 1) ? 1 : (atomicAdd(&counters[((size_t)z * nqt + qt) * H + h], 1) == nparts - 1);
            __syncthreads();
            if (bs.flag) {
                gb_merge_parts(slot_of, first_g, last_g, O, L, key_pad, z, h, zh, qt, N, st);
            }
        }
        a += k1 - k0;
    }

    // ---- query tiles behind the last unpadded token of their sequence: zeros, L = -inf ----
    for (int e = (int)blockIdx.x; e < Z * H * nqt; e += G) {
        const int z = e / (H * nqt), rem = e - z * (H * nqt);
        const int h = rem / nqt, qt = rem - h * nqt;
        if (qt * GA_THREADS < bs.n_eff[z]) continue;
        float* Oh = O + (size_t)z * st.o[0] + (size_t)h * st.o[1];
        const int chunk = tid & 15;
        for (int ql = tid >> 4; ql < GA_THREADS; ql += GA_THREADS / 16) {
            const int qi = qt * GA_THREADS + ql;
            if (qi >= N) break;
            *reinterpret_cast<float4*>(Oh + (size_t)qi * (size_t)st.o[2] + 4 * chunk) = make_float4(0.f, 0.f, 0.f, 0.f);
            if (L && chunk == 0) L[((size_t)z * H + h) * N + qi] = -INFINITY;
        }
    }
}

// ---------------- padded batches, second schedule: long items split, longest parts first ----------------
//
// The items (batch, head, query tile) of a padded batch differ in the length of their key loops.  When there are fewer
// live items than the chip has workgroup slots (`cap`), the longest are split along the keys into equal parts until
// the parts fill the slots: the smallest part length T for which sum_items ceil(c_item / T) <= cap.  Parts are numbered
// longest first (sequences ranked by the length of their parts; within a sequence tile-major, the heads of a tile side
// by side, so that with 8 heads each XCD keeps to one head) and workgroup p takes part p: the hardware hands the
// workgroups out in this order.  An item that is not split is written directly; the parts of a split item meet as in
// the balanced schedule (state in the workspace, a ticket per part, the last arriver adds them up in part order).
// With at least `cap` live items nothing is split and the launch is the plain grid in longest-first order.
__global__ __launch_bounds__(GA_THREADS, 2)
void geo_attn_fwd_split_kernel(const uint16_t* __restrict__ Q, const uint16_t* __restrict__ K,
                               const uint16_t* __restrict__ V, const float* __restrict__ coords,
                               const float* __restrict__ sigma, const uint8_t* __restrict__ key_pad,
                               float* __restrict__ O, float* __restrict__ L,
                               int* __restrict__ plan, float* __restrict__ parts,
                               const int Z, const int H, const int N, const int nqt, const int cap,
                               const GaStrides st)
{
    extern __shared__ __align__(16) unsigned char ga_dyn_smem[];
    BalSmem& bs = *reinterpret_cast<BalSmem*>(ga_dyn_smem);
    const int tid = (int)threadIdx.x;
    const int G = (int)gridDim.x;
    const int* tile_last = plan;
    const int* wide      = plan + (size_t)Z * nqt;
    int*       counters  = plan + (size_t)2 * Z * nqt;

    if (ga_plan_has_wide_tile(wide, Z * nqt, bs.flag)) {
        for (int item = (int)blockIdx.x; item < Z * H * nqt; item += G) {
            __syncthreads();
            geo_attn_fwd_body<true, false, 2>(*reinterpret_cast<Smem*>(ga_dyn_smem), item, Q, K, V, coords, sigma, key_pad, O, L,
                                              H, N, Z * H, nqt, 1, nullptr, 0.f, 1.f, st);
        }
        return;
    }
    // (the tables below live in the K ring until the part begins: order[r], count prefix[r], splits[r] per rank)
    int* order  = reinterpret_cast<int*>(&bs.pipe.kring[0][0]);
    int* splits = order + GB_MAX_Z;
    for (int z = tid; z < Z; z += GA_THREADS) {
        int last = 0;
        for (int qt = 0; qt < nqt; ++qt) last = max(last, tile_last[(size_t)z * nqt + qt]);
        bs.n_eff[z] = last;
    }
    if (tid == 0) bs.flag = 0x7fffffff;
    __syncthreads();
    // live items, steps, longest key loop
    int items = 0, c_max = 0;
    long steps = 0;
    for (int z = 0; z < Z; ++z) {
        const int ne = bs.n_eff[z];
        const int nq = (ne + GA_THREADS - 1) / GA_THREADS, c = (ne + GA_BN - 1) / GA_BN;
        items += H * nq; steps += (long)H * nq * c; c_max = max(c_max, c);
    }
    int T = max(c_max, 1);
    if (items < cap && items > 0) {
        // the smallest part length whose parts fit the slots; thread t tries T_min + t
        const int T_min = max((int)((steps + cap - 1) / cap), 1);
        const int Tt = T_min + tid;
        if (Tt <= c_max) {
            int n = 0;
            for (int z = 0; z < Z; ++z) {
                const int ne = bs.n_eff[z];
                const int nq = (ne + GA_THREADS - 1) / GA_THREADS, c = (ne + GA_BN - 1) / GA_BN;
                n += H * nq * ((c + Tt - 1) / Tt);
            }
            if (n <= cap) atomicMin(&bs.flag, Tt);
        }
        __syncthreads();
        T = min(bs.flag, c_max);
    }
    // rank the sequences by the length of their parts (longest first), count their parts
    int* plen_of = splits + GB_MAX_Z;                // (by batch item, until the ranks are known)
    for (int z = tid; z < Z; z += GA_THREADS) {
        const int c = (bs.n_eff[z] + GA_BN - 1) / GA_BN;
        const int s = max((c + T - 1) / T, 1);
        plen_of[z] = (c + s - 1) / s;
    }
    __syncthreads();
    for (int z = tid; z < Z; z += GA_THREADS) {
        const int plen = plen_of[z];
        int r = 0;
        for (int u = 0; u < Z; ++u) { const int pu = plen_of[u]; r += (pu > plen || (pu == plen && u < z)) ? 1 : 0; }
        const int c = (bs.n_eff[z] + GA_BN - 1) / GA_BN;
        order[r] = z;
        splits[r] = max((c + T - 1) / T, 1);
    }
    __syncthreads();
    if (tid == 0) {
        int run = 0;
        for (int r = 0; r < Z; ++r) {
            bs.prefix[r] = run;
            const int ne = bs.n_eff[order[r]];
            run += H * ((ne + GA_THREADS - 1) / GA_THREADS) * splits[r];
        }
        bs.prefix[Z] = run;
    }
    __syncthreads();
    const int n_parts = bs.prefix[Z];
    // Workgroup -> part.  The parts are numbered longest first, and the first `cap` workgroups are resident together, two
    // per compute unit: workgroup b and workgroup b + cap / 2 share one (the dispatcher gives every compute unit its
    // first workgroup before any gets its second).  The second half takes the parts in reverse, so the longest part is
    // paired with the shortest (or with none): when the short one is done the long one has the unit to itself.
    // The heads keep their pairing (a head of small sigma with one of large sigma, see below).
    // (Only where the parts differ in length: with equal parts, a single sequence, the order of the query tiles is worth
    // more.  cfg 4 x 8 x 4096 padded 146 -> 141 us, 8 x 8 x 2048 padded 109 -> 101, 2 x 8 x 8192 padded 125 -> 119; one
    // sequence of 8192 tokens would lose 2 %.)
    int p = (int)blockIdx.x;
    auto part_len = [&](const int r) { const int c = (bs.n_eff[order[r]] + GA_BN - 1) / GA_BN; return (c + splits[r] - 1) / splits[r]; };
    const bool uneven = part_len(0) != part_len(Z - 1);
    const bool mirrored = uneven && p >= (cap >> 1) && p < cap;
    if (mirrored) p = cap - 1 - (p - (cap >> 1));
    if (p < n_parts) {
        int r = 0;
        while (bs.prefix[r + 1] <= p) ++r;
        r = __builtin_amdgcn_readfirstlane(r);
        const int z = order[r], s = splits[r];
        const int ne = bs.n_eff[z];
        const int c = (ne + GA_BN - 1) / GA_BN, plen = (c + s - 1) / s;
        const int base = bs.prefix[r];
        const int idx = p - base;
        // (the second half of a sequence's parts takes the heads in mirrored order: an XCD, which sees the workgroups
        // whose number is its own modulo 8, then works on a head of small sigma and one of large sigma, few near tiles and many)
        const int rest = idx / H, nq = (ne + GA_THREADS - 1) / GA_THREADS;
        const int h = ((2 * rest >= nq * s) != mirrored) ? H - 1 - idx % H : idx % H;
        const int part = rest % s, qt = rest / s;
        const int zh = z * H + h;
        __syncthreads();                                      // (the tables in the K ring have been read)
        if (s == 1) {
            geo_attn_fwd_pipe_part<false>(bs.pipe, zh, qt, 0, c, ne, nullptr, Q, K, V, coords, sigma, key_pad, O, L, H, N, 1, st);
        } else {
            auto slot_of = [&](const int j) -> float* { return parts + (size_t)(base + (qt * s + j) * H + h) * GB_PART_FLOATS; };
            const int k0 = part * plen, k1 = min(c, k0 + plen);
            const int rc = geo_attn_fwd_pipe_part<true>(bs.pipe, zh, qt, k0, k1, ne, slot_of(part),
                                                        Q, K, V, coords, sigma, key_pad, O, L, H, N, 1, st);
            if (rc == 0) {
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                __syncthreads();
                if (tid == 0) bs.flag = (atomicAdd(&counters[((size_t)z * nqt + qt) * H + h], 1) == s - 1);
                __syncthreads();
                if (bs.flag) gb_merge_parts(slot_of, 0, s - 1, O, L, key_pad, z, h, zh, qt, N, st);
            }
        }
    }

    // ---- query tiles behind the last unpadded token of their sequence: zeros, L = -inf ----
    for (int e = (int)blockIdx.x; e < Z * H * nqt; e += G) {
        const int z = e / (H * nqt), rem = e - z * (H * nqt);
        const int h = rem / nqt, qt = rem - h * nqt;
        if (qt * GA_THREADS < bs.n_eff[z]) continue;
        float* Oh = O + (size_t)z * st.o[0] + (size_t)h * st.o[1];
        const int chunk = tid & 15;
        for (int ql = tid >> 4; ql < GA_THREADS; ql += GA_THREADS / 16) {
            const int qi = qt * GA_THREADS + ql;
            if (qi >= N) break;
            *reinterpret_cast<float4*>(Oh + (size_t)qi * (size_t)st.o[2] + 4 * chunk) = make_float4(0.f, 0.f, 0.f, 0.f);
            if (L && chunk == 0) L[((size_t)z * H + h) * N + qi] = -INFINITY;
        }
    }
}

struct GaVariant { const char* name; };
const GaVariant kVariants[] = { {"auto"}, {"dist_mfma"}, {"dist_valu"}, {"one_block_per_wave"}, {"two_blocks_per_wave"},
                                {"pipelined"}, {"pipelined_dist_mfma"}, {"split_keys"}, {"balanced"}, {"split_items"} };
constexpr int kNumVariants = (int)(sizeof(kVariants) / sizeof(kVariants[0]));

}  // namespace

extern "C" int proteus_geo_attn_num_variants(void) { return kNumVariants; }

extern "C" const char* proteus_geo_attn_variant_name(int tuning) {
    return (tuning >= 0 && tuning < kNumVariants) ? kVariants[tuning].name : nullptr;
}

extern "C" int proteus_geo_attn_fwd_check(const uint16_t* Q, const uint16_t* K, const uint16_t* V,
                                          const float* coords, const float* sigma,
                                          const uint8_t* key_pad_mask,
                                          const float* O, const float* L,
                                          int Z, int H, int N, int d_head, int tuning)
{
    (void)key_pad_mask; (void)L;
    if (!Q || !K || !V || !coords || !sigma || !O) return PROTEUS_ERR_NULL_POINTER;
    if (Z <= 0 || H <= 0 || N <= 0) return PROTEUS_ERR_BAD_SHAPE;
    if (N > PROTEUS_ATTN_MAX_N || (long)Z * H > 65535) return PROTEUS_ERR_BAD_SHAPE;
    if (d_head != 32 && d_head != 64 && d_head != 128) return PROTEUS_ERR_BAD_HEAD_DIM;
    if (tuning < 0 || tuning >= kNumVariants) return PROTEUS_ERR_BAD_TUNING;
    if (((uintptr_t)Q & 15) || ((uintptr_t)K & 15) || ((uintptr_t)V & 15) || ((uintptr_t)O & 15)) return PROTEUS_ERR_BAD_ALIGNMENT;
    return PROTEUS_OK;
}

namespace {
// more than 64 KB of dynamic LDS must be allowed once per kernel and device (remembered for the first 64 devices)
int allow_lds(const void* kernel, size_t bytes, std::atomic<unsigned long long>& allowed) {
    int dev = 0;
    const hipError_t got = hipGetDevice(&dev);
    if (got != hipSuccess) return (int)got;
    if (dev < 0 || dev >= 64 || !((allowed.load(std::memory_order_relaxed) >> dev) & 1ull)) {
        const hipError_t attr = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
        if (attr != hipSuccess) return (int)attr;
        if (dev >= 0 && dev < 64) allowed.fetch_or(1ull << dev, std::memory_order_relaxed);
    }
    return (int)hipSuccess;
}

// Compute units of the current device, looked up once per device.
int device_cus(int* cus_out) {
    static std::atomic<int> cached[64] = {};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    int cus = (dev >= 0 && dev < 64) ? cached[dev].load(std::memory_order_relaxed) : 0;
    if (cus == 0) {
        e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
        if (e != hipSuccess) return (int)e;
        if (cus < 1) cus = 1;
        if (dev >= 0 && dev < 64) cached[dev].store(cus, std::memory_order_relaxed);
    }
    *cus_out = cus;
    return (int)hipSuccess;
}

int launch_attn_pipe(const uint16_t* Q, const uint16_t* K, const uint16_t* V, const float* coords, const float* sigma,
                     const uint8_t* key_pad_mask, float* O, float* L, int Z, int H, int N, bool take_all,
                     const GaStrides& gs, hipStream_t st)
{
    static std::atomic<unsigned long long> allowed{0ull};
    const int rc = allow_lds(reinterpret_cast<const void*>(geo_attn_fwd_pipe_kernel<64>), GA_PIPE_LDS, allowed);
    if (rc != (int)hipSuccess) return rc;
    constexpr int BM = GA_WAVES * 64;
    const int n_qtiles = (N + BM - 1) / BM;
    const int ZH = Z * H;
    const unsigned n_wgs = (unsigned)n_qtiles * (unsigned)ZH;
    hipLaunchKernelGGL(geo_attn_fwd_pipe_kernel<64>, dim3(take_all ? n_wgs : 2 * n_wgs), dim3(GA_THREADS), GA_PIPE_LDS, st,
                       Q, K, V, coords, sigma, key_pad_mask, O, L, H, N, ZH, n_qtiles, (int)n_wgs, take_all ? 1 : 0, gs);
    return (int)hipGetLastError();
}

// Number of persistent workgroups of the balanced launch on the current device: two per compute unit, a multiple of 8
// (one eighth of the line of steps per XCD), at most GB_MAX_WGS.
int balanced_grid(int* G) {
    int cus = 0;
    const int rc = device_cus(&cus);
    if (rc != (int)hipSuccess) return rc;
    int g = 2 * cus;
    if (g > GB_MAX_WGS) g = GB_MAX_WGS;
    g &= ~7;
    if (g < 8) g = 8;
    *G = g;
    return (int)hipSuccess;
}

// Are the schedules that cut items into parts possible for this shape (the pipelined body's head dimension, lengths
// and prefix sums that fit the workgroup's LDS and 31-bit arithmetic)?  From the shape alone.
bool padded_schedules_possible(const uint8_t* key_pad_mask, int Z, int H, int N, int d_head) {
    (void)key_pad_mask;
    if (d_head != GA_D || Z > GB_MAX_Z) return false;
    const long nqt = (N + GA_THREADS - 1) / GA_THREADS, c = (N + GA_BN - 1) / GA_BN;
    return (long)Z * H * nqt * c < (1L << 30);
}

// The balanced schedule (equal shares of steps) runs only where the tuning asks for it.
bool balanced_applies(const uint8_t* key_pad_mask, int Z, int H, int N, int d_head, bool forced) {
    return forced && padded_schedules_possible(key_pad_mask, Z, H, N, d_head);
}

// The split-items schedule is what a padded batch gets by itself when a workspace comes with it and the pipelined
// body is the right one: sequences of at least 1024 tokens and 8192 steps in the dense batch.  Measured against the plain
// grid (which takes the templated body for masked batches up to N = 1024): 4 x 8 x 4096 with lengths 2344-3702
// 164 -> 142 us, 2 x 8 x 8192 (3555, 4019) 165 -> 123 us, 16 x 8 x 1024 (159-1000) 72 -> 65 us, 8 x 8 x 2048 (1180-1985: nothing
// to split) 107 -> 110 us; the encoder's 8 x 8 x 1024 (4096 steps) 34 -> 45 us, hence the threshold.
bool split_applies(const uint8_t* key_pad_mask, int Z, int H, int N, int d_head, bool forced) {
    if (!padded_schedules_possible(key_pad_mask, Z, H, N, d_head)) return false;
    const long nqt = (N + GA_THREADS - 1) / GA_THREADS, c = (N + GA_BN - 1) / GA_BN;
    if (forced) return true;
    // without a mask every item is as long as the others: splitting pays where the items do not fill the chip's
    // workgroup slots (Z = 1, H = 8: N = 4096 98 -> 80 us, N = 8192 256 -> 217 us; Z = 3, N = 3000 163 -> 147 us; N = 2048 48 -> 49 us)
    if (!key_pad_mask) return N > 2048 && (long)Z * H * nqt < GB_MAX_WGS;
    return N >= 1024 && (long)Z * H * nqt * c >= 8192;
}

// The plan and the persistent grid.
int launch_attn_balanced(const uint16_t* Q, const uint16_t* K, const uint16_t* V, const float* coords, const float* sigma,
                         const uint8_t* key_pad_mask, float* O, float* L, void* workspace, int Z, int H, int N,
                         const GaStrides& gs, hipStream_t st)
{
    static std::atomic<unsigned long long> allowed{0ull};
    int rc = allow_lds(reinterpret_cast<const void*>(geo_attn_fwd_balanced_kernel), sizeof(BalSmem), allowed);
    if (rc != (int)hipSuccess) return rc;
    int G = 0;
    rc = balanced_grid(&G);
    if (rc != (int)hipSuccess) return rc;
    const int nqt = (N + GA_THREADS - 1) / GA_THREADS;
    int*   plan  = static_cast<int*>(workspace);
    float* parts = reinterpret_cast<float*>(static_cast<unsigned char*>(workspace) + gb_parts_offset(Z, H, nqt));
    hipLaunchKernelGGL(geo_attn_plan_kernel, dim3(nqt, Z), dim3(GA_THREADS), 0, st, coords, sigma, key_pad_mask, plan, Z, H, N, nqt);
    hipLaunchKernelGGL(geo_attn_fwd_balanced_kernel, dim3(G), dim3(GA_THREADS), sizeof(BalSmem), st,
                       Q, K, V, coords, sigma, key_pad_mask, O, L, plan, parts, Z, H, N, nqt, gs);
    return (int)hipGetLastError();
}

// The plan and the grid of the split-items schedule: one workgroup per part, at least `cap` of them.
int launch_attn_split(const uint16_t* Q, const uint16_t* K, const uint16_t* V, const float* coords, const float* sigma,
                      const uint8_t* key_pad_mask, float* O, float* L, void* workspace, int Z, int H, int N,
                      const GaStrides& gs, hipStream_t st)
{
    static std::atomic<unsigned long long> allowed{0ull};
    int rc = allow_lds(reinterpret_cast<const void*>(geo_attn_fwd_split_kernel), sizeof(BalSmem), allowed);
    if (rc != (int)hipSuccess) return rc;
    int cap = 0;
    rc = balanced_grid(&cap);
    if (rc != (int)hipSuccess) return rc;
    const int nqt = (N + GA_THREADS - 1) / GA_THREADS;
    const long items = (long)Z * H * nqt;
    const unsigned grid = (unsigned)(items > cap ? items : cap);
    int*   plan  = static_cast<int*>(workspace);
    float* parts = reinterpret_cast<float*>(static_cast<unsigned char*>(workspace) + gb_parts_offset(Z, H, nqt));
    hipLaunchKernelGGL(geo_attn_plan_kernel, dim3(nqt, Z), dim3(GA_THREADS), 0, st, coords, sigma, key_pad_mask, plan, Z, H, N, nqt);
    hipLaunchKernelGGL(geo_attn_fwd_split_kernel, dim3(grid), dim3(GA_THREADS), sizeof(BalSmem), st,
                       Q, K, V, coords, sigma, key_pad_mask, O, L, plan, parts, Z, H, N, nqt, cap, gs);
    return (int)hipGetLastError();
}

// d_head and operand type to the kernels.  With two query blocks per wave, d = 64 (here) or 32 (attn_fwd_d32), bf16
// operands and the README logits the software-pipelined kernel runs (automatically for large grids of long sequences,
// or when the tuning asks).
int launch_attn(bool legacy, bool f16, int d_head, const uint16_t* Q, const uint16_t* K, const uint16_t* V, const float* coords,
                const float* sigma, const uint8_t* key_pad_mask, float* O, float* L, int Z, int H, int N, int tuning,
                const float* beta, float min_rbf, float max_rbf, const GaStrides& gs, hipStream_t st,
                void* workspace = nullptr, size_t workspace_bytes = 0)
{
    const bool pipe_tuning = tuning == 5 || tuning == 6 || tuning == 8 || tuning == 9;
    if (d_head == 32)      // (has the pipelined kernel, 5 and 6, but not the schedules over parts)
        return proteus_internal::attn_fwd_d32(legacy, f16, Q, K, V, coords, sigma, key_pad_mask, O, L, Z, H, N, (tuning == 8 || tuning == 9) ? 0 : tuning,
                                              beta, min_rbf, max_rbf, gs, st);
    if (d_head == 128)
        return proteus_internal::attn_fwd_d128(legacy, f16, Q, K, V, coords, sigma, key_pad_mask, O, L, Z, H, N, pipe_tuning ? 0 : tuning,
                                               beta, min_rbf, max_rbf, gs, st);
    // A padded batch with a workspace to exchange partial results in: long items split and handed out longest first
    // (by itself where it pays, see split_applies), or the balanced schedule where the tuning asks for it.
    if (!legacy && workspace && workspace_bytes >= proteus_geo_attn_fwd_workspace_bytes(Z, H, N, d_head, tuning) &&
        proteus_geo_attn_fwd_workspace_bytes(Z, H, N, d_head, tuning) > 0) {
        if ((tuning == 0 || tuning == 9) && split_applies(key_pad_mask, Z, H, N, d_head, tuning == 9))
            return launch_attn_split(Q, K, V, coords, sigma, key_pad_mask, O, L, workspace, Z, H, N, gs, st);
        if (tuning == 8 && balanced_applies(key_pad_mask, Z, H, N, d_head, true))
            return launch_attn_balanced(Q, K, V, coords, sigma, key_pad_mask, O, L, workspace, Z, H, N, gs, st);
    }
    if (tuning == 8 || tuning == 9) tuning = 0;
    // The pipelined kernel pays a longer prologue back from about 16 key tiles per workgroup on, and only where its
    // 256-query workgroups fill most of the chip's 512 slots: measured against the templated body it wins from 416
    // workgroups and N = 1024 on (3-11 %), loses below (up to 384 workgroups the body's 128-query workgroups are faster,
    // see launch_attn_dh; 6-10 % at N = 256 and 512).  A batch that
    // comes with a padding mask is taken to be ragged: up to N = 1024 such a batch runs 12-17 % faster on the body's
    // 128-query workgroups (twice as many, half as long: they even out), so it goes there.
    const long wgs2 = (long)((N + GA_WAVES * 64 - 1) / (GA_WAVES * 64)) * Z * H;
    const bool small_ragged = key_pad_mask != nullptr && N <= 1024 && wgs2 <= 1024;
    if (!legacy && (tuning == 5 || tuning == 6 || (tuning == 0 && wgs2 > 384 && N >= 1024 && !small_ragged)))
        return launch_attn_pipe(Q, K, V, coords, sigma, key_pad_mask, O, L, Z, H, N, tuning == 6, gs, st);
    return launch_attn_dh<64>(legacy, f16, Q, K, V, coords, sigma, key_pad_mask, O, L, Z, H, N, (tuning == 5 || tuning == 6) ? 4 : tuning,
                              beta, min_rbf, max_rbf, gs, st);
}
// contiguous [Z,H,N,d] tensors
GaStrides contiguous_strides(int H, int N, int d) {
    GaStrides gs;
    const long t[3] = {(long)H * N * d, (long)N * d, (long)d};
    for (int i = 0; i < 3; ++i) { gs.q[i] = t[i]; gs.k[i] = t[i]; gs.v[i] = t[i]; gs.o[i] = t[i]; }
    return gs;
}

// strides[12]: (batch, head, token) element strides of Q, K, V, O in this order
int strides_from(const int64_t* strides, int Z, int H, int N, int d, GaStrides& gs) {
    if (!strides) return PROTEUS_ERR_NULL_POINTER;
    long* dst[4] = {gs.q, gs.k, gs.v, gs.o};
    for (int t = 0; t < 4; ++t) {
        const int64_t sz = strides[3 * t], sh = strides[3 * t + 1], sn = strides[3 * t + 2];
        // rows of d contiguous elements that do not overlap and stay 16-byte aligned; a sequence's byte
        // offsets fit the 31 bits of a buffer-load offset
        if (sz < 0 || sh < 0 || sn < d) return PROTEUS_ERR_BAD_LAYOUT;
        const int align = (t == 3) ? 4 : 8;
        if ((sz % align) || (sh % align) || (sn % align)) return PROTEUS_ERR_BAD_ALIGNMENT;
        if ((Z > 1 && sz == 0) || (H > 1 && sh == 0)) return PROTEUS_ERR_BAD_LAYOUT;
        if ((long)N * sn * (t == 3 ? 4 : 2) >= (1L << 31)) return PROTEUS_ERR_BAD_SHAPE;
        dst[t][0] = (long)sz; dst[t][1] = (long)sh; dst[t][2] = (long)sn;
    }
    return PROTEUS_OK;
}
}  // namespace

extern "C" int proteus_geo_attn_fwd_strided_check(const uint16_t* Q, const uint16_t* K, const uint16_t* V,
                                                  const int64_t* strides,
                                                  const float* coords, const float* sigma, const uint8_t* key_pad_mask,
                                                  const float* O, const float* L,
                                                  int Z, int H, int N, int d_head, int tuning)
{
    const int rc = proteus_geo_attn_fwd_check(Q, K, V, coords, sigma, key_pad_mask, O, L, Z, H, N, d_head, tuning);
    if (rc != PROTEUS_OK) return rc;
    GaStrides gs;
    return strides_from(strides, Z, H, N, d_head, gs);
}

extern "C" int proteus_geo_attn_fwd_strided(const uint16_t* Q, const uint16_t* K, const uint16_t* V,
                                            const int64_t* strides,
                                            const float* coords, const float* sigma, const uint8_t* key_pad_mask,
                                            float* O, float* L,
                                            int Z, int H, int N, int d_head, int tuning, void* stream)
{
    int rc = proteus_geo_attn_fwd_check(Q, K, V, coords, sigma, key_pad_mask, O, L, Z, H, N, d_head, tuning);
    if (rc != PROTEUS_OK) return rc;
    GaStrides gs;
    rc = strides_from(strides, Z, H, N, d_head, gs);
    if (rc != PROTEUS_OK) return rc;
    return launch_attn(false, false, d_head, Q, K, V, coords, sigma, key_pad_mask, O, L, Z, H, N, tuning, nullptr, 0.f, 1.f, gs,
                       reinterpret_cast<hipStream_t>(stream));
}

extern "C" int proteus_geo_attn_fwd(const uint16_t* Q, const uint16_t* K, const uint16_t* V,
                                    const float* coords, const float* sigma,
                                    const uint8_t* key_pad_mask,
                                    float* O, float* L,
                                    int Z, int H, int N, int d_head, int tuning, void* stream)
{
    const int rc = proteus_geo_attn_fwd_check(Q, K, V, coords, sigma, key_pad_mask, O, L, Z, H, N, d_head, tuning);
    if (rc != PROTEUS_OK) return rc;
    return launch_attn(false, false, d_head, Q, K, V, coords, sigma, key_pad_mask, O, L, Z, H, N, tuning, nullptr, 0.f, 1.f,
                       contiguous_strides(H, N, d_head), reinterpret_cast<hipStream_t>(stream));
}

extern "C" size_t proteus_geo_attn_fwd_workspace_bytes(int Z, int H, int N, int d_head, int tuning)
{
    if (Z <= 0 || H <= 0 || N <= 0 || N > PROTEUS_ATTN_MAX_N || (long)Z * H > 65535) return 0;
    if (tuning != 0 && tuning != 8 && tuning != 9) return 0;
    // (whether a mask will be passed is not known here: sized as if)
    const uint8_t* some_mask = reinterpret_cast<const uint8_t*>(1);
    if (tuning == 8 ? !balanced_applies(some_mask, Z, H, N, d_head, true)
                    : !(split_applies(some_mask, Z, H, N, d_head, tuning == 9) || split_applies(nullptr, Z, H, N, d_head, tuning == 9))) return 0;
    const int nqt = (N + GA_THREADS - 1) / GA_THREADS;
    return gb_parts_offset(Z, H, nqt) + (size_t)2 * GB_MAX_WGS * GB_PART_FLOATS * sizeof(float);
}

extern "C" int proteus_geo_attn_fwd_ws_check(const uint16_t* Q, const uint16_t* K, const uint16_t* V, const int64_t* strides,
                                             const float* coords, const float* sigma, const uint8_t* key_pad_mask,
                                             const float* O, const float* L, const void* workspace, size_t workspace_bytes,
                                             int Z, int H, int N, int d_head, int tuning)
{
    const int rc = proteus_geo_attn_fwd_check(Q, K, V, coords, sigma, key_pad_mask, O, L, Z, H, N, d_head, tuning);
    if (rc != PROTEUS_OK) return rc;
    if (workspace_bytes != 0 && !workspace) return PROTEUS_ERR_NULL_POINTER;
    if ((uintptr_t)workspace & 255) return PROTEUS_ERR_BAD_ALIGNMENT;
    if (strides) {
        GaStrides gs;
        return strides_from(strides, Z, H, N, d_head, gs);
    }
    return PROTEUS_OK;
}

extern "C" int proteus_geo_attn_fwd_ws(const uint16_t* Q, const uint16_t* K, const uint16_t* V, const int64_t* strides,
                                       const float* coords, const float* sigma, const uint8_t* key_pad_mask,
                                       float* O, float* L, void* workspace, size_t workspace_bytes,
                                       int Z, int H, int N, int d_head, int tuning, void* stream)
{
    int rc = proteus_geo_attn_fwd_ws_check(Q, K, V, strides, coords, sigma, key_pad_mask, O, L, workspace, workspace_bytes,
                                           Z, H, N, d_head, tuning);
    if (rc != PROTEUS_OK) return rc;
    GaStrides gs = contiguous_strides(H, N, d_head);
    if (strides) {
        rc = strides_from(strides, Z, H, N, d_head, gs);
        if (rc != PROTEUS_OK) return rc;
    }
    return launch_attn(false, false, d_head, Q, K, V, coords, sigma, key_pad_mask, O, L, Z, H, N, tuning, nullptr, 0.f, 1.f, gs,
                       reinterpret_cast<hipStream_t>(stream), workspace, workspace_bytes);
}

namespace {
int legacy_args_check(const float* beta, float min_rbf, float max_rbf, int operand_type) {
    if (!beta) return PROTEUS_ERR_NULL_POINTER;
    if (!(max_rbf > min_rbf)) return PROTEUS_ERR_BAD_SHAPE;
    if (operand_type != PROTEUS_OPERAND_BF16 && operand_type != PROTEUS_OPERAND_F16) return PROTEUS_ERR_BAD_OPERAND_TYPE;
    return PROTEUS_OK;
}
}  // namespace

extern "C" int proteus_geo_attn_legacy_fwd(const uint16_t* Q, const uint16_t* K, const uint16_t* V,
                                           const float* coords, const float* sigma, const float* beta,
                                           const uint8_t* key_pad_mask,
                                           float* O, float* L,
                                           int Z, int H, int N, int d_head,
                                           float min_rbf, float max_rbf, int operand_type, int tuning, void* stream)
{
    int rc = proteus_geo_attn_fwd_check(Q, K, V, coords, sigma, key_pad_mask, O, L, Z, H, N, d_head, tuning);
    if (rc != PROTEUS_OK) return rc;
    rc = legacy_args_check(beta, min_rbf, max_rbf, operand_type);
    if (rc != PROTEUS_OK) return rc;
    // a pair mask makes the result sensitive to the last bits of the rbf: use direct distances then
    if ((tuning == 0 || tuning >= 3) && (min_rbf > 0.f || max_rbf < 1.f)) tuning = 2;
    return launch_attn(true, operand_type == PROTEUS_OPERAND_F16, d_head, Q, K, V, coords, sigma, key_pad_mask, O, L, Z, H, N, tuning,
                       beta, min_rbf, max_rbf, contiguous_strides(H, N, d_head), reinterpret_cast<hipStream_t>(stream));
}

extern "C" int proteus_geo_attn_legacy_fwd_strided(const uint16_t* Q, const uint16_t* K, const uint16_t* V,
                                                   const int64_t* strides,
                                                   const float* coords, const float* sigma, const float* beta,
                                                   const uint8_t* key_pad_mask,
                                                   float* O, float* L,
                                                   int Z, int H, int N, int d_head,
                                                   float min_rbf, float max_rbf, int operand_type, int tuning, void* stream)
{
    int rc = proteus_geo_attn_fwd_check(Q, K, V, coords, sigma, key_pad_mask, O, L, Z, H, N, d_head, tuning);
    if (rc != PROTEUS_OK) return rc;
    rc = legacy_args_check(beta, min_rbf, max_rbf, operand_type);
    if (rc != PROTEUS_OK) return rc;
    GaStrides gs;
    rc = strides_from(strides, Z, H, N, d_head, gs);
    if (rc != PROTEUS_OK) return rc;
    if ((tuning == 0 || tuning >= 3) && (min_rbf > 0.f || max_rbf < 1.f)) tuning = 2;
    return launch_attn(true, operand_type == PROTEUS_OPERAND_F16, d_head, Q, K, V, coords, sigma, key_pad_mask, O, L, Z, H, N, tuning,
                       beta, min_rbf, max_rbf, gs, reinterpret_cast<hipStream_t>(stream));
}
