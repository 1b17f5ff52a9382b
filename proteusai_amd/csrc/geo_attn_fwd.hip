// RBF-scaled geometric flash-attention forward for gfx950 (MI355X), d_head = 64.
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
#include <stdint.h>
#include <type_traits>
#include "proteus_hip.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float  floatx16 __attribute__((ext_vector_type(16)));
typedef float  floatx2 __attribute__((ext_vector_type(2)));
typedef short  shortx4 __attribute__((ext_vector_type(4)));
typedef unsigned uint4v __attribute__((ext_vector_type(4)));

constexpr int GA_WAVES   = 4;
constexpr int GA_THREADS = GA_WAVES * 64;
// 32-query blocks per wave: 2 (256 queries per workgroup; every LDS fragment serves both blocks), or 1 for
// grids that would otherwise leave half of the wave slots empty
constexpr int GA_BN      = 64;              // keys per tile
constexpr int GA_D       = 64;              // head dim
constexpr int GA_LDK     = GA_D + 8;        // LDS row stride of the K tile (bf16 elements)
constexpr int GA_LDV     = GA_BN + 4;       // LDS row stride of the V^T tile: 34 dwords, so the 32 rows a half-wave
                                            // reads 8 bytes from fall into 32 different bank pairs
constexpr int GA_LDG     = 40;              // LDS row stride of the key geometry tile (24 used)
constexpr float LOG2E    = 1.4426950408889634f;
// Largest squared distance (scaled units) of a workgroup's queries from their origin for
// which the matrix-core distance path is used.
constexpr float GA_MFMA_DIST_MAX_RHO2 = 1000.0f;
// exp2(-d^2) < 2^-25 for scaled distances d > GA_FAR: s*(1+rbf) then rounds to s in fp32
constexpr float GA_FAR = 5.0f;
// Lazy softmax reference: a block re-bases when the sum of its 16 exponentials per lane passes 2^24 (log2 units)
constexpr float GA_REBASE     = 20.0f;
constexpr float GA_REBASE_SUM = 16777216.0f;

// Element strides (batch, head, token) of Q, K, V (bf16) and O (f32); the head dimension is contiguous.
struct GaStrides { long q[3], k[3], v[3], o[3]; };

// One staged key tile.  Two of them are kept so that the next tile can be written
// while the current one is still being read (one barrier per tile).
struct __align__(16) TileBuf {
    uint16_t k[GA_BN * GA_LDK];      // K tile   [key][d]
    uint16_t vt[GA_D * GA_LDV];      // V^T tile [d][key]
    uint16_t geo[GA_BN * GA_LDG];    // key side of the distance contraction, 24 bf16 per key
    float    cx[GA_BN], cy[GA_BN], cz[GA_BN];   // scaled key coordinates (vector-ALU distance path)
    float    bias[GA_BN];            // 0 for a valid key, -inf for a padded / out-of-range one
    int      flags[4];               // [0] tile has a masked key, [1] tile has a valid key
    int      near[GA_WAVES];         // == tile number + 1 if a key of the tile can matter to wave w's multiplier
};

struct __align__(16) Smem {
    TileBuf  tile[2];
    float4   sphere[GA_WAVES];       // per wave: centre of its queries (scaled frame) and (GA_FAR + radius)^2
    int      n_eff;                  // 1 + index of the last valid key of this batch item
    unsigned rho2_bits;              // max |scaled query|^2 over the workgroup (bits of a non-negative float)
    int      q_first, q_last;        // first / last unpadded query of the workgroup
};

// Exchange between the two half-waves: lane l and lane l^32 hold the same query.
// v_permlane32_swap exchanges lanes 32..63 of its first register with lanes 0..31
// of its second; starting from two copies of x, the first ends up holding the
// low half's value in every lane and the second the high half's.  (Written as
// inline assembly: the compiler builtin folds the two results of identical
// inputs into one.)
__device__ __forceinline__ void xhalf_both(float x, float& lo, float& hi) {
    lo = x; hi = x;
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(lo), "+v"(hi));
}
__device__ __forceinline__ float xhalf_max(float x) { float a, b; xhalf_both(x, a, b); return fmaxf(a, b); }
__device__ __forceinline__ float xhalf_sum(float x) { float a, b; xhalf_both(x, a, b); return a + b; }

__device__ __forceinline__ unsigned pack_bf16(float a, float b) {
    floatx2 f = {a, b};
    return __builtin_bit_cast(unsigned, __builtin_convertvector(f, bf16x2));
}

// c + the two bf16 values packed in w (v_dot2_f32_bf16 against ones).  The softmax row sum is taken over the
// probabilities AS THE P.V PRODUCT SEES THEM (rounded to bf16), so O is a convex combination of V rows to fp32
// rounding and D = rowsum(O dO) cancels against dP in the backward the way the exact quantities do.
__device__ __forceinline__ float add_packed_bf16(const unsigned w, const float c) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, w), __builtin_bit_cast(bf16x2, 0x3f803f80u), c, false);
}

// a = h + m + l with h, m, l representable in bf16 (exact for any finite float whose pieces do not underflow)
__device__ __forceinline__ void split3(float a, float& h, float& m, float& l) {
    h = (float)(__bf16)a;
    const float r1 = a - h;
    m = (float)(__bf16)r1;
    l = (float)(__bf16)(r1 - m);
}

// DIST_VALU selects how the distances are evaluated: false = on the matrix cores, true = directly on
// the vector ALU.  Unless take_all is set both bodies are run for every group of queries (by two
// workgroups of one launch): a group is computed with the matrix-core distances if its queries lie
// within GA_MFMA_DIST_MAX_RHO2 of their origin and with the direct ones otherwise, and the body that
// does not own it returns after the prologue.
// LEGACY selects the logits of the reference's Triton kernel instead of the README multiplier:
//   s = S + beta_h * (2 (rbf - min_rbf)/(max_rbf - min_rbf) - 1) * |S|, pairs with rbf outside [min_rbf, max_rbf] masked
//   (old/old_scripts/attn/geometric_attn.py:193-201).
template <bool DIST_VALU, bool LEGACY, int GA_QB>
__device__ __forceinline__
void geo_attn_fwd_body(Smem& sm, const int block_id,
                       const uint16_t* __restrict__ Q, const uint16_t* __restrict__ K,
                       const uint16_t* __restrict__ V, const float* __restrict__ coords,
                       const float* __restrict__ sigma, const uint8_t* __restrict__ key_pad,
                       float* __restrict__ O, float* __restrict__ L,
                       const int H, const int N, const int ZH, const int n_qtiles, const int take_all,
                       const float* __restrict__ beta, const float min_rbf, const float max_rbf, const GaStrides& st)
{

    const int tid  = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int half = lane >> 5;          // which 4-row group of every 8 accumulator rows
    const int col  = lane & 31;          // accumulator column = query within a block

    // Workgroup -> (query tile, batch*head).  Consecutive workgroup ids go round-robin over the
    // 8 XCDs.  Each XCD owns ZH/8 (batch, head) pairs for the first half of the query tiles and the
    // mirrored pairs (ZH-1-zh) for the second half: the K and V an XCD touches at any time stay
    // few enough for its L2, and a head whose sigma makes the multiplier matter for many tiles is
    // paired with one for which it matters for few, so the XCDs finish together.
    int zh, qt;
    {
        const int id = block_id;
        if ((ZH & 7) == 0) {
            const int per_xcd = ZH >> 3;
            const int r = id >> 3;
            zh = (id & 7) + 8 * (r % per_xcd);
            qt = r / per_xcd;
            if (2 * qt >= n_qtiles) zh = ZH - 1 - zh;
        } else {
            zh = id % ZH;
            qt = id / ZH;
        }
    }
    const int z  = zh / H;
    const int h  = zh - z * H;
    const uint16_t* Qh = Q + (size_t)z * st.q[0] + (size_t)h * st.q[1];
    const uint16_t* Kh = K + (size_t)z * st.k[0] + (size_t)h * st.k[1];
    const uint16_t* Vh = V + (size_t)z * st.v[0] + (size_t)h * st.v[1];
    float*          Oh = O + (size_t)z * st.o[0] + (size_t)h * st.o[1];
    const size_t q_pitch = (size_t)st.q[2], o_pitch = (size_t)st.o[2];
    const int    k_pitch = (int)st.k[2] * 2, v_pitch = (int)st.v[2] * 2;      // bytes; N * pitch fits 31 bits (checked on the host)
    const float*    cz = coords + (size_t)z * N * 3;
    const uint8_t*  mz = key_pad ? key_pad + (size_t)z * N : nullptr;

    const float sg = sigma[h];
    // exp(-d^2/(2 sg^2)) = exp2(-(d*cs)^2) with cs = sqrt(log2(e)/2)/sg
    const float cscale = 0.84932180028801907f / sg;
    // legacy logits: beta * rbf_norm = rbf * lg_a + lg_b
    const float lg_beta = LEGACY ? beta[h] : 0.f;
    const float lg_a = LEGACY ? 2.0f * lg_beta / (max_rbf - min_rbf) : 0.f;
    const float lg_b = LEGACY ? -lg_beta * (2.0f * min_rbf / (max_rbf - min_rbf) + 1.0f) : 0.f;
    if (tid == 0) { sm.n_eff = mz ? 0 : N; sm.rho2_bits = 0u; sm.q_first = 0x7fffffff; sm.q_last = -1; }
    __syncthreads();

    // ---- this lane's queries: one per block ----
    constexpr int GA_BM = GA_WAVES * 32 * GA_QB;          // queries per workgroup
    const int qbase = qt * GA_BM + wave * (32 * GA_QB);
    int   q[GA_QB];
    bool  q_in[GA_QB], q_ok[GA_QB];
#pragma unroll
    for (int b = 0; b < GA_QB; ++b) {
        q[b]    = qbase + 32 * b + col;
        q_in[b] = q[b] < N;
        q_ok[b] = q_in[b] && !(mz && mz[q[b]]);
    }
    // first and last unpadded query of the workgroup (wave-level reduction, then one LDS atomic each)
    int wave_first, wave_last;
    {
        int lo = 0x7fffffff, hi = -1;
#pragma unroll
        for (int b = 0; b < GA_QB; ++b) if (q_ok[b]) { lo = min(lo, q[b]); hi = max(hi, q[b]); }
        for (int o = 32; o > 0; o >>= 1) { lo = min(lo, __shfl_xor(lo, o)); hi = max(hi, __shfl_xor(hi, o)); }
        if (lane == 0) { atomicMin(&sm.q_first, lo); atomicMax(&sm.q_last, hi); }
        wave_first = lo; wave_last = hi;
    }
    __syncthreads();
    const int q_first = sm.q_first, q_last = sm.q_last;
    if (q_last < 0) {
        // every query of this workgroup is padded (or out of range): zeros, L = -inf, done
        if (take_all || DIST_VALU) {      // exactly one of the two bodies writes them
#pragma unroll
            for (int b = 0; b < GA_QB; ++b) {
                if (!q_in[b]) continue;
                float* orow = Oh + (size_t)q[b] * o_pitch;
#pragma unroll
                for (int g = 0; g < 8; ++g)
                    *reinterpret_cast<float4*>(orow + 8 * g + 4 * half) = make_float4(0.f, 0.f, 0.f, 0.f);
                if (L && half == 0) L[(size_t)zh * N + q[b]] = -INFINITY;
            }
        }
        return;
    }
    // Origin of the scaled frame: midway between the first and the last unpadded query of the
    // workgroup.  Only unpadded tokens enter it (and the radius below), so whatever sits in padded
    // positions cannot change which code path, and hence which rounding, the valid rows see.
    const float ox = 0.5f * (cz[3 * q_first] + cz[3 * q_last]);
    const float oy = 0.5f * (cz[3 * q_first + 1] + cz[3 * q_last + 1]);
    const float oz = 0.5f * (cz[3 * q_first + 2] + cz[3 * q_last + 2]);
    const int q_mirror = (wave_first != 0x7fffffff) ? wave_first : q_first;
    // With the reference's logits on the direct-distance path the rbf decides a pair mask, so it is evaluated
    // exactly as the backward kernel evaluates it (raw coordinates, exp2(-d^2 cs2), same operation order): a pair is
    // then in range in both or in neither.
    constexpr bool RAW_DIST = LEGACY && DIST_VALU;
    const float cs2 = 0.72134752044448170368f / (sg * sg);       // log2(e)/2 / sigma^2
    float qx[GA_QB], qy[GA_QB], qz[GA_QB], qn2[GA_QB];
    float qrx[GA_QB], qry[GA_QB], qrz[GA_QB];
#pragma unroll
    for (int b = 0; b < GA_QB; ++b) {
        const int qc = q_ok[b] ? q[b] : q_mirror;      // a padded lane mirrors a valid query: finite, in-range data
        qrx[b] = cz[3 * qc]; qry[b] = cz[3 * qc + 1]; qrz[b] = cz[3 * qc + 2];
        qx[b] = (qrx[b] - ox) * cscale; qy[b] = (qry[b] - oy) * cscale; qz[b] = (qrz[b] - oz) * cscale;
        qn2[b] = qx[b] * qx[b] + qy[b] * qy[b] + qz[b] * qz[b];
    }
    {
        float qn2max = 0.f;
#pragma unroll
        for (int b = 0; b < GA_QB; ++b) qn2max = fmaxf(qn2max, qn2[b]);
        atomicMax(&sm.rho2_bits, __builtin_bit_cast(unsigned, qn2max));
    }

    // ---- sphere around this wave's queries, for the far-tile test ----
    {
        // centre: midway between the wave's first and last unpadded query (the workgroup's, if it has none)
        const int   qa = q_mirror, qb = (wave_last >= 0) ? wave_last : q_first;
        const float wx = (0.5f * (cz[3 * qa] + cz[3 * qb]) - ox) * cscale;
        const float wy = (0.5f * (cz[3 * qa + 1] + cz[3 * qb + 1]) - oy) * cscale;
        const float wz = (0.5f * (cz[3 * qa + 2] + cz[3 * qb + 2]) - oz) * cscale;
        float r2 = 0.f;
#pragma unroll
        for (int b = 0; b < GA_QB; ++b) {
            const float dx = qx[b] - wx, dy = qy[b] - wy, dz = qz[b] - wz;
            r2 = fmaxf(r2, dx * dx + dy * dy + dz * dz);
        }
        for (int o = 32; o > 0; o >>= 1) r2 = fmaxf(r2, __shfl_xor(r2, o));
        const float t = GA_FAR + __builtin_sqrtf(r2) * 1.0001f;
        if (lane == 0) sm.sphere[wave] = make_float4(wx, wy, wz, t * t);
    }

    // ---- 1 + index of the last unpadded key: trailing padded tiles are never visited ----
    if (mz) {
        int last = 0;
        for (int j = tid; j < N; j += GA_THREADS) if (!mz[j]) last = j + 1;
        for (int o = 32; o > 0; o >>= 1) last = max(last, __shfl_xor(last, o));
        if (lane == 0) atomicMax(&sm.n_eff, last);
    }
    __syncthreads();
    const int  n_eff = sm.n_eff;
    constexpr bool use_mfma_dist = !DIST_VALU;
    if (!take_all) {
        const bool compact = __builtin_bit_cast(float, sm.rho2_bits) <= GA_MFMA_DIST_MAX_RHO2;
        if (compact == DIST_VALU) return;       // the other instantiation owns this workgroup
    }

    // Q^T as the B operand: lane (half, col) holds d = 16*ks + 8*half + 0..7 of its query,
    // pre-multiplied by 1/sqrt(64) = 2^-3 (exact in bf16)
    bf16x8 qreg[GA_QB][4];
#pragma unroll
    for (int b = 0; b < GA_QB; ++b) {
        const int qc = q_ok[b] ? q[b] : q_mirror;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            const uint4 raw = *reinterpret_cast<const uint4*>(Qh + (size_t)qc * q_pitch + ks * 16 + half * 8);
            bf16x8 v = __builtin_bit_cast(bf16x8, raw);
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = (__bf16)((float)v[e] * 0.125f);
            qreg[b][ks] = v;
        }
    }

    // Query side of the distance contraction.  Slot s of the 24:
    //   6c+{0..5}, c = x,y,z : key pieces (h,h,m,m,h,l) against query pieces 2*(h,m,h,m,l,h)
    //   18..20 : key -|x'_k|^2 pieces (h,m,l) against 1
    //   21..23 : 1 against query -|x'_q|^2 pieces (h,m,l)
    // First MFMA (K=16): half-wave hf holds slots 8*hf+0..7; second (K=8): slots 16+4*hf+0..3.
    uint4 gq0[GA_QB];
    uint2 gq1[GA_QB];
#pragma unroll
    for (int b = 0; b < GA_QB; ++b) {
        float xh, xm, xl, yh, ym, yl, zh_, zm, zl, nh, nm, nl;
        split3(2.0f * qx[b], xh, xm, xl);
        split3(2.0f * qy[b], yh, ym, yl);
        split3(2.0f * qz[b], zh_, zm, zl);
        split3(-qn2[b], nh, nm, nl);
        // slots 0..7: x(h,m,h,m,l,h) y(h,m)      slots 8..15: y(h,m,l,h) z(h,m,h,m)
        // slots 16..19: z(l,h) 1 1                slots 20..23: 1 n(h,m,l)
        if (half == 0) {
            gq0[b] = make_uint4(pack_bf16(xh, xm), pack_bf16(xh, xm), pack_bf16(xl, xh), pack_bf16(yh, ym));
            gq1[b] = make_uint2(pack_bf16(zl, zh_), pack_bf16(1.f, 1.f));
        } else {
            gq0[b] = make_uint4(pack_bf16(yh, ym), pack_bf16(yl, yh), pack_bf16(zh_, zm), pack_bf16(zh_, zm));
            gq1[b] = make_uint2(pack_bf16(1.f, nh), pack_bf16(nm, nl));
        }
    }

    // Online softmax with a LAZY reference: p = exp(s - m2) where m2 is the maximum the query had seen when
    // it was last re-based, not the running maximum.  A block re-bases (exact maximum, rescale of O and l) only
    // if a query has nothing accumulated yet or one of its exponentials passed 2^GA_REBASE; everywhere else
    // no maximum is taken at all, and -m2 enters the score product itself as one more contraction slot
    // (-m2 split exactly into three bf16 pieces against ones), so the accumulator times log2(e) is the exponent.
    floatx16 oacc[GA_QB][2];
    float m2[GA_QB], l_run[GA_QB];
    uint2 moff[GA_QB];           // B operand of the offset product: slots 0..2 = pieces of -m2 (half-wave 0 only)
#pragma unroll
    for (int b = 0; b < GA_QB; ++b) {
#pragma unroll
        for (int dt = 0; dt < 2; ++dt)
#pragma unroll
            for (int r = 0; r < 16; ++r) oacc[b][dt][r] = 0.f;
        m2[b] = 0.f;             // reference of the exponentials (natural units), same in both half-waves
        l_run[b] = 0.f;          // this half-wave's part of the running sum
        moff[b] = make_uint2(0u, 0u);
    }
    const unsigned ones2 = 0x3f803f80u;      // bf16 (1, 1)
    float log2e = LOG2E;                     // kept in a vector register: an all-register multiply issues faster
    asm volatile("" : "+v"(log2e));

    // staging roles
    const int kp   = tid & 31;   // V: key pair
    const int vdc  = tid >> 5;   // V: 8-wide d chunk
    const int krow = tid >> 3;   // K: key row (0..31, +32 on the second pass)
    const int kdc  = tid & 7;    // K: 8-wide d chunk
    const int gkey = tid >> 2;   // geometry: key
    const int gcmp = tid & 3;    // geometry: x, y, z, -norm^2; far test: against wave gcmp's sphere

    // registers holding the tile in flight from global memory.  load_tile only ISSUES loads; nothing
    // it fetches is touched until store_tile, one tile of computation later, so the wait for them
    // lands there.  Buffer loads: base in SGPRs, one 32-bit lane offset, and reads past the end of a
    // tensor return zeros (no bounds branches on the last tile).
    uint4v kreg[2], vreg[2];
    uint4v graw = {0u, 0u, 0u, 0u};         // raw key coordinates (x, y, z and one dword beyond)
    unsigned mbyte = 0;                     // raw padding byte of key tid (threads < 64)
    unsigned mk0 = 0, mk1 = 0, mv0 = 0, mv1 = 0, mg = 0;   // raw padding bytes of the keys this thread stages
    int loaded_j0 = 0;
    // the range ends with the last row, so rows past the end of the sequence read as zeros whatever lies behind them
    const __amdgpu_buffer_rsrc_t rK = __builtin_amdgcn_make_buffer_rsrc((void*)Kh, 0, (N - 1) * k_pitch + GA_D * 2, 0x00020000);
    const __amdgpu_buffer_rsrc_t rV = __builtin_amdgcn_make_buffer_rsrc((void*)Vh, 0, (N - 1) * v_pitch + GA_D * 2, 0x00020000);
    const __amdgpu_buffer_rsrc_t rC = __builtin_amdgcn_make_buffer_rsrc((void*)cz, 0, N * 12, 0x00020000);
    const __amdgpu_buffer_rsrc_t rM = __builtin_amdgcn_make_buffer_rsrc((void*)(mz ? mz : key_pad), 0, mz ? N : 0, 0x00020000);
    const int koff = krow * k_pitch + kdc * 16;              // byte offsets inside a tile
    const int voff = 2 * kp * v_pitch + vdc * 16;
    const int goff = 12 * gkey;

    auto load_tile = [&](const int j0) {
        loaded_j0 = j0;
        // the tile offset goes into the lane offset, not the scalar offset: only the former is range-checked
        kreg[0] = __builtin_amdgcn_raw_buffer_load_b128(rK, koff + j0 * k_pitch, 0, 0);
        kreg[1] = __builtin_amdgcn_raw_buffer_load_b128(rK, koff + (j0 + 32) * k_pitch, 0, 0);
        vreg[0] = __builtin_amdgcn_raw_buffer_load_b128(rV, voff + j0 * v_pitch, 0, 0);
        vreg[1] = __builtin_amdgcn_raw_buffer_load_b128(rV, voff + (j0 + 1) * v_pitch, 0, 0);
        graw    = __builtin_amdgcn_raw_buffer_load_b128(rC, goff + j0 * 12, 0, 0);
        if (mz) {
            mbyte = __builtin_amdgcn_raw_buffer_load_b8(rM, lane + j0, 0, 0);      // used by wave 0 only
            mk0 = __builtin_amdgcn_raw_buffer_load_b8(rM, krow + j0, 0, 0);
            mk1 = __builtin_amdgcn_raw_buffer_load_b8(rM, krow + 32 + j0, 0, 0);
            mv0 = __builtin_amdgcn_raw_buffer_load_b8(rM, 2 * kp + j0, 0, 0);
            mv1 = __builtin_amdgcn_raw_buffer_load_b8(rM, 2 * kp + 1 + j0, 0, 0);
            mg  = __builtin_amdgcn_raw_buffer_load_b8(rM, gkey + j0, 0, 0);
        }
    };

    auto store_tile = [&](TileBuf& tb, const int tile_id) {
        // (elements are copied to scalars first: bit-casting a vector element expression directly reads element 0)
        const unsigned rx = graw[0], ry = graw[1], rz = graw[2];
        float gx = (__builtin_bit_cast(float, rx) - ox) * cscale;
        float gy = (__builtin_bit_cast(float, ry) - oy) * cscale;
        float gz = (__builtin_bit_cast(float, rz) - oz) * cscale;
        if (mz) {
            // whatever a padded key holds (even NaN) is replaced by zeros: everything downstream stays
            // finite and the -inf bias alone removes the key
            if (mk0) kreg[0] = uint4v{0u, 0u, 0u, 0u};
            if (mk1) kreg[1] = uint4v{0u, 0u, 0u, 0u};
            if (mv0) vreg[0] = uint4v{0u, 0u, 0u, 0u};
            if (mv1) vreg[1] = uint4v{0u, 0u, 0u, 0u};
            if (mg) { gx = 0.f; gy = 0.f; gz = 0.f; }
        }
        if (loaded_j0 + gkey >= N) { gx = 0.f; gy = 0.f; gz = 0.f; }
        const bool kvalid = (loaded_j0 + tid < N) && (mbyte == 0);
        *reinterpret_cast<uint4v*>(&tb.k[krow * GA_LDK + kdc * 8]) = kreg[0];
        *reinterpret_cast<uint4v*>(&tb.k[(krow + 32) * GA_LDK + kdc * 8]) = kreg[1];
        {
            const unsigned a[4] = {vreg[0][0], vreg[0][1], vreg[0][2], vreg[0][3]};
            const unsigned b[4] = {vreg[1][0], vreg[1][1], vreg[1][2], vreg[1][3]};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                // V^T[d][key pair]: low half-word = even key, high half-word = odd key
                const unsigned lo = __builtin_amdgcn_perm(b[e], a[e], 0x05040100u);
                const unsigned hi = __builtin_amdgcn_perm(b[e], a[e], 0x07060302u);
                *reinterpret_cast<unsigned*>(&tb.vt[(vdc * 8 + 2 * e) * GA_LDV + 2 * kp]) = lo;
                *reinterpret_cast<unsigned*>(&tb.vt[(vdc * 8 + 2 * e + 1) * GA_LDV + 2 * kp]) = hi;
            }
        }
        {
            // far test of this thread's key against the sphere of wave gcmp; the flag holds the tile
            // number + 1, so it never needs clearing
            const float4 sph = sm.sphere[gcmp];
            const float dx = gx - sph.x, dy = gy - sph.y, dz = gz - sph.z;
            const uint64_t bal = __builtin_amdgcn_ballot_w64(dx * dx + dy * dy + dz * dz <= sph.w);
            if (lane == 0) {
#pragma unroll
                for (int w = 0; w < GA_WAVES; ++w)
                    if (bal & (0x1111111111111111ull << w)) tb.near[w] = tile_id + 1;
            }
        }
        if (use_mfma_dist) {
            // the four threads of a key write the pieces of x, y, z and -|x'|^2 (6 slots = 12 bytes each)
            const float a = (gcmp == 0) ? gx : (gcmp == 1) ? gy : (gcmp == 2) ? gz : -(gx * gx + gy * gy + gz * gz);
            float hh, mm, ll;
            split3(a, hh, mm, ll);
            unsigned w0, w1, w2;
            if (gcmp < 3) { w0 = pack_bf16(hh, hh); w1 = pack_bf16(mm, mm); w2 = pack_bf16(hh, ll); }
            else          { w0 = pack_bf16(hh, mm); w1 = pack_bf16(ll, 1.f); w2 = pack_bf16(1.f, 1.f); }
            unsigned* dst = reinterpret_cast<unsigned*>(&tb.geo[gkey * GA_LDG + 6 * gcmp]);
            dst[0] = w0; dst[1] = w1; dst[2] = w2;
        } else if (gcmp == 0) {
            if (RAW_DIST) {
                const bool gone = (mz && mg) || (loaded_j0 + gkey >= N);
                tb.cx[gkey] = gone ? 0.f : __builtin_bit_cast(float, rx);
                tb.cy[gkey] = gone ? 0.f : __builtin_bit_cast(float, ry);
                tb.cz[gkey] = gone ? 0.f : __builtin_bit_cast(float, rz);
            } else {
                tb.cx[gkey] = gx; tb.cy[gkey] = gy; tb.cz[gkey] = gz;
            }
        }
        if (tid < GA_BN) {
            tb.bias[tid] = kvalid ? 0.f : -INFINITY;
            const uint64_t bal = __builtin_amdgcn_ballot_w64(kvalid);
            if (tid == 0) { tb.flags[0] = (bal != ~0ull); tb.flags[1] = (bal != 0ull); }
        }
    };

    auto apply_rbf = [&](const float sv, float rbf) -> float {
        if (!LEGACY) return __builtin_fmaf(sv, rbf, sv);
        rbf = fminf(rbf, 1.0f);          // the matrix-core distance can come out a rounding error below zero
        const float t = __builtin_fmaf(__builtin_fmaf(rbf, lg_a, lg_b), fabsf(sv), sv);
        return (rbf >= min_rbf && rbf <= max_rbf) ? t : -INFINITY;
    };

    // multiplier, mask, exponentials of one 32-key x 32-query block; returns P^T packed for the two
    // K=16 steps.  Accumulator register r of key block mt is key  mt*32 + 8*(r/4) + 4*half + (r%4).
    // On entry sacc holds s (natural units) for a near block and s - m2 for a far one; it is turned into the
    // exponent (s' - m2) log2(e) first.
    auto softmax_block = [&](const TileBuf& tb, const int mt, const int b, floatx16& sacc, const floatx16& dacc,
                             const bool has_masked, const bool near, uint4 (&pb)[2]) {
        if (near) {
            const float mneg = -m2[b] * log2e;
            if (use_mfma_dist) {
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    sacc[r] = __builtin_fmaf(apply_rbf(sacc[r], __builtin_amdgcn_exp2f(dacc[r])), log2e, mneg);
            } else {
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int kb0 = mt * 32 + 8 * g + 4 * half;
                    const float4 kx = *reinterpret_cast<const float4*>(&tb.cx[kb0]);
                    const float4 ky = *reinterpret_cast<const float4*>(&tb.cy[kb0]);
                    const float4 kz = *reinterpret_cast<const float4*>(&tb.cz[kb0]);
                    const float kxs[4] = {kx.x, kx.y, kx.z, kx.w};
                    const float kys[4] = {ky.x, ky.y, ky.z, ky.w};
                    const float kzs[4] = {kz.x, kz.y, kz.z, kz.w};
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        float rbf;
                        if (RAW_DIST) {
                            const float dx = qrx[b] - kxs[v], dy = qry[b] - kys[v], dz = qrz[b] - kzs[v];
                            const float d2 = __builtin_fmaf(dz, dz, __builtin_fmaf(dy, dy, dx * dx));
                            rbf = __builtin_amdgcn_exp2f(-d2 * cs2);
                        } else {
                            const float dx = qx[b] - kxs[v], dy = qy[b] - kys[v], dz = qz[b] - kzs[v];
                            const float d2 = dx * dx + dy * dy + dz * dz;
                            rbf = __builtin_amdgcn_exp2f(-d2);
                        }
                        sacc[4 * g + v] = __builtin_fmaf(apply_rbf(sacc[4 * g + v], rbf), log2e, mneg);
                    }
                }
            }
        } else {
#pragma unroll
            for (int r = 0; r < 16; ++r) sacc[r] *= log2e;
        }
        if (has_masked) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const float4 bb = *reinterpret_cast<const float4*>(&tb.bias[mt * 32 + 8 * g + 4 * half]);
                sacc[4 * g + 0] += bb.x; sacc[4 * g + 1] += bb.y; sacc[4 * g + 2] += bb.z; sacc[4 * g + 3] += bb.w;
            }
        }
        float lsum = 0.f;
        auto exponentials = [&]() {
            lsum = 0.f;
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                // contraction slot e of this half-wave is key mt*32 + 16*t + 8*(e/4) + 4*half + (e%4)
                float p[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) p[e] = __builtin_amdgcn_exp2f(sacc[8 * t + e]);
                pb[t] = make_uint4(pack_bf16(p[0], p[1]), pack_bf16(p[2], p[3]), pack_bf16(p[4], p[5]), pack_bf16(p[6], p[7]));
                lsum = add_packed_bf16(pb[t].x, lsum); lsum = add_packed_bf16(pb[t].y, lsum);
                lsum = add_packed_bf16(pb[t].z, lsum); lsum = add_packed_bf16(pb[t].w, lsum);
            }
        };
        exponentials();
        // re-base where a query has nothing yet (first contact) or an exponential ran away; +inf is caught too
        if (__builtin_amdgcn_ballot_w64(!(lsum <= GA_REBASE_SUM) || l_run[b] == 0.f) != 0) {
            float tmax = sacc[0];
#pragma unroll
            for (int r = 1; r < 16; ++r) tmax = fmaxf(tmax, sacc[r]);
            tmax = xhalf_max(tmax);
            const float l_tot = xhalf_sum(l_run[b]);
            float delta = 0.f;                          // by how much this query's reference moves (log2 units)
            if (tmax != -INFINITY && (l_tot == 0.f || tmax > GA_REBASE)) delta = tmax;
            // a query without anything accumulated has nothing to rescale (and its delta may be hugely negative)
            const float alpha = (l_tot == 0.f) ? 1.0f : __builtin_amdgcn_exp2f(-delta);
#pragma unroll
            for (int dt = 0; dt < 2; ++dt)
#pragma unroll
                for (int r = 0; r < 16; ++r) oacc[b][dt][r] *= alpha;
            l_run[b] *= alpha;
            m2[b] = __builtin_fmaf(delta, 0.69314718055994531f, m2[b]);
#pragma unroll
            for (int r = 0; r < 16; ++r) sacc[r] -= delta;
            exponentials();
            float oh, om, ol;
            split3(-m2[b], oh, om, ol);
            moff[b] = (half == 0) ? make_uint2(pack_bf16(oh, om), pack_bf16(ol, 0.f)) : make_uint2(0u, 0u);
        }
        l_run[b] += lsum;
    };

    // LDS -> register fragment loads, issued well ahead of the matrix instructions that consume them
    auto load_kf = [&](const TileBuf& tb, const int mt, uint4 (&kf)[4]) {
#pragma unroll
        for (int ks = 0; ks < 4; ++ks)
            kf[ks] = *reinterpret_cast<const uint4*>(&tb.k[(mt * 32 + col) * GA_LDK + ks * 16 + half * 8]);
    };
    auto load_vf = [&](const TileBuf& tb, const int mt, const int t, uint4 (&vf)[2]) {
#pragma unroll
        for (int dt = 0; dt < 2; ++dt) {
            const uint16_t* row = &tb.vt[(dt * 32 + col) * GA_LDV + mt * 32 + 16 * t + 4 * half];
            const uint2 a0 = *reinterpret_cast<const uint2*>(row);
            const uint2 a1 = *reinterpret_cast<const uint2*>(row + 8);
            vf[dt] = make_uint4(a0.x, a0.y, a1.x, a1.y);
        }
    };

    // One 32-key block of the staged tile against both query blocks.  kf holds this block's K fragments on
    // entry; if `more`, it is refilled with the next block's right after the score products have consumed it, so
    // those reads (and the first V^T fragments) are in flight during the exponentials.
    auto key_block = [&](const TileBuf& tb, const int mt, const bool has_masked, const bool near, uint4 (&kf)[4], const bool more) {
        floatx16 sacc[GA_QB];
#pragma unroll
        for (int b = 0; b < GA_QB; ++b) {
#pragma unroll
            for (int r = 0; r < 16; ++r) sacc[b][r] = 0.f;
#pragma unroll
            for (int ks = 0; ks < 4; ++ks)
                sacc[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, kf[ks]), qreg[b][ks], sacc[b], 0, 0, 0);
            if (!near)      // s - m2 straight from the matrix cores: ones against the pieces of -m2
                sacc[b] = __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(__builtin_bit_cast(shortx4, make_uint2(ones2, ones2)),
                                                                   __builtin_bit_cast(shortx4, moff[b]), sacc[b], 0, 0, 0);
        }
        uint4 g0 = make_uint4(0, 0, 0, 0);
        uint2 g1 = make_uint2(0, 0);
        if (near && use_mfma_dist) {
            const uint16_t* grow = &tb.geo[(mt * 32 + col) * GA_LDG];
            g0 = *reinterpret_cast<const uint4*>(grow + 8 * half);
            g1 = *reinterpret_cast<const uint2*>(grow + 16 + 4 * half);
        }
        (void)more;
        uint4 pb[GA_QB][2];
#pragma unroll
        for (int b = 0; b < GA_QB; ++b) {
            floatx16 dacc = {};
            if (near && use_mfma_dist) {
#pragma unroll
                for (int r = 0; r < 16; ++r) dacc[r] = 0.f;
                dacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, g0), __builtin_bit_cast(bf16x8, gq0[b]), dacc, 0, 0, 0);
                dacc = __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(__builtin_bit_cast(shortx4, g1), __builtin_bit_cast(shortx4, gq1[b]), dacc, 0, 0, 0);
            }
            softmax_block(tb, mt, b, sacc[b], dacc, has_masked, near, pb[b]);
        }
        // every V^T fragment read from LDS serves both query blocks
        if (more) load_kf(tb, mt + 1, kf);
        uint4 vf0[2], vf1[2];
        load_vf(tb, mt, 0, vf0);
        load_vf(tb, mt, 1, vf1);
#pragma unroll
        for (int dt = 0; dt < 2; ++dt)
#pragma unroll
            for (int b = 0; b < GA_QB; ++b)
                oacc[b][dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, vf0[dt]), __builtin_bit_cast(bf16x8, pb[b][0]), oacc[b][dt], 0, 0, 0);
#pragma unroll
        for (int dt = 0; dt < 2; ++dt)
#pragma unroll
            for (int b = 0; b < GA_QB; ++b)
                oacc[b][dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, vf1[dt]), __builtin_bit_cast(bf16x8, pb[b][1]), oacc[b][dt], 0, 0, 0);
    };

    // ---- key loop: tile t is computed from LDS while tile t+1 travels global -> registers -> the other LDS buffer ----
    const int ntiles = (n_eff + GA_BN - 1) / GA_BN;
    if (tid < GA_WAVES) { sm.tile[0].near[tid] = 0; sm.tile[1].near[tid] = 0; }
    __syncthreads();
    if (ntiles > 0) {
        load_tile(0);
        store_tile(sm.tile[0], 0);
        if (ntiles > 1) load_tile(GA_BN);
    }
    __syncthreads();
    for (int t = 0; t < ntiles; ++t) {
        const TileBuf& tb = sm.tile[t & 1];
        const bool has_valid  = tb.flags[1] != 0;
        const bool has_masked = tb.flags[0] != 0;
        const bool near       = LEGACY || tb.near[wave] == t + 1;
        if (has_valid) {
            uint4 kf[4];
            load_kf(tb, 0, kf);
            key_block(tb, 0, has_masked, near, kf, true);
            key_block(tb, 1, has_masked, near, kf, false);
        }
        if (t + 1 < ntiles) {
            store_tile(sm.tile[(t + 1) & 1], t + 1);
            if (t + 2 < ntiles) load_tile((t + 2) * GA_BN);
        }
        __syncthreads();
    }

    // ---- epilogue ----
#pragma unroll
    for (int b = 0; b < GA_QB; ++b) {
        const float l_tot = xhalf_sum(l_run[b]);
        const bool  row_ok = q_ok[b] && l_tot > 0.f;
        const float inv_l = row_ok ? 1.0f / l_tot : 0.f;
        if (q_in[b]) {
            float* orow = Oh + (size_t)q[b] * o_pitch;
#pragma unroll
            for (int dt = 0; dt < 2; ++dt)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
                    if (row_ok) v = make_float4(oacc[b][dt][4 * g] * inv_l, oacc[b][dt][4 * g + 1] * inv_l,
                                                oacc[b][dt][4 * g + 2] * inv_l, oacc[b][dt][4 * g + 3] * inv_l);
                    *reinterpret_cast<float4*>(orow + dt * 32 + 8 * g + 4 * half) = v;
                }
            if (L && half == 0) L[(size_t)zh * N + q[b]] = row_ok ? m2[b] + __logf(l_tot) : -INFINITY;
        }
    }
}

#include "geo_attn_fwd_pipe.inc"

// One distance path for the whole grid ...
template <bool DIST_VALU, bool LEGACY, int GA_QB>
__global__ __launch_bounds__(GA_THREADS, 2)
void geo_attn_fwd_kernel(const uint16_t* __restrict__ Q, const uint16_t* __restrict__ K,
                         const uint16_t* __restrict__ V, const float* __restrict__ coords,
                         const float* __restrict__ sigma, const uint8_t* __restrict__ key_pad,
                         float* __restrict__ O, float* __restrict__ L,
                         const int H, const int N, const int ZH, const int n_qtiles,
                         const float* __restrict__ beta, const float min_rbf, const float max_rbf, const GaStrides st)
{
    __shared__ Smem sm;
    geo_attn_fwd_body<DIST_VALU, LEGACY, GA_QB>(sm, (int)blockIdx.x, Q, K, V, coords, sigma, key_pad, O, L, H, N, ZH, n_qtiles, 1,
                                                beta, min_rbf, max_rbf, st);
}

// ... or both over one grid of twice the size: workgroup g and workgroup n_wgs + g look at the same queries, the
// first with the matrix-core distances, the second with the direct ones, and the one that does not own them
// returns after the prologue.  One launch instead of two: the early exits overlap with the work.
template <bool LEGACY, int GA_QB>
__global__ __launch_bounds__(GA_THREADS, 2)
void geo_attn_fwd_both_kernel(const uint16_t* __restrict__ Q, const uint16_t* __restrict__ K,
                              const uint16_t* __restrict__ V, const float* __restrict__ coords,
                              const float* __restrict__ sigma, const uint8_t* __restrict__ key_pad,
                              float* __restrict__ O, float* __restrict__ L,
                              const int H, const int N, const int ZH, const int n_qtiles, const int n_wgs,
                              const float* __restrict__ beta, const float min_rbf, const float max_rbf, const GaStrides st)
{
    __shared__ Smem sm;
    const int id = (int)blockIdx.x;
    if (id < n_wgs)
        geo_attn_fwd_body<false, LEGACY, GA_QB>(sm, id, Q, K, V, coords, sigma, key_pad, O, L, H, N, ZH, n_qtiles, 0,
                                                beta, min_rbf, max_rbf, st);
    else
        geo_attn_fwd_body<true, LEGACY, GA_QB>(sm, id - n_wgs, Q, K, V, coords, sigma, key_pad, O, L, H, N, ZH, n_qtiles, 0,
                                               beta, min_rbf, max_rbf, st);
}

// The pipelined body over the first half of a doubled grid, the direct-distance body (for workgroups whose
// queries are spread too widely for the matrix-core distances) over the second; take_all: the pipelined body alone.
__global__ __launch_bounds__(GA_THREADS, 2)
void geo_attn_fwd_pipe_kernel(const uint16_t* __restrict__ Q, const uint16_t* __restrict__ K,
                              const uint16_t* __restrict__ V, const float* __restrict__ coords,
                              const float* __restrict__ sigma, const uint8_t* __restrict__ key_pad,
                              float* __restrict__ O, float* __restrict__ L,
                              const int H, const int N, const int ZH, const int n_qtiles, const int n_wgs, const int take_all,
                              const GaStrides st)
{
    extern __shared__ __align__(16) unsigned char ga_dyn_smem[];
    const int id = (int)blockIdx.x;
    if (id < n_wgs)
        geo_attn_fwd_pipe_body(*reinterpret_cast<PipeSmem*>(ga_dyn_smem), id, Q, K, V, coords, sigma, key_pad, O, L,
                               H, N, ZH, n_qtiles, take_all, st);
    else
        geo_attn_fwd_body<true, false, 2>(*reinterpret_cast<Smem*>(ga_dyn_smem), id - n_wgs, Q, K, V, coords, sigma, key_pad, O, L,
                                          H, N, ZH, n_qtiles, 0, nullptr, 0.f, 1.f, st);
}
constexpr size_t GA_PIPE_LDS = sizeof(PipeSmem) > sizeof(Smem) ? sizeof(PipeSmem) : sizeof(Smem);
static_assert(GA_PIPE_LDS <= 80 * 1024, "two workgroups per compute unit");

struct GaVariant { const char* name; };
const GaVariant kVariants[] = { {"auto"}, {"dist_mfma"}, {"dist_valu"}, {"one_block_per_wave"}, {"two_blocks_per_wave"},
                                {"pipelined"}, {"pipelined_dist_mfma"} };
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
    if (d_head != GA_D) return PROTEUS_ERR_BAD_HEAD_DIM;
    if (tuning < 0 || tuning >= kNumVariants) return PROTEUS_ERR_BAD_TUNING;
    if (((uintptr_t)Q & 15) || ((uintptr_t)K & 15) || ((uintptr_t)V & 15) || ((uintptr_t)O & 15)) return PROTEUS_ERR_BAD_ALIGNMENT;
    return PROTEUS_OK;
}

namespace {
template <bool LEGACY, int QB>
int launch_attn_qb(const uint16_t* Q, const uint16_t* K, const uint16_t* V, const float* coords, const float* sigma,
                   const uint8_t* key_pad_mask, float* O, float* L, int Z, int H, int N, int dist,
                   const float* beta, float min_rbf, float max_rbf, const GaStrides& gs, hipStream_t st)
{
    constexpr int BM = GA_WAVES * 32 * QB;
    const int n_qtiles = (N + BM - 1) / BM;
    const int ZH = Z * H;
    const unsigned n_wgs = (unsigned)n_qtiles * (unsigned)ZH;
    // dist 0: each workgroup picks its distance path (one launch over twice the grid, see the kernel);
    // 1 / 2: force the matrix-core / vector-ALU path everywhere
    if (dist == 0)
        hipLaunchKernelGGL((geo_attn_fwd_both_kernel<LEGACY, QB>), dim3(2 * n_wgs), dim3(GA_THREADS), 0, st,
                           Q, K, V, coords, sigma, key_pad_mask, O, L, H, N, ZH, n_qtiles, (int)n_wgs, beta, min_rbf, max_rbf, gs);
    else if (dist == 1)
        hipLaunchKernelGGL((geo_attn_fwd_kernel<false, LEGACY, QB>), dim3(n_wgs), dim3(GA_THREADS), 0, st,
                           Q, K, V, coords, sigma, key_pad_mask, O, L, H, N, ZH, n_qtiles, beta, min_rbf, max_rbf, gs);
    else
        hipLaunchKernelGGL((geo_attn_fwd_kernel<true, LEGACY, QB>), dim3(n_wgs), dim3(GA_THREADS), 0, st,
                           Q, K, V, coords, sigma, key_pad_mask, O, L, H, N, ZH, n_qtiles, beta, min_rbf, max_rbf, gs);
    return (int)hipGetLastError();
}

int launch_attn_pipe(const uint16_t* Q, const uint16_t* K, const uint16_t* V, const float* coords, const float* sigma,
                     const uint8_t* key_pad_mask, float* O, float* L, int Z, int H, int N, bool take_all,
                     const GaStrides& gs, hipStream_t st)
{
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(geo_attn_fwd_pipe_kernel),
                                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)GA_PIPE_LDS);
    if (attr != hipSuccess) return (int)attr;
    constexpr int BM = GA_WAVES * 64;
    const int n_qtiles = (N + BM - 1) / BM;
    const int ZH = Z * H;
    const unsigned n_wgs = (unsigned)n_qtiles * (unsigned)ZH;
    hipLaunchKernelGGL(geo_attn_fwd_pipe_kernel, dim3(take_all ? n_wgs : 2 * n_wgs), dim3(GA_THREADS), GA_PIPE_LDS, st,
                       Q, K, V, coords, sigma, key_pad_mask, O, L, H, N, ZH, n_qtiles, (int)n_wgs, take_all ? 1 : 0, gs);
    return (int)hipGetLastError();
}

template <bool LEGACY>
int launch_attn(const uint16_t* Q, const uint16_t* K, const uint16_t* V, const float* coords, const float* sigma,
                const uint8_t* key_pad_mask, float* O, float* L, int Z, int H, int N, int tuning,
                const float* beta, float min_rbf, float max_rbf, const GaStrides& gs, hipStream_t st)
{
    // Two query blocks per wave unless that leaves at most one workgroup per compute unit (256 of them on
    // this chip, two workgroups each): then one block per wave doubles the waves in flight.  With two blocks per
    // wave the README logits take the software-pipelined kernel.
    const long wgs2 = (long)((N + GA_WAVES * 64 - 1) / (GA_WAVES * 64)) * Z * H;
    bool one_block = wgs2 <= 256;
    int dist = tuning;
    bool pipelined = !LEGACY && tuning == 0 && !one_block;
    bool take_all = false;
    if (tuning == 3) { one_block = true;  dist = 0; }
    if (tuning == 4) { one_block = false; dist = 0; }
    if (tuning == 5 || tuning == 6) {                   // the pipelined kernel whatever the grid (6: without the direct-distance body beside it)
        if (LEGACY) { one_block = false; dist = 0; }
        else { pipelined = true; take_all = (tuning == 6); }
    }
    if (pipelined) return launch_attn_pipe(Q, K, V, coords, sigma, key_pad_mask, O, L, Z, H, N, take_all, gs, st);
    return one_block ? launch_attn_qb<LEGACY, 1>(Q, K, V, coords, sigma, key_pad_mask, O, L, Z, H, N, dist, beta, min_rbf, max_rbf, gs, st)
                     : launch_attn_qb<LEGACY, 2>(Q, K, V, coords, sigma, key_pad_mask, O, L, Z, H, N, dist, beta, min_rbf, max_rbf, gs, st);
}
// contiguous [Z,H,N,64] tensors
GaStrides contiguous_strides(int H, int N) {
    GaStrides gs;
    const long t[3] = {(long)H * N * GA_D, (long)N * GA_D, (long)GA_D};
    for (int i = 0; i < 3; ++i) { gs.q[i] = t[i]; gs.k[i] = t[i]; gs.v[i] = t[i]; gs.o[i] = t[i]; }
    return gs;
}

// strides[12]: (batch, head, token) element strides of Q, K, V, O in this order
int strides_from(const int64_t* strides, int Z, int H, int N, GaStrides& gs) {
    if (!strides) return PROTEUS_ERR_NULL_POINTER;
    long* dst[4] = {gs.q, gs.k, gs.v, gs.o};
    for (int t = 0; t < 4; ++t) {
        const int64_t sz = strides[3 * t], sh = strides[3 * t + 1], sn = strides[3 * t + 2];
        // rows of 64 contiguous elements that do not overlap and stay 16-byte aligned; a sequence's byte
        // offsets fit the 31 bits of a buffer-load offset
        if (sz < 0 || sh < 0 || sn < GA_D) return PROTEUS_ERR_BAD_LAYOUT;
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
    return strides_from(strides, Z, H, N, gs);
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
    rc = strides_from(strides, Z, H, N, gs);
    if (rc != PROTEUS_OK) return rc;
    return launch_attn<false>(Q, K, V, coords, sigma, key_pad_mask, O, L, Z, H, N, tuning, nullptr, 0.f, 1.f, gs,
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
    return launch_attn<false>(Q, K, V, coords, sigma, key_pad_mask, O, L, Z, H, N, tuning, nullptr, 0.f, 1.f, contiguous_strides(H, N),
                              reinterpret_cast<hipStream_t>(stream));
}

extern "C" int proteus_geo_attn_legacy_fwd(const uint16_t* Q, const uint16_t* K, const uint16_t* V,
                                           const float* coords, const float* sigma, const float* beta,
                                           const uint8_t* key_pad_mask,
                                           float* O, float* L,
                                           int Z, int H, int N, int d_head,
                                           float min_rbf, float max_rbf, int tuning, void* stream)
{
    const int rc = proteus_geo_attn_fwd_check(Q, K, V, coords, sigma, key_pad_mask, O, L, Z, H, N, d_head, tuning);
    if (rc != PROTEUS_OK) return rc;
    if (!beta) return PROTEUS_ERR_NULL_POINTER;
    if (!(max_rbf > min_rbf)) return PROTEUS_ERR_BAD_SHAPE;
    // a pair mask makes the result sensitive to the last bits of the rbf: use direct distances then
    if ((tuning == 0 || tuning >= 3) && (min_rbf > 0.f || max_rbf < 1.f)) tuning = 2;
    return launch_attn<true>(Q, K, V, coords, sigma, key_pad_mask, O, L, Z, H, N, tuning, beta, min_rbf, max_rbf, contiguous_strides(H, N),
                             reinterpret_cast<hipStream_t>(stream));
}

extern "C" int proteus_geo_attn_legacy_fwd_strided(const uint16_t* Q, const uint16_t* K, const uint16_t* V,
                                                   const int64_t* strides,
                                                   const float* coords, const float* sigma, const float* beta,
                                                   const uint8_t* key_pad_mask,
                                                   float* O, float* L,
                                                   int Z, int H, int N, int d_head,
                                                   float min_rbf, float max_rbf, int tuning, void* stream)
{
    int rc = proteus_geo_attn_fwd_check(Q, K, V, coords, sigma, key_pad_mask, O, L, Z, H, N, d_head, tuning);
    if (rc != PROTEUS_OK) return rc;
    if (!beta) return PROTEUS_ERR_NULL_POINTER;
    if (!(max_rbf > min_rbf)) return PROTEUS_ERR_BAD_SHAPE;
    GaStrides gs;
    rc = strides_from(strides, Z, H, N, gs);
    if (rc != PROTEUS_OK) return rc;
    if ((tuning == 0 || tuning >= 3) && (min_rbf > 0.f || max_rbf < 1.f)) tuning = 2;
    return launch_attn<true>(Q, K, V, coords, sigma, key_pad_mask, O, L, Z, H, N, tuning, beta, min_rbf, max_rbf, gs,
                             reinterpret_cast<hipStream_t>(stream));
}
