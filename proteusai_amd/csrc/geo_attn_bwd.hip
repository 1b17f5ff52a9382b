// RBF-scaled geometric attention backward for gfx950 (MI355X): dQ, dK, dV, d sigma (and d beta).
//
// What it computes (reference: old/old_scripts/attn/geometric_attn.py:262-543, wrapper :609-660), with
// S = q.k/sqrt(d), rbf = exp(-|r_i - r_j|^2/(2 sigma_h^2)) and the logits t(S, rbf) of the forward kernel:
//     P    = exp(t - L_i)                 (L: the forward's logsumexp; 0 for a masked pair)      :453
//     dV_j = sum_i P_ij dO_i                                                                      :459
//     dP   = dO_i . V_j ;  dt = P (dP - D_i),  D_i = sum_d O_id dO_id                             :462-465
//     dS   = dt * dt/dS ;  dQ_i = sum_j dS_ij K_j / sqrt(d) ;  dK_j = sum_i dS_ij Q_i / sqrt(d)   :468,500-505
//     d sigma_h = sum dt * dt/drbf * rbf * |r_i - r_j|^2 / sigma_h^3                              :473,494-497
//   README logits  t = S (1 + rbf):             dt/dS = 1 + rbf,              dt/drbf = S
//   LEGACY logits  t = S + beta Rn |S|, Rn = 2 (rbf - min)/(max - min) - 1   (:448-449):
//                  dt/dS = 1 + beta Rn sign(S), dt/drbf = 2 beta |S|/(max - min), d beta_h = sum dt Rn |S|  (:468-479)
//
// Two passes instead of the reference's one kernel with atomic adds into dQ (:501-503), run by the two
// halves of one launch:
//   OWN_Q = false  a wave owns 32 keys, streams the queries, accumulates dK, dV (and d sigma, d beta);
//   OWN_Q = true   a wave owns 32 queries, streams the keys, accumulates dQ.
// Both are the same code.  Scores are computed with the rows of the streamed ("other") tokens in the
// accumulator rows and the wave's own token in the accumulator column (lane % 32), so a lane owns one own
// token: S = other . own^T and dP likewise on v_mfma_f32_32x32x16_bf16 with the own side held in registers
// as the B operand for the whole kernel.  P and dS are, after bf16 conversion, directly the B operands of
// the accumulating products (dV^T += dO^T P, dK^T += Q^T dS; dQ^T += K^T dS) whose A operands are the
// transposed tiles staged in LDS, read in the accumulator's row order.  No atomics except the one
// per-wave add into d sigma / d beta; dQ, dK, dV are deterministic.

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>
#include "proteus_hip.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float  floatx16 __attribute__((ext_vector_type(16)));
typedef float  floatx2 __attribute__((ext_vector_type(2)));

constexpr int GB_WAVES   = 4;
constexpr int GB_THREADS = GB_WAVES * 64;
constexpr int GB_OWN     = GB_WAVES * 32;   // own tokens per workgroup
constexpr int GB_BN      = 64;              // streamed tokens per tile
constexpr int GB_D       = 64;
constexpr int GB_LDR     = GB_D + 8;        // row stride of a row-major tile [token][d] (bf16 elements)
constexpr int GB_LDT     = GB_BN + 4;       // row stride of a transposed tile [d][token]: 34 dwords, so the 32 rows a
                                            // half-wave reads 8 bytes from fall into 32 different bank pairs
constexpr float LOG2E    = 1.4426950408889634f;

struct __align__(16) BwdSmem {
    uint16_t ra[GB_BN * GB_LDR];     // other tokens, first tensor  (K or Q), row-major:  A operand of S
    uint16_t rb[GB_BN * GB_LDR];     // other tokens, second tensor (V or dO), row-major: A operand of dP
    uint16_t ta[GB_D * GB_LDT];      // first tensor transposed:  A operand of dQ^T / dK^T
    uint16_t tb[GB_D * GB_LDT];      // second tensor transposed (dO^T): A operand of dV^T (keys-own pass only)
    float    rx[GB_BN], ry[GB_BN], rz[GB_BN];   // coordinates of the other tokens
    float    rl[GB_BN], rd[GB_BN];   // per other token that is a usable query: -L*log2(e) and D; -inf and 0 for an
                                     // unusable one (padded / out of range / empty row).  When they are keys:
                                     // rl = 0 for a usable key, -inf for an unusable one
};

__device__ __forceinline__ unsigned pack_bf16(float a, float b) {
    floatx2 f = {a, b};
    return __builtin_bit_cast(unsigned, __builtin_convertvector(f, bf16x2));
}

// Element strides (batch, head, token) of Q, K, V, dO (bf16) and dQ, dK, dV (f32); the head dimension is contiguous.
struct GbStrides { long q[3], k[3], v[3], g[3], dq[3], dk[3], dv[3]; };

template <bool OWN_Q, bool LEGACY>
__device__ __forceinline__
void geo_attn_bwd_body(BwdSmem& sm, const int block_id,
                       const uint16_t* __restrict__ Q, const uint16_t* __restrict__ K,
                       const uint16_t* __restrict__ V, const uint16_t* __restrict__ dO,
                       const float* __restrict__ coords, const float* __restrict__ sigma,
                       const float* __restrict__ beta, const uint8_t* __restrict__ key_pad,
                       const float* __restrict__ Lse, const float* __restrict__ Dvec,
                       float* __restrict__ dQ, float* __restrict__ dK, float* __restrict__ dV,
                       float* __restrict__ d_sigma, float* __restrict__ d_beta,
                       const int H, const int N, const int n_otiles, const float min_rbf, const float max_rbf, const GbStrides& st)
{

    const int tid  = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int half = lane >> 5;
    const int col  = lane & 31;

    const int ot = block_id % n_otiles;
    const int zh = block_id / n_otiles;
    const int z  = zh / H;
    const int h  = zh - z * H;
    const size_t lin_off = (size_t)zh * (size_t)N;         // L and D are contiguous [Z,H,N]
    auto at = [&](const long (&t)[3]) { return (size_t)z * (size_t)t[0] + (size_t)h * (size_t)t[1]; };
    const float*   cz = coords + (size_t)z * N * 3;
    const uint8_t* mz = key_pad ? key_pad + (size_t)z * N : nullptr;
    const float*   Lh = Lse + lin_off;
    const float*   Dh = Dvec + lin_off;

    const float sg  = sigma[h];
    const float cs2 = 0.72134752044448170368f / (sg * sg);       // log2(e)/2 / sigma^2: rbf = exp2(-d^2 cs2)
    const float bt  = LEGACY ? beta[h] : 0.f;
    const float rinv = LEGACY ? 1.0f / (max_rbf - min_rbf) : 0.f;
    const float rn_a = 2.0f * rinv, rn_b = -(2.0f * min_rbf * rinv + 1.0f);   // Rn = rbf rn_a + rn_b

    // ---- own token of this lane ----
    const int  o      = ot * GB_OWN + wave * 32 + col;
    const bool own_in = o < N;
    const int  oc     = own_in ? o : N - 1;
    const bool own_ok = own_in && !(mz && mz[oc]);
    // An unusable own token (padded, out of range, or a query without any unmasked pair) is given zero
    // operands, zero coordinates and an exponent offset of +inf: every pair with it gets P = exp2(-inf) = 0
    // and all its products stay finite, without a select per pair.
    bool  own_use = own_ok;
    float own_l2 = 0.f, own_d = 0.f;
    if (OWN_Q) {
        const float l = Lh[oc];
        own_use = own_ok && (l > -INFINITY);
        own_l2 = own_use ? l * LOG2E : 0.f;
        own_d  = own_use ? Dh[oc] : 0.f;
    }
    if (!own_use) own_l2 = INFINITY;
    // Validity needs no select per pair: an unusable token's operands are zeros, so its S, dP and every
    // product it is contracted in vanish; the exponent offset of an unusable QUERY is -inf (its L is -inf
    // or garbage), which makes its P an exact 0.  An unusable KEY streamed past a query gets the offset
    // -inf as well, but only in tiles that hold one (otherwise a query with a very negative L could
    // overflow P for it, and inf * 0 is not 0).
    const float own_off = -own_l2;
    const float ox = own_use ? cz[3 * oc] : 0.f, oy = own_use ? cz[3 * oc + 1] : 0.f, oz = own_use ? cz[3 * oc + 2] : 0.f;
    // bounding box of the wave's usable own tokens (for the far-tile test)
    float blo[3] = {own_use ? ox : 3.0e38f, own_use ? oy : 3.0e38f, own_use ? oz : 3.0e38f};
    float bhi[3] = {own_use ? ox : -3.0e38f, own_use ? oy : -3.0e38f, own_use ? oz : -3.0e38f};
#pragma unroll
    for (int c = 0; c < 3; ++c)
        for (int off = 32; off > 0; off >>= 1) { blo[c] = fminf(blo[c], __shfl_xor(blo[c], off)); bhi[c] = fmaxf(bhi[c], __shfl_xor(bhi[c], off)); }
    // exp2(-d^2 cs2) < 2^-25 beyond this distance: s*(1+rbf) rounds to s in fp32
    const float far2 = 25.0f / cs2;
    // B operands: lane (half, col) holds d = 16*ks + 8*half + 0..7 of its own token; the first one carries 1/sqrt(64)
    const uint16_t* Bs_src = OWN_Q ? Q + at(st.q) : K + at(st.k);
    const uint16_t* Bp_src = OWN_Q ? dO + at(st.g) : V + at(st.v);
    const size_t bs_pitch = (size_t)(OWN_Q ? st.q[2] : st.k[2]), bp_pitch = (size_t)(OWN_Q ? st.g[2] : st.v[2]);
    bf16x8 bs[4], bp[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
        const uint4 r0 = *reinterpret_cast<const uint4*>(Bs_src + (size_t)oc * bs_pitch + ks * 16 + half * 8);
        const uint4 r1 = *reinterpret_cast<const uint4*>(Bp_src + (size_t)oc * bp_pitch + ks * 16 + half * 8);
        bf16x8 v = __builtin_bit_cast(bf16x8, own_use ? r0 : make_uint4(0u, 0u, 0u, 0u));
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = (__bf16)((float)v[e] * 0.125f);
        bs[ks] = v;
        bp[ks] = __builtin_bit_cast(bf16x8, own_use ? r1 : make_uint4(0u, 0u, 0u, 0u));
    }

    floatx16 acc_a[2], acc_b[2];       // OWN_Q: dQ^T (acc_a).  keys own: dK^T (acc_a), dV^T (acc_b).  [d half][16 rows]
#pragma unroll
    for (int dt = 0; dt < 2; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) { acc_a[dt][r] = 0.f; acc_b[dt][r] = 0.f; }
    float sum_sigma = 0.f, sum_beta = 0.f;
    // log2(e) in a vector register: as a literal it would make each instruction that uses it a
    // scalar-operand one (4 clocks instead of about 2.5)
    float log2e_v = LOG2E;
    asm volatile("" : "+v"(log2e_v));

    // staging roles: a thread moves the 8-wide d chunk `dc` of the token pair `kp`
    const int kp = tid & 31;
    const int dc = tid >> 5;
    const uint16_t* Ra_src = OWN_Q ? K + at(st.k) : Q + at(st.q);
    const uint16_t* Rb_src = OWN_Q ? V + at(st.v) : dO + at(st.g);
    // element offsets inside a (batch, head) slice fit 31 bits (checked on the host)
    const int ra_pitch = (int)(OWN_Q ? st.k[2] : st.q[2]), rb_pitch = (int)(OWN_Q ? st.v[2] : st.g[2]);

    // registers holding the tile in flight from global memory: requested before the current tile is
    // computed, written to LDS after it (padded tokens as zeros)
    uint4 ga0, ga1, gb0, gb1;
    float gx = 0.f, gy = 0.f, gz = 0.f, gl = 0.f, gd = 0.f;
    unsigned gm0 = 0, gm1 = 0, gm = 0;      // raw padding bytes of the two staged tokens / of token tid
    int gj0 = 0;
    // Only requests: every address is clamped into range and nothing that comes back is looked at before
    // store_tile, so no load waits for another.
    auto load_tile = [&](const int j0) {
        gj0 = j0;
        const int ta_ = min(j0 + 2 * kp, N - 1), tb_ = min(j0 + 2 * kp + 1, N - 1);
        ga0 = *reinterpret_cast<const uint4*>(Ra_src + (ta_ * ra_pitch + dc * 8));
        ga1 = *reinterpret_cast<const uint4*>(Ra_src + (tb_ * ra_pitch + dc * 8));
        gb0 = *reinterpret_cast<const uint4*>(Rb_src + (ta_ * rb_pitch + dc * 8));
        gb1 = *reinterpret_cast<const uint4*>(Rb_src + (tb_ * rb_pitch + dc * 8));
        if (mz) { gm0 = mz[ta_]; gm1 = mz[tb_]; }
        if (tid < GB_BN) {
            const int tc = min(j0 + tid, N - 1);
            gx = cz[3 * tc]; gy = cz[3 * tc + 1]; gz = cz[3 * tc + 2];
            if (mz) gm = mz[tc];
            if (!OWN_Q) { gl = Lh[tc]; gd = Dh[tc]; }
        }
    };
    auto store_tile = [&]() {
        {
            // padded / out-of-range tokens as zeros
            const uint4 zero = make_uint4(0u, 0u, 0u, 0u);
            if (gj0 + 2 * kp >= N || gm0) { ga0 = zero; gb0 = zero; }
            if (gj0 + 2 * kp + 1 >= N || gm1) { ga1 = zero; gb1 = zero; }
        }
        *reinterpret_cast<uint4*>(&sm.ra[(2 * kp) * GB_LDR + dc * 8])     = ga0;
        *reinterpret_cast<uint4*>(&sm.ra[(2 * kp + 1) * GB_LDR + dc * 8]) = ga1;
        *reinterpret_cast<uint4*>(&sm.rb[(2 * kp) * GB_LDR + dc * 8])     = gb0;
        *reinterpret_cast<uint4*>(&sm.rb[(2 * kp + 1) * GB_LDR + dc * 8]) = gb1;
        const unsigned xa[4] = {ga0.x, ga0.y, ga0.z, ga0.w}, ya[4] = {ga1.x, ga1.y, ga1.z, ga1.w};
        const unsigned xb[4] = {gb0.x, gb0.y, gb0.z, gb0.w}, yb[4] = {gb1.x, gb1.y, gb1.z, gb1.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            // [d][token pair]: low half-word = even token, high half-word = odd token
            *reinterpret_cast<unsigned*>(&sm.ta[(dc * 8 + 2 * e) * GB_LDT + 2 * kp])     = __builtin_amdgcn_perm(ya[e], xa[e], 0x05040100u);
            *reinterpret_cast<unsigned*>(&sm.ta[(dc * 8 + 2 * e + 1) * GB_LDT + 2 * kp]) = __builtin_amdgcn_perm(ya[e], xa[e], 0x07060302u);
            if (!OWN_Q) {
                *reinterpret_cast<unsigned*>(&sm.tb[(dc * 8 + 2 * e) * GB_LDT + 2 * kp])     = __builtin_amdgcn_perm(yb[e], xb[e], 0x05040100u);
                *reinterpret_cast<unsigned*>(&sm.tb[(dc * 8 + 2 * e + 1) * GB_LDT + 2 * kp]) = __builtin_amdgcn_perm(yb[e], xb[e], 0x07060302u);
            }
        }
        if (tid < GB_BN) {       // = wave 0, one token per lane
            bool gok = (gj0 + tid < N) && gm == 0;
            if (!OWN_Q) gok = gok && (gl > -INFINITY);
            // an unusable token's coordinates, L and D may hold anything: zeros keep every product finite
            if (!gok) { gx = 0.f; gy = 0.f; gz = 0.f; gd = 0.f; }
            gl = gok ? (OWN_Q ? 0.f : -gl * LOG2E) : -INFINITY;
            sm.rx[tid] = gx; sm.ry[tid] = gy; sm.rz[tid] = gz;
            sm.rl[tid] = gl; sm.rd[tid] = gd;
        }
    };

    const int ntiles = (N + GB_BN - 1) / GB_BN;
    load_tile(0);
    for (int t = 0; t < ntiles; ++t) {
        __syncthreads();                      // the previous tile has been consumed
        store_tile();
        if (t + 1 < ntiles) load_tile((t + 1) * GB_BN);
        __syncthreads();

        // far-tile test: lane l takes the tile's token l and measures its distance to the box of this wave's own
        // tokens.  If every usable token is beyond `far2` the multiplier is 1 to fp32 rounding and its derivative
        // terms vanish, so the geometry is skipped for the whole tile (the legacy logits depend on rbf down to 0:
        // always evaluated).
        bool near = true, any_bad = false;
        {
            const bool usable = sm.rl[lane] > -INFINITY;
            any_bad = OWN_Q && __builtin_amdgcn_ballot_w64(!usable) != 0;
            if (!LEGACY) {
                const float p[3] = {sm.rx[lane], sm.ry[lane], sm.rz[lane]};
                float g2 = 0.f;
#pragma unroll
                for (int c = 0; c < 3; ++c) {
                    const float gap = fmaxf(fmaxf(blo[c] - p[c], p[c] - bhi[c]), 0.f);
                    g2 = __builtin_fmaf(gap, gap, g2);
                }
                near = __builtin_amdgcn_ballot_w64(usable && !(g2 > far2)) != 0;
            }
        }

        // ---- S and dP of a 32 x 32 block: rows = other tokens, column = own token ----
        auto score_mfma = [&](const int mt, floatx16& sa, floatx16& pa) {
#pragma unroll
            for (int r = 0; r < 16; ++r) { sa[r] = 0.f; pa[r] = 0.f; }
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) {
                const uint4 fa = *reinterpret_cast<const uint4*>(&sm.ra[(mt * 32 + col) * GB_LDR + ks * 16 + half * 8]);
                const uint4 fb = *reinterpret_cast<const uint4*>(&sm.rb[(mt * 32 + col) * GB_LDR + ks * 16 + half * 8]);
                sa = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, fa), bs[ks], sa, 0, 0, 0);
                pa = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, fb), bp[ks], pa, 0, 0, 0);
            }
        };
        // The queries-own pass has the registers to issue the second block's matrix products before the
        // first block's vector work, so they run under it; the keys-own pass takes the blocks one at a time.
        auto process_block = [&](const int mt, const floatx16& sacc, const floatx16& pacc) {
            // ---- per pair: multiplier, P, dt, dS; accumulator register r is row 8*(r/4) + 4*half + (r%4).
            // Unusable tokens carry +inf in their exponent offset: P = exp2(-inf) = 0, and since their
            // operands and coordinates are zeros everything derived from P is an exact 0 as well. ----
            float pv[16], ds[16];
            auto pairs = [&](auto near_c) {
                constexpr bool NEAR = decltype(near_c)::value;
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int rb0 = mt * 32 + 8 * g + 4 * half;
                    float ls[4] = {0.f, 0.f, 0.f, 0.f};
                    if (!OWN_Q || any_bad) {
                        const float4 kl = *reinterpret_cast<const float4*>(&sm.rl[rb0]);
                        ls[0] = kl.x; ls[1] = kl.y; ls[2] = kl.z; ls[3] = kl.w;
                    }
                    float xs[4] = {0.f, 0.f, 0.f, 0.f}, ys[4] = {0.f, 0.f, 0.f, 0.f}, zs[4] = {0.f, 0.f, 0.f, 0.f};
                    float dds[4] = {0.f, 0.f, 0.f, 0.f};
                    if (NEAR) {
                        const float4 kx = *reinterpret_cast<const float4*>(&sm.rx[rb0]);
                        const float4 ky = *reinterpret_cast<const float4*>(&sm.ry[rb0]);
                        const float4 kz = *reinterpret_cast<const float4*>(&sm.rz[rb0]);
                        xs[0] = kx.x; xs[1] = kx.y; xs[2] = kx.z; xs[3] = kx.w;
                        ys[0] = ky.x; ys[1] = ky.y; ys[2] = ky.z; ys[3] = ky.w;
                        zs[0] = kz.x; zs[1] = kz.y; zs[2] = kz.z; zs[3] = kz.w;
                    }
                    if (!OWN_Q) {
                        const float4 kd = *reinterpret_cast<const float4*>(&sm.rd[rb0]);
                        dds[0] = kd.x; dds[1] = kd.y; dds[2] = kd.z; dds[3] = kd.w;
                    }
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        const int r = 4 * g + v;
                        const float s  = sacc[r];
                        const float off = OWN_Q ? (any_bad ? own_off + ls[v] : own_off) : ls[v];   // -(L log2e) of the pair's query, -inf if unusable
                        const float dd = OWN_Q ? own_d : dds[v];
                        if (!NEAR) {
                            const float p  = __builtin_amdgcn_exp2f(__builtin_fmaf(s, log2e_v, off));
                            const float dt = p * (pacc[r] - dd);
                            pv[r] = p;
                            ds[r] = dt;
                            continue;
                        }
                        const float dx = ox - xs[v], dy = oy - ys[v], dz = oz - zs[v];
                        const float d2 = __builtin_fmaf(dz, dz, __builtin_fmaf(dy, dy, dx * dx));
                        const float rbf = __builtin_amdgcn_exp2f(-d2 * cs2);
                        if (!LEGACY) {
                            const float tl = __builtin_fmaf(s, rbf, s);
                            const float p  = __builtin_amdgcn_exp2f(__builtin_fmaf(tl, log2e_v, off));
                            const float dt = p * (pacc[r] - dd);
                            pv[r] = p;
                            ds[r] = __builtin_fmaf(dt, rbf, dt);                    // dt/dS = 1 + rbf
                            if (!OWN_Q) sum_sigma = __builtin_fmaf(dt * s, rbf * d2, sum_sigma);   // dt/drbf = S
                        } else {
                            const float rn = __builtin_fmaf(rbf, rn_a, rn_b);
                            const float as = fabsf(s);
                            const float tl = __builtin_fmaf(bt * rn, as, s);
                            const bool  in_range = rbf >= min_rbf && rbf <= max_rbf;
                            const float p  = in_range ? __builtin_amdgcn_exp2f(__builtin_fmaf(tl, log2e_v, off)) : 0.f;
                            const float dt = p * (pacc[r] - dd);
                            pv[r] = p;
                            ds[r] = dt * (1.0f + bt * rn * (s > 0.f ? 1.0f : (s < 0.f ? -1.0f : 0.f)));
                            if (!OWN_Q) {
                                sum_sigma = __builtin_fmaf(dt * as, rbf * d2, sum_sigma);
                                sum_beta  = __builtin_fmaf(dt * rn, as, sum_beta);
                            }
                        }
                    }
                }
            };
            if (near) pairs(std::true_type{}); else pairs(std::false_type{});
            // ---- accumulating products: contraction over the other tokens of this block ----
#pragma unroll
            for (int t2 = 0; t2 < 2; ++t2) {
                // contraction slot e of this half-wave is other token mt*32 + 16*t2 + 8*(e/4) + 4*half + (e%4)
                const uint4 dsb = make_uint4(pack_bf16(ds[8 * t2 + 0], ds[8 * t2 + 1]), pack_bf16(ds[8 * t2 + 2], ds[8 * t2 + 3]),
                                             pack_bf16(ds[8 * t2 + 4], ds[8 * t2 + 5]), pack_bf16(ds[8 * t2 + 6], ds[8 * t2 + 7]));
                const uint4 pb  = make_uint4(pack_bf16(pv[8 * t2 + 0], pv[8 * t2 + 1]), pack_bf16(pv[8 * t2 + 2], pv[8 * t2 + 3]),
                                             pack_bf16(pv[8 * t2 + 4], pv[8 * t2 + 5]), pack_bf16(pv[8 * t2 + 6], pv[8 * t2 + 7]));
#pragma unroll
                for (int dt = 0; dt < 2; ++dt) {
                    const uint16_t* rowa = &sm.ta[(dt * 32 + col) * GB_LDT + mt * 32 + 16 * t2 + 4 * half];
                    const uint2 a0 = *reinterpret_cast<const uint2*>(rowa);
                    const uint2 a1 = *reinterpret_cast<const uint2*>(rowa + 8);
                    const uint4 fa = make_uint4(a0.x, a0.y, a1.x, a1.y);
                    acc_a[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, fa), __builtin_bit_cast(bf16x8, dsb), acc_a[dt], 0, 0, 0);
                    if (!OWN_Q) {
                        const uint16_t* rowb = &sm.tb[(dt * 32 + col) * GB_LDT + mt * 32 + 16 * t2 + 4 * half];
                        const uint2 b0 = *reinterpret_cast<const uint2*>(rowb);
                        const uint2 b1 = *reinterpret_cast<const uint2*>(rowb + 8);
                        const uint4 fb = make_uint4(b0.x, b0.y, b1.x, b1.y);
                        acc_b[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, fb), __builtin_bit_cast(bf16x8, pb), acc_b[dt], 0, 0, 0);
                    }
                }
            }
        };
        if constexpr (OWN_Q) {
            floatx16 sa[2], pa[2];
            score_mfma(0, sa[0], pa[0]);
            score_mfma(1, sa[1], pa[1]);
            process_block(0, sa[0], pa[0]);
            process_block(1, sa[1], pa[1]);
        } else {
#pragma unroll 1
            for (int mt = 0; mt < 2; ++mt) {
                floatx16 sa, pa;
                score_mfma(mt, sa, pa);
                process_block(mt, sa, pa);
            }
        }
    }

    // ---- epilogue: lane (half, col) holds d = dt*32 + 8*g + 4*half + 0..3 of its own token ----
    if (own_in) {
        float* out_a = OWN_Q ? dQ + at(st.dq) + (size_t)o * (size_t)st.dq[2] : dK + at(st.dk) + (size_t)o * (size_t)st.dk[2];
        float* out_b = dV + at(st.dv) + (size_t)o * (size_t)st.dv[2];
#pragma unroll
        for (int dt = 0; dt < 2; ++dt)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                float4 va = make_float4(0.f, 0.f, 0.f, 0.f), vb = va;
                if (own_ok) {
                    va = make_float4(acc_a[dt][4 * g] * 0.125f, acc_a[dt][4 * g + 1] * 0.125f,
                                     acc_a[dt][4 * g + 2] * 0.125f, acc_a[dt][4 * g + 3] * 0.125f);
                    vb = make_float4(acc_b[dt][4 * g], acc_b[dt][4 * g + 1], acc_b[dt][4 * g + 2], acc_b[dt][4 * g + 3]);
                }
                *reinterpret_cast<float4*>(out_a + dt * 32 + 8 * g + 4 * half) = va;
                if (!OWN_Q) *reinterpret_cast<float4*>(out_b + dt * 32 + 8 * g + 4 * half) = vb;
            }
    }
    if (!OWN_Q) {
        // A lane's sums hold the pairs of its own key only.  For an unusable own key they are worth nothing, and not
        // even zero for sure: its scores are 0, so against a query with a very negative L its P can overflow (its dK
        // and dV columns are overwritten with zeros above; here inf * 0 would leave a NaN).
        if (!own_use) { sum_sigma = 0.f; sum_beta = 0.f; }
        for (int off = 32; off > 0; off >>= 1) {
            sum_sigma += __shfl_xor(sum_sigma, off);
            if (LEGACY) sum_beta += __shfl_xor(sum_beta, off);
        }
        if (lane == 0) {
            // d rbf / d sigma = rbf d^2 / sigma^3; the legacy logits carry 2 beta/(max - min) in dt/drbf
            const float k = (LEGACY ? 2.0f * bt * rinv : 1.0f) / (sg * sg * sg);
            if (d_sigma) atomicAdd(&d_sigma[h], sum_sigma * k);
            if (LEGACY && d_beta) atomicAdd(&d_beta[h], sum_beta);
        }
    }
}

// Both passes in one launch over twice the grid: workgroups [0, n_wgs) own keys (dK, dV, d sigma, d beta),
// workgroups [n_wgs, 2 n_wgs) own queries (dQ).  The passes are independent, so one fills the other's tail.
template <bool LEGACY>
__global__ __launch_bounds__(GB_THREADS, 2)
void geo_attn_bwd_kernel(const uint16_t* __restrict__ Q, const uint16_t* __restrict__ K,
                         const uint16_t* __restrict__ V, const uint16_t* __restrict__ dO,
                         const float* __restrict__ coords, const float* __restrict__ sigma,
                         const float* __restrict__ beta, const uint8_t* __restrict__ key_pad,
                         const float* __restrict__ Lse, const float* __restrict__ Dvec,
                         float* __restrict__ dQ, float* __restrict__ dK, float* __restrict__ dV,
                         float* __restrict__ d_sigma, float* __restrict__ d_beta,
                         const int H, const int N, const int n_otiles, const int n_wgs,
                         const float min_rbf, const float max_rbf, const GbStrides st)
{
    __shared__ BwdSmem sm;
    const int id = (int)blockIdx.x;
    if (id < n_wgs)
        geo_attn_bwd_body<false, LEGACY>(sm, id, Q, K, V, dO, coords, sigma, beta, key_pad, Lse, Dvec, dQ, dK, dV, d_sigma, d_beta,
                                         H, N, n_otiles, min_rbf, max_rbf, st);
    else
        geo_attn_bwd_body<true, LEGACY>(sm, id - n_wgs, Q, K, V, dO, coords, sigma, beta, key_pad, Lse, Dvec, dQ, dK, dV, d_sigma, d_beta,
                                        H, N, n_otiles, min_rbf, max_rbf, st);
}

template <bool LEGACY>
int launch_bwd(const uint16_t* Q, const uint16_t* K, const uint16_t* V, const uint16_t* dO,
               const float* coords, const float* sigma, const float* beta, const uint8_t* mask,
               const float* L, const float* D, float* dQ, float* dK, float* dV, float* d_sigma, float* d_beta,
               int Z, int H, int N, float min_rbf, float max_rbf, const GbStrides& gs, hipStream_t st)
{
    const int n_otiles = (N + GB_OWN - 1) / GB_OWN;
    const unsigned n_wgs = (unsigned)n_otiles * (unsigned)(Z * H);
    hipLaunchKernelGGL((geo_attn_bwd_kernel<LEGACY>), dim3(2 * n_wgs), dim3(GB_THREADS), 0, st,
                       Q, K, V, dO, coords, sigma, beta, mask, L, D, dQ, dK, dV, d_sigma, d_beta, H, N, n_otiles, (int)n_wgs,
                       min_rbf, max_rbf, gs);
    return (int)hipGetLastError();
}

GbStrides contiguous_strides(int H, int N) {
    GbStrides gs;
    const long t[3] = {(long)H * N * GB_D, (long)N * GB_D, (long)GB_D};
    long* all[7] = {gs.q, gs.k, gs.v, gs.g, gs.dq, gs.dk, gs.dv};
    for (int a = 0; a < 7; ++a) for (int i = 0; i < 3; ++i) all[a][i] = t[i];
    return gs;
}

// strides[21]: (batch, head, token) element strides of Q, K, V, dO, dQ, dK, dV in this order
int strides_from(const int64_t* strides, int Z, int H, int N, GbStrides& gs) {
    if (!strides) return PROTEUS_ERR_NULL_POINTER;
    long* dst[7] = {gs.q, gs.k, gs.v, gs.g, gs.dq, gs.dk, gs.dv};
    for (int t = 0; t < 7; ++t) {
        const int64_t sz = strides[3 * t], sh = strides[3 * t + 1], sn = strides[3 * t + 2];
        if (sz < 0 || sh < 0 || sn < GB_D) return PROTEUS_ERR_BAD_LAYOUT;
        const int align = (t >= 4) ? 4 : 8;            // 16-byte rows: f32 outputs, bf16 inputs
        if ((sz % align) || (sh % align) || (sn % align)) return PROTEUS_ERR_BAD_ALIGNMENT;
        if ((Z > 1 && sz == 0) || (H > 1 && sh == 0)) return PROTEUS_ERR_BAD_LAYOUT;
        if ((long)N * sn >= (1L << 30)) return PROTEUS_ERR_BAD_SHAPE;
        dst[t][0] = (long)sz; dst[t][1] = (long)sh; dst[t][2] = (long)sn;
    }
    return PROTEUS_OK;
}

}  // namespace

extern "C" int proteus_geo_attn_bwd_check(const uint16_t* Q, const uint16_t* K, const uint16_t* V, const uint16_t* dO,
                                          const float* coords, const float* sigma, const float* beta,
                                          const uint8_t* key_pad_mask, const float* L, const float* D,
                                          const float* dQ, const float* dK, const float* dV,
                                          const float* d_sigma, const float* d_beta,
                                          int Z, int H, int N, int d_head, float min_rbf, float max_rbf)
{
    (void)key_pad_mask; (void)d_sigma; (void)d_beta;
    if (!Q || !K || !V || !dO || !coords || !sigma || !L || !D || !dQ || !dK || !dV) return PROTEUS_ERR_NULL_POINTER;
    if (Z <= 0 || H <= 0 || N <= 0) return PROTEUS_ERR_BAD_SHAPE;
    if (N > PROTEUS_ATTN_MAX_N || (long)Z * H > 65535) return PROTEUS_ERR_BAD_SHAPE;
    if (d_head != GB_D) return PROTEUS_ERR_BAD_HEAD_DIM;
    if (beta && !(max_rbf > min_rbf)) return PROTEUS_ERR_BAD_SHAPE;
    if (((uintptr_t)Q & 15) || ((uintptr_t)K & 15) || ((uintptr_t)V & 15) || ((uintptr_t)dO & 15) ||
        ((uintptr_t)dQ & 15) || ((uintptr_t)dK & 15) || ((uintptr_t)dV & 15)) return PROTEUS_ERR_BAD_ALIGNMENT;
    return PROTEUS_OK;
}

extern "C" int proteus_geo_attn_bwd(const uint16_t* Q, const uint16_t* K, const uint16_t* V, const uint16_t* dO,
                                    const float* coords, const float* sigma, const float* beta,
                                    const uint8_t* key_pad_mask, const float* L, const float* D,
                                    float* dQ, float* dK, float* dV, float* d_sigma, float* d_beta,
                                    int Z, int H, int N, int d_head, float min_rbf, float max_rbf, void* stream)
{
    const int rc = proteus_geo_attn_bwd_check(Q, K, V, dO, coords, sigma, beta, key_pad_mask, L, D, dQ, dK, dV,
                                              d_sigma, d_beta, Z, H, N, d_head, min_rbf, max_rbf);
    if (rc != PROTEUS_OK) return rc;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    if (beta)
        return launch_bwd<true>(Q, K, V, dO, coords, sigma, beta, key_pad_mask, L, D, dQ, dK, dV, d_sigma, d_beta,
                                Z, H, N, min_rbf, max_rbf, contiguous_strides(H, N), st);
    return launch_bwd<false>(Q, K, V, dO, coords, sigma, nullptr, key_pad_mask, L, D, dQ, dK, dV, d_sigma, nullptr,
                             Z, H, N, 0.f, 1.f, contiguous_strides(H, N), st);
}

extern "C" int proteus_geo_attn_bwd_strided_check(const uint16_t* Q, const uint16_t* K, const uint16_t* V, const uint16_t* dO,
                                                  const int64_t* strides,
                                                  const float* coords, const float* sigma, const float* beta,
                                                  const uint8_t* key_pad_mask, const float* L, const float* D,
                                                  const float* dQ, const float* dK, const float* dV,
                                                  const float* d_sigma, const float* d_beta,
                                                  int Z, int H, int N, int d_head, float min_rbf, float max_rbf)
{
    const int rc = proteus_geo_attn_bwd_check(Q, K, V, dO, coords, sigma, beta, key_pad_mask, L, D, dQ, dK, dV,
                                              d_sigma, d_beta, Z, H, N, d_head, min_rbf, max_rbf);
    if (rc != PROTEUS_OK) return rc;
    GbStrides gs;
    return strides_from(strides, Z, H, N, gs);
}

extern "C" int proteus_geo_attn_bwd_strided(const uint16_t* Q, const uint16_t* K, const uint16_t* V, const uint16_t* dO,
                                            const int64_t* strides,
                                            const float* coords, const float* sigma, const float* beta,
                                            const uint8_t* key_pad_mask, const float* L, const float* D,
                                            float* dQ, float* dK, float* dV, float* d_sigma, float* d_beta,
                                            int Z, int H, int N, int d_head, float min_rbf, float max_rbf, void* stream)
{
    int rc = proteus_geo_attn_bwd_check(Q, K, V, dO, coords, sigma, beta, key_pad_mask, L, D, dQ, dK, dV,
                                        d_sigma, d_beta, Z, H, N, d_head, min_rbf, max_rbf);
    if (rc != PROTEUS_OK) return rc;
    GbStrides gs;
    rc = strides_from(strides, Z, H, N, gs);
    if (rc != PROTEUS_OK) return rc;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    if (beta)
        return launch_bwd<true>(Q, K, V, dO, coords, sigma, beta, key_pad_mask, L, D, dQ, dK, dV, d_sigma, d_beta,
                                Z, H, N, min_rbf, max_rbf, gs, st);
    return launch_bwd<false>(Q, K, V, dO, coords, sigma, nullptr, key_pad_mask, L, D, dQ, dK, dV, d_sigma, nullptr,
                             Z, H, N, 0.f, 1.f, gs, st);
}
