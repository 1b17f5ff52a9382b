// Operand types of the attention kernels' matrix products: bf16 (default) or fp16 (the reference casts Q, K, V to
// fp16, old/old_scripts/attn/geometric_attn.py:567-569).  Both are 16-bit patterns in memory and in LDS; only the
// matrix instruction, the conversions to the type and the row sum of packed pairs differ.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace proteus_ops {

typedef __bf16   bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16   bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8  __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2  __attribute__((ext_vector_type(2)));
typedef float    floatx16 __attribute__((ext_vector_type(16)));
typedef float    floatx2  __attribute__((ext_vector_type(2)));

template <bool F16> struct Operand;

template <> struct Operand<false> {
    typedef bf16x8 vec8;
    // largest exponential (log2 units) a lazily re-based softmax may hold before it re-bases, and the row-sum alarm
    static constexpr float REBASE = 20.0f, REBASE_SUM = 16777216.0f;
    static __device__ __forceinline__ floatx16 mfma(const uint4 a, const vec8 b, const floatx16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ unsigned pack(const float a, const float b) {
        const floatx2 f = {a, b};
        return __builtin_bit_cast(unsigned, __builtin_convertvector(f, bf16x2));
    }
    // c + the two values packed in w (v_dot2 against ones)
    static __device__ __forceinline__ float add_packed(const unsigned w, const float c) {
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, w), __builtin_bit_cast(bf16x2, 0x3f803f80u), c, false);
    }
    // eight raw elements times a power of two (exact)
    static __device__ __forceinline__ vec8 scaled(const uint4 raw, const float s) {
        bf16x8 v = __builtin_bit_cast(bf16x8, raw);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = (__bf16)((float)v[e] * s);
        return v;
    }
    static __device__ __forceinline__ vec8 raw8(const uint4 raw) { return __builtin_bit_cast(bf16x8, raw); }
};

template <> struct Operand<true> {
    typedef f16x8 vec8;
    // fp16 ends at 65504: exponentials stay below 2^14
    static constexpr float REBASE = 10.0f, REBASE_SUM = 16384.0f;
    static __device__ __forceinline__ floatx16 mfma(const uint4 a, const vec8 b, const floatx16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ unsigned pack(const float a, const float b) {
        const floatx2 f = {a, b};
        return __builtin_bit_cast(unsigned, __builtin_convertvector(f, f16x2));      // round to nearest even
    }
    static __device__ __forceinline__ float add_packed(const unsigned w, const float c) {
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, w), __builtin_bit_cast(f16x2, 0x3c003c00u), c, false);
    }
    static __device__ __forceinline__ vec8 scaled(const uint4 raw, const float s) {
        f16x8 v = __builtin_bit_cast(f16x8, raw);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = (_Float16)((float)v[e] * s);
        return v;
    }
    static __device__ __forceinline__ vec8 raw8(const uint4 raw) { return __builtin_bit_cast(f16x8, raw); }
};

// S = (q . k)/sqrt(d) with q pre-multiplied by the power of two QS (exact in either type) and the remaining factor
// RHO = 1/(sqrt(d) QS) (1 or 2^-1/2) applied to the fp32 product.
template <int D> struct HeadDim;
template <> struct HeadDim<32>  { static constexpr float QS = 0.25f,  RHO = 0.70710678118654752f, INV_SQRT = 0.17677669529663688f; };
template <> struct HeadDim<64>  { static constexpr float QS = 0.125f, RHO = 1.0f,                 INV_SQRT = 0.125f; };
template <> struct HeadDim<128> { static constexpr float QS = 0.125f, RHO = 0.70710678118654752f, INV_SQRT = 0.08838834764831845f; };

// XOR swizzle of the 16-byte chunks of a row-major LDS tile of 16-bit elements with rows of 2 D bytes (chunk c of
// row r sits at slot c ^ tile_swizzle<D>(r)), under which both kinds of reads are free of bank conflicts (64 banks of
// 4 bytes):
//  * 16-byte fragment reads: 16 lanes read one chunk of 16 consecutive rows;
//  * transposing reads (ds_read_b64_tr_b16): 16 lanes read 32 bytes (an even chunk and the next) of four consecutive
//    rows, aligned to four.
// d = 32 (64-byte rows: rows r, r+4, r+8, r+12 share banks): (r >> 2) & 3.
// d = 64 (128-byte rows: the even and the odd rows each share banks): the 8 even and the 8 odd rows of 16 consecutive
//   ones get 8 different values, and rows r, r + 2 of an aligned group of four differ in bits 1..2.
// d = 128 (256-byte rows: all rows share banks): a permutation of r & 15 whose upper three bits differ among four
//   consecutive rows.
template <int D> __device__ __forceinline__ int tile_swizzle(int r);
template <> __device__ __forceinline__ int tile_swizzle<32>(int r)  { return (r >> 2) & 3; }
template <> __device__ __forceinline__ int tile_swizzle<64>(int r)  { return (((r >> 1) & 1) << 2) | ((r >> 2) & 3); }
template <> __device__ __forceinline__ int tile_swizzle<128>(int r) { return ((r & 3) << 2) | ((r >> 2) & 3); }

}  // namespace proteus_ops
