// Helpers shared by the MFMA decode kernels (gfx950, wave64).
//
// v_mfma_f32_16x16x32_f16 operand layout, lane l, n = l % 16, blk = l / 16:
//   A[i = n][k = 8*blk + j]   j = 0..7 (eight fp16 per lane)
//   B[k = 8*blk + j][n]
//   D[i = 4*blk + r][n]       r = 0..3 (four fp32 per lane)
// MFMA sums over k, so any assignment of channels (tokens) to k-slots is valid as
// long as A and B agree.
#pragma once
#include "attend.hpp"

namespace vq {

typedef uint32_t u32;
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ f16x2 as_h2(u32 u) { return __builtin_bit_cast(f16x2, u); }
__device__ __forceinline__ u32 as_u(f16x2 h) { return __builtin_bit_cast(u32, h); }
__device__ __forceinline__ f16x8 as_h8(u32 a, u32 b, u32 c, u32 d) {
    u32x4 v = {a, b, c, d};
    return __builtin_bit_cast(f16x8, v);
}
__device__ __forceinline__ f16x8 as_h8(uint4 v) { return as_h8(v.x, v.y, v.z, v.w); }
__device__ __forceinline__ f16x2 h2(float a) { f16x2 r = {(f16)a, (f16)a}; return r; }
// A constant the optimiser must keep in a vector register, so that
// (w & mask) | magic becomes one v_and_or_b32 (mask in a scalar register).
__device__ __forceinline__ u32 vreg_const(u32 x) { asm volatile("" : "+v"(x)); return x; }
// {lo half of a, lo half of b} and {hi half of a, hi half of b}
__device__ __forceinline__ u32 pair_lo(u32 a, u32 b) { return __builtin_amdgcn_perm(b, a, 0x05040100u); }
__device__ __forceinline__ u32 pair_hi(u32 a, u32 b) { return __builtin_amdgcn_perm(b, a, 0x07060302u); }

constexpr int MF_ROWS = 16;               // M/N width of the MFMA
constexpr int MF_D = 128;                 // head dim
constexpr int MF_PART = MF_D + 2;         // floats per partial: max, sum, accumulator
constexpr float LOG2E = 1.4426950408889634f;
constexpr float LN2 = 0.6931471805599453f;
// The softmax reference point only has to stay within this many log2 units of the
// true running maximum: P may then reach 2^RESCALE_SLACK, far inside fp16 range, and
// the accumulators are rescaled a handful of times per wave instead of every time a
// row's maximum creeps up.
constexpr float RESCALE_SLACK = 8.0f;

// Magic constants: an fp16 whose mantissa field receives the code.  A 4-bit code
// in mantissa bits 4..7 of 64.0 reads 64 + code; a 2-bit code in bits 6..7 of 16.0
// reads 16 + code.
template <int BITS> struct Magic {
    static constexpr u32 bits = BITS == 4 ? 0x54005400u : 0x4C004C00u;
    static constexpr u32 mask = BITS == 4 ? 0x00F000F0u : 0x00C000C0u;
    static constexpr float off = BITS == 4 ? 64.f : 16.f;
    static constexpr u32 neg_off_pair = BITS == 4 ? 0xD400D400u : 0xCC00CC00u;   // {-off, -off}
};

// Eight codes of one packed word as fp16 values (offset + code), in k-slot pair order.
// BITS == 4: the word holds codes 0..7, pair p = (code p, code p + 4).
// BITS == 2: `w` is the word shifted right by 8*half; it then holds codes
//            4*half + 0..3 and 4*half + 8..11 in its two byte lanes, pair p =
//            (code 4*half + p, code 4*half + p + 8).
// The offset is NOT removed here: an MFMA against a constant operand accounts for it.
template <int BITS> __device__ __forceinline__ f16x8 unpack8(u32 w, u32 magic) {
    constexpr u32 mask = Magic<BITS>::mask;
    u32 r0, r1, r2, r3;
    if (BITS == 4) {
        r0 = ((w << 4) & mask) | magic;
        r1 = (w & mask) | magic;
        r2 = ((w >> 4) & mask) | magic;
        r3 = ((w >> 8) & mask) | magic;
    } else {
        r0 = ((w << 6) & mask) | magic;
        r1 = ((w << 4) & mask) | magic;
        r2 = ((w << 2) & mask) | magic;
        r3 = (w & mask) | magic;
    }
    return as_h8(r0, r1, r2, r3);
}

// channel (0..31 inside a lane's 32-channel slice) of k-slot pair p of k-step ks
template <int BITS> __device__ __forceinline__ constexpr int kchan_lo(int ks, int p) {
    return BITS == 4 ? 8 * ks + p : 16 * (ks / 2) + 4 * (ks % 2) + p;
}
template <int BITS> __device__ __forceinline__ constexpr int kchan_hi(int ks, int p) {
    return kchan_lo<BITS>(ks, p) + (BITS == 4 ? 4 : 8);
}
// token (0..31 inside a unit) of k-slot pair p of lane group blk in the P.V product
template <int BITS> __device__ __forceinline__ constexpr int vtok_lo(int blk, int p) {
    return BITS == 4 ? 8 * blk + p : 16 * (blk / 2) + 4 * (blk % 2) + p;
}
template <int BITS> __device__ __forceinline__ constexpr int vtok_gap() { return BITS == 4 ? 4 : 8; }

__device__ __forceinline__ float ldq(const void *p, int tag, int64_t i) {
    if (tag == VQ_F16) return (float)((const f16 *)p)[i];
    if (tag == VQ_BF16) return bf16_to_f32(((const u16 *)p)[i]);
    return ((const float *)p)[i];
}

__device__ __forceinline__ f16x8 ones8() { return as_h8(0x3C003C00u, 0x3C003C00u, 0x3C003C00u, 0x3C003C00u); }

// value of lane (lane + N) of the same 16-lane row, 0 past the row's end
template <int N> __device__ __forceinline__ float row_shl(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x100 + N, 0xF, 0xF, true));
}

// load through a block-uniform base plus a 32-bit per-lane byte offset
template <typename T> __device__ __forceinline__ T ldg(const char *base, u32 off) {
    return *reinterpret_cast<const T *>(base + off);
}

// launchers of the two kernels (packed prefix, fp16 tail); each writes (max, sum, accumulator)
// partials [rows][nparts][MF_PART] that the shared merge kernel combines
void launch_mfma_tail(const vq_attend_args &a, int nsplit, int nparts, float *ws, hipStream_t st);
void launch_mfma_packed_f16meta(const vq_attend_args &a, int nsplit, int64_t split_len, int nparts, float *ws, hipStream_t st);
void launch_mfma_packed_f32meta(const vq_attend_args &a, int nsplit, int64_t split_len, int nparts, float *ws, hipStream_t st);

}  // namespace vq
