// Wave-level Hadamard building block for gfx950: transforms the 9 low index bits of a
// 512-element tile on the matrix cores, with no cross-lane data movement.
//
// Role of the reference's device-callable seam
//   HadamardTransform<dtype,N>::hadamard_transform_device(in, out, sm)   csrc/hada_handler.cuh:227-264
// but built for 64-wide wavefronts and MFMA register layouts rather than mma.sync fragments.
//
// Layout algebra.  One wavefront holds a tile of 512 elements, 8 per lane.  Name the lane bits
// lo = lane & 15, hi = lane >> 4 and the per-lane slot j = 0..7.  A *tile map* says which element
// index bit each of those positions carries:
//     2-byte elements:  j -> e0 e1 e2,   lo -> e3..e6,   hi -> e7 e8   (lane l holds e = 8l + j)
//     4-byte elements:  j -> e0 e1 e8,   lo -> e2..e5,   hi -> e6 e7   (two 16-byte loads / lane)
// Stage 1 is v_mfma_f32_16x16x32 with the data as the A operand (row = lo, K = 8*hi + j) and a
// masked Hadamard matrix G1 as B.  It transforms the five K bits and, because the MFMA result
// layout puts rows on (hi, r) and columns on lo, it leaves the untouched lo bits on (hi, r).
// Stage 2 is v_mfma_f32_16x16x16 with the stage-1 result reused *as the A operand* (which reads
// it transposed) against G2: it transforms those four bits and moves the stage-1 bits back to
// (hi, r).  The column order of G1 is chosen so that after stage 2 lane l again holds
// e = 8l + j (resp. the 4-byte map): the result layout equals the load layout, stores are
// 16-byte and coalesced, and in-place operation is safe.
//
// Bits >= log2(n) are masked out of G1/G2 (identity), so one tile can hold several short rows.
// Both stages carry a power-of-two factor (exact) that keeps 16-bit intermediates in range; the
// caller folds the inverse into its output scale (tile_stage_shift, split_output_scale).
#pragma once

#include <type_traits>

#include "common.hpp"

namespace mi {

template <int ESIZE>
struct TileMap;

template <>
struct TileMap<2> {
    // element bit carried by canonical stage-1 bit q (q0..q2 = j bits, q3..q4 = hi bits)
    static constexpr int qe[5] = {0, 1, 2, 7, 8};
    static constexpr int lo_e0 = 3;  // lo bits carry e3..e6
};

template <>
struct TileMap<4> {
    static constexpr int qe[5] = {0, 1, 8, 6, 7};
    static constexpr int lo_e0 = 2;  // lo bits carry e2..e5
};

// Masks of the stage-1 (5 canonical bits) and stage-2 (4 bits) index bits that lie inside a
// transform of length 2^p.
template <int ESIZE>
__host__ __device__ inline void tile_masks(uint32_t p, uint32_t& mask1, uint32_t& mask2)
{
    constexpr int qe[5] = {TileMap<ESIZE>::qe[0], TileMap<ESIZE>::qe[1], TileMap<ESIZE>::qe[2],
                           TileMap<ESIZE>::qe[3], TileMap<ESIZE>::qe[4]};
    mask1 = 0;
    for (int b = 0; b < 5; ++b)
        if ((uint32_t)qe[b] < p) mask1 |= 1u << b;
    mask2 = 0;
    for (int b = 0; b < 4; ++b)
        if ((uint32_t)(TileMap<ESIZE>::lo_e0 + b) < p) mask2 |= 1u << b;
}

// Splits the factor that must follow the two MFMA stages, scale * 2^tile_stage_shift(p), into a
// power of two folded into the stage-2 operand (exp2, kept small enough for fp16 operands) and a
// residual multiplier (1.0f exactly when the scale is a power of two).
struct OutputScale {
    int exp2;
    float mult;
};
inline OutputScale split_output_scale(double scale, int stage_shift)
{
    OutputScale r{0, 1.0f};
    const double f = scale * (double)(1u << stage_shift);
    if (!(f > 0.0) || f != f || f > 1e30) {  // zero, negative, NaN, huge: plain multiplier
        r.mult = (float)f;
        return r;
    }
    int e;
    (void)__builtin_frexp(f, &e);  // f = m * 2^e, m in [0.5, 1)
    e -= 1;                        // f = (2m) * 2^e, 2m in [1, 2)
    const int ec = e < -10 ? -10 : (e > 10 ? 10 : e);
    r.exp2 = ec;
    r.mult = (float)(f / __builtin_ldexp(1.0, ec));
    return r;
}

// log2 of the attenuation of stage 1 over k index bits.  bf16 operands: 2^-(k/2), the square root
// of the stage's gain.  fp16 operands (`narrow_range`): 2^-(k-1), so that the 16-bit value between
// the stages, a sum of 2^k inputs, never exceeds twice the largest input; with the square-root
// factor an input pattern that the full transform spreads out could already overflow fp16 there
// (partial sums up to 8x the largest input at k = 5).
__host__ __device__ inline int stage1_shift(int k, bool narrow_range)
{
    return narrow_range && k > 1 ? k - 1 : k >> 1;
}

// log2 of the (power-of-two) attenuation the two MFMA stages apply for a transform of length 2^p.
// `narrow_range`: the matrix-core operand type is fp16 (see stage1_shift).
template <int ESIZE>
__host__ __device__ inline int tile_stage_shift(uint32_t p, bool narrow_range)
{
    uint32_t m1, m2;
    tile_masks<ESIZE>(p, m1, m2);
    return stage1_shift(__builtin_popcount(m1), narrow_range) + (__builtin_popcount(m2) >> 1);
}
template <class T16>
constexpr bool kNarrowRange = std::is_same<T16, F16>::value;

// Per-lane Hadamard operands for the two stages.
template <class T16>
struct TileOperands {
    typename T16::V8 g1[2];  // stage-1 B operand for output halves t = 0, 1
    typename T16::V4 g2;     // stage-2 B operand
};

// `exp2` is an extra power-of-two factor folded (exactly) into the stage-2 operand, so that a
// power-of-two output scale costs no multiply at all.
template <class T16, int ESIZE>
__device__ __forceinline__ void make_tile_operands(uint32_t p, TileOperands<T16>& ops, int exp2 = 0)
{
    using E = typename T16::E;
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t lo = lane & 15u, hi = lane >> 4;
    uint32_t mask1, mask2;
    tile_masks<ESIZE>(p, mask1, mask2);
    const float c1 = __builtin_ldexpf(1.0f, -stage1_shift(__popc(mask1), kNarrowRange<T16>));
    const float c2 = __builtin_ldexpf(1.0f, exp2 - (__popc(mask2) >> 1));
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        const uint32_t np = 16u * t + lo;  // stage-1 output column
        // column -> canonical bits: n'0->q0, n'1->q1, n'2->q3, n'3->q4, n'4->q2
        const uint32_t qn = (np & 3u) | (((np >> 2) & 1u) << 3) | (((np >> 3) & 1u) << 4) |
                            (((np >> 4) & 1u) << 2);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const uint32_t qk = 8u * hi + j;
            ops.g1[t][j] = (E)masked_hadamard_entry(qk, qn, mask1, c1);
        }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) ops.g2[j] = (E)masked_hadamard_entry(4u * hi + j, lo, mask2, c2);
}

template <class T16>
__device__ __forceinline__ typename T16::V4 narrow4(f32x4 v)
{
    using E = typename T16::E;
    typename T16::V4 r;
    r[0] = (E)v[0];
    r[1] = (E)v[1];
    r[2] = (E)v[2];
    r[3] = (E)v[3];
    return r;
}

// 16-bit tile: `a` = the lane's 8 elements.  Result acc[t][r] = element 8*lane + 4t + r.
template <class T16>
__device__ __forceinline__ void tile_transform(typename T16::V8 a, const TileOperands<T16>& ops,
                                               f32x4 (&acc)[2])
{
    const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        f32x4 d1 = T16::mfma32(a, ops.g1[t], zero);
        acc[t] = T16::mfma16(narrow4<T16>(d1), ops.g2, zero);
    }
}

// Exact three-way split of fp32 values into bf16 pieces (8 + 8 + 8 significand bits), x = h + m + l,
// for the eight elements of a tile operand.  By truncation: h = the upper 16 bits of x, m = the
// upper 16 bits of x - h, l = x - h - m, which has at most eight significant bits left and is
// therefore a bf16 value itself.  Every subtraction is exact; per value that is two ANDs, two
// subtractions and one and a half byte permutes, all full-rate vector instructions (rounding
// conversions to bf16 take three times as long).
struct SplitTileF32 {
    bf16x8 h, m, l;
};
__device__ __forceinline__ void split_tile_f32(const float (&v)[8], SplitTileF32& s)
{
    u32x4 hp, mp, lp;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        uint32_t h[2], m[2], l[2];
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const float x = v[2 * j + e];
            h[e] = __float_as_uint(x) & 0xffff0000u;
            const float r = x - __uint_as_float(h[e]);
            m[e] = __float_as_uint(r) & 0xffff0000u;
            l[e] = __float_as_uint(r - __uint_as_float(m[e]));
        }
        // upper halves of two values into one register, the first value in the lower half
        hp[j] = __builtin_amdgcn_perm(h[1], h[0], 0x07060302u);
        mp[j] = __builtin_amdgcn_perm(m[1], m[0], 0x07060302u);
        lp[j] = __builtin_amdgcn_perm(l[1], l[0], 0x07060302u);
    }
    s.h = __builtin_bit_cast(bf16x8, hp);
    s.m = __builtin_bit_cast(bf16x8, mp);
    s.l = __builtin_bit_cast(bf16x8, lp);
}

// fp32 tile.  Stage 1 runs on the bf16 matrix cores: the three bf16 pieces of every input are
// multiplied by the +-2^-k Hadamard operand and accumulated in fp32, so each product is exact and
// the only rounding is the fp32 accumulation.  Stage 2 takes the fp32 sums as they are, as the A
// operand of four v_mfma_f32_16x16x4_f32 (MFMA r contracts index 4 hi + r: A[lo][hi] = d1[r],
// B[hi][lo] = G2[4 hi + r][lo]); again every product is exact.  That costs 128 matrix-core cycles
// per half tile instead of 48, and saves the second three-way split, half of the vector
// arithmetic of the tile, which is what bounds the callers that transform many tiles per
// wavefront.  v[j] = the lane's 8 elements under TileMap<4>.
// Result acc[t][r] = element 256t + 4*lane + r.
__device__ __forceinline__ void tile_transform_f32(const float (&v)[8],
                                                   const TileOperands<BF16>& ops, f32x4 (&acc)[2])
{
    SplitTileF32 s;
    split_tile_f32(v, s);
    float g2f[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) g2f[r] = (float)ops.g2[r];
    const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        f32x4 d1 = BF16::mfma32(s.l, ops.g1[t], zero);
        d1 = BF16::mfma32(s.m, ops.g1[t], d1);
        d1 = BF16::mfma32(s.h, ops.g1[t], d1);
        f32x4 d2 = __builtin_amdgcn_mfma_f32_16x16x4f32(d1[0], g2f[0], zero, 0, 0, 0);
        d2 = __builtin_amdgcn_mfma_f32_16x16x4f32(d1[1], g2f[1], d2, 0, 0, 0);
        d2 = __builtin_amdgcn_mfma_f32_16x16x4f32(d1[2], g2f[2], d2, 0, 0, 0);
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(d1[3], g2f[3], d2, 0, 0, 0);
    }
}

// The MFMA part of the same transform for a pair of tiles, for a caller that runs one wavefront
// per SIMD and overlaps the pieces by hand: `split_tile_f32` is pure vector arithmetic (it can sit
// in the shadow of another pair's MFMAs), `tile_pair_mfma_f32` issues the four MFMA chains of the
// pair (2 tiles x 2 halves) round-robin, so that every MFMA depends on one issued four slots
// earlier rather than on its predecessor.  (tile_transform_f32 called twice leaves the seven
// MFMAs of each chain back to back, each waiting for the one before: about 1100 cycles per tile
// on a lone wavefront.)  Results are bit-identical to tile_transform_f32.
__device__ __forceinline__ void tile_pair_mfma_f32(const SplitTileF32 (&s)[2], const TileOperands<BF16>& ops,
                                                   f32x4 (&acc)[2][2])
{
    // scheduling fence for MFMAs only: vector, scalar and memory instructions may cross it
    constexpr int kKeepMfmaOrder = 0x3f6;
    float g2f[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) g2f[r] = (float)ops.g2[r];
    const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
    f32x4 d1[2][2];
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
        for (int t = 0; t < 2; ++t) d1[c][t] = BF16::mfma32(s[c].l, ops.g1[t], zero);
    __builtin_amdgcn_sched_barrier(kKeepMfmaOrder);
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
        for (int t = 0; t < 2; ++t) d1[c][t] = BF16::mfma32(s[c].m, ops.g1[t], d1[c][t]);
    __builtin_amdgcn_sched_barrier(kKeepMfmaOrder);
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
        for (int t = 0; t < 2; ++t) d1[c][t] = BF16::mfma32(s[c].h, ops.g1[t], d1[c][t]);
    __builtin_amdgcn_sched_barrier(kKeepMfmaOrder);
#pragma unroll
    for (int r = 0; r < 4; ++r) {
#pragma unroll
        for (int c = 0; c < 2; ++c)
#pragma unroll
            for (int t = 0; t < 2; ++t)
                acc[c][t] = __builtin_amdgcn_mfma_f32_16x16x4f32(d1[c][t][r], g2f[r], r ? acc[c][t] : zero, 0, 0, 0);
        __builtin_amdgcn_sched_barrier(kKeepMfmaOrder);
    }
}
// In-register butterflies over XB tile-index bits (element bits 9 .. 9+XB-1) of NT tiles.
template <int NT, int XB>
__device__ __forceinline__ void cross_tile_butterflies(f32x4 (&acc)[NT][2])
{
#pragma unroll
    for (int b = 0; b < XB; ++b) {
#pragma unroll
        for (int c = 0; c < NT; ++c) {
            if (c & (1 << b)) continue;
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                const f32x4 x = acc[c][t], y = acc[c | (1 << b)][t];
                acc[c][t] = x + y;
                acc[c | (1 << b)][t] = x - y;
            }
        }
    }
}

}  // namespace mi
