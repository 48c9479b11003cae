// Pieces shared by the 16-bit register-resident fused GEMM kernels (fused_gemm_xreg.hip,
// fused_gemm_xreg_k2048.hip): the MFMA with its B operand in the accumulation-register file and the
// column transforms of the prologue.
#pragma once
#include "xreg_common.hpp"

namespace mi {
namespace xreg {

// acc (+)= A(16 x 32) * B(32 x 16) with B read straight from the accumulation-register file, where
// the transformed operand lives for the whole kernel, and the accumulator in ordinary registers.
// Inline assembly because the compiler, left to itself, copies register-file-resident operands
// into ordinary registers before every use (v_accvgpr_read, four per fragment), and those copies
// wait for the matrix-core pipeline.  What the compiler no longer sees: the result is written when
// the instruction retires, not when it issues; readers of `c` other than the next accumulate must
// come at least one more MFMA (or drain_mfma()) later.
template <class T16>
struct XMfma;
template <>
struct XMfma<BF16> {
    static __device__ __forceinline__ void first(f32x4& c, bf16x8 a, bf16x8 b)
    {
        asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, 0" : "=v"(c) : "v"(a), "a"(b));
    }
    static __device__ __forceinline__ void next(f32x4& c, bf16x8 a, bf16x8 b)
    {
        asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "a"(b));
    }
    // adds a pair of adjacent 16-bit values to memory (performed in the L2, nothing returned)
    static __device__ __forceinline__ void add_pair_to_memory(uint32_t lane_off, uint32_t v, void* base)
    {
        asm volatile("global_atomic_pk_add_bf16 %0, %1, %2" ::"v"(lane_off), "v"(v), "s"(base) : "memory");
    }
};
template <>
struct XMfma<F16> {
    static __device__ __forceinline__ void first(f32x4& c, f16x8 a, f16x8 b)
    {
        asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, 0" : "=v"(c) : "v"(a), "a"(b));
    }
    static __device__ __forceinline__ void next(f32x4& c, f16x8 a, f16x8 b)
    {
        asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "a"(b));
    }
    static __device__ __forceinline__ void add_pair_to_memory(uint32_t lane_off, uint32_t v, void* base)
    {
        asm volatile("global_atomic_pk_add_f16 %0, %1, %2" ::"v"(lane_off), "v"(v), "s"(base) : "memory");
    }
};
// the same for one fp32 value, `offset` bytes behind the lane's address
__device__ __forceinline__ void add_f32_to_memory(uint32_t lane_off, float v, void* base, int offset)
{
    asm volatile("global_atomic_add_f32 %0, %1, %2 offset:%3" ::"v"(lane_off), "v"(v), "s"(base), "i"(offset) : "memory");
}

// A column = two 512-element tiles.  Stage 1 as in tile_transform; stage 2 contracts the two
// tiles' stage-1 results together (K = 32: 16 stage-2 inputs of each tile) against [G2; +G2] and
// [G2; -G2], which yields the transform of the first and of the second half of the column (the
// butterfly over element bit 9) without any vector arithmetic.
template <class T16>
struct PairOperands {
    typename T16::V8 g1[2];
    typename T16::V8 g2s, g2d;
};

template <class T16>
__device__ __forceinline__ void make_pair_operands(PairOperands<T16>& po, int exp2)
{
    TileOperands<T16> ops;
    make_tile_operands<T16, 2>(10, ops, exp2);
    po.g1[0] = ops.g1[0];
    po.g1[1] = ops.g1[1];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        po.g2s[j] = ops.g2[j];
        po.g2s[4 + j] = ops.g2[j];
        po.g2d[j] = ops.g2[j];
        po.g2d[4 + j] = -ops.g2[j];
    }
}

// lo_half / hi_half: lane l's elements 8l .. 8l+7 of H_1024 (x) restricted to k < 512 / k >= 512
template <class T16>
__device__ __forceinline__ void column_transform(typename T16::V8 t0, typename T16::V8 t1,
                                                 const PairOperands<T16>& po,
                                                 typename T16::V8& lo_half, typename T16::V8& hi_half)
{
    using E = typename T16::E;
    const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const f32x4 d0 = T16::mfma32(t0, po.g1[h], zero);
        const f32x4 d1 = T16::mfma32(t1, po.g1[h], zero);
        typename T16::V8 a2;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            a2[r] = (E)d0[r];
            a2[4 + r] = (E)d1[r];
        }
        const f32x4 s = T16::mfma32(a2, po.g2s, zero);
        const f32x4 d = T16::mfma32(a2, po.g2d, zero);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            lo_half[4 * h + r] = (E)s[r];
            hi_half[4 * h + r] = (E)d[r];
        }
    }
}

// The same without the final rounding: s[h] / d[h] hold elements 4h .. 4h+3 of the lane's eight for
// the first / second half (K = 2048 adds one more butterfly, between two such pairs, in fp32).
template <class T16>
__device__ __forceinline__ void column_pair_f32(typename T16::V8 t0, typename T16::V8 t1,
                                                const PairOperands<T16>& po, f32x4 (&s)[2],
                                                f32x4 (&d)[2])
{
    using E = typename T16::E;
    const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const f32x4 d0 = T16::mfma32(t0, po.g1[h], zero);
        const f32x4 d1 = T16::mfma32(t1, po.g1[h], zero);
        typename T16::V8 a2;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            a2[r] = (E)d0[r];
            a2[4 + r] = (E)d1[r];
        }
        s[h] = T16::mfma32(a2, po.g2s, zero);
        d[h] = T16::mfma32(a2, po.g2d, zero);
    }
}

// The same for the sum (NEGATE = false) or difference (true) of two 1024-element columns, formed in
// the accumulators of stage 1 (which is linear), so that the 16-bit value between the stages is
// rounded once and stage 2 runs once: s, d = halves of H_1024 (x +- y), x = [t0; t1], y = [u0; u1].
template <class T16, bool NEGATE>
__device__ __forceinline__ void column_pair_combined_f32(typename T16::V8 t0, typename T16::V8 t1,
                                                         typename T16::V8 u0, typename T16::V8 u1,
                                                         const PairOperands<T16>& po, f32x4 (&s)[2],
                                                         f32x4 (&d)[2])
{
    using E = typename T16::E;
    const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        // (sign bits flipped: exact for either 16-bit type)
        const u32x4 flip = {0x80008000u, 0x80008000u, 0x80008000u, 0x80008000u};
        const typename T16::V8 g1y =
            NEGATE ? __builtin_bit_cast(typename T16::V8, __builtin_bit_cast(u32x4, po.g1[h]) ^ flip) : po.g1[h];
        const f32x4 d0 = T16::mfma32(u0, g1y, T16::mfma32(t0, po.g1[h], zero));
        const f32x4 d1 = T16::mfma32(u1, g1y, T16::mfma32(t1, po.g1[h], zero));
        typename T16::V8 a2;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            a2[r] = (E)d0[r];
            a2[4 + r] = (E)d1[r];
        }
        s[h] = T16::mfma32(a2, po.g2s, zero);
        d[h] = T16::mfma32(a2, po.g2d, zero);
    }
}

}  // namespace xreg
}  // namespace mi
