// Randomized Hadamard + FP8 (OCP E4M3FN) quantize epilogue (mi_rht_quant_fp8), gfx950.  The
// reference has no FP8 path; the arithmetic convention is the one stated in include/mi_hadamard.h.
//
// Quantize kernel: the stand-alone transform's tiles (one 16-byte load per 8 elements, two MFMA
// stages per 512-element tile) with
//   - the +-1 diagonal folded into the load as a sign-bit XOR (exact), its masks kept in LDS (they
//     are the same for every row),
//   - for n > 512 the butterflies between a row's tiles folded into the second MFMA stage: output
//     tile o is the sum over tile pairs of [a(2i); a(2i+1)] contracted with [+-G2; +-G2], the signs
//     (-1)^popcount(o & tile), accumulated on the matrix cores (no vector add/sub at all),
//   - the result rounded to bf16 as mi_fwht would store it, the row amax taken on the fp32 values
//     by a lane reduction over the lanes that share a row,
//   - v_cvt_pk_fp8_f32 for the narrowing (hardware RNE to E4M3FN), 8 codes = one 8-byte store.
// Two costs set the kernel's time at [8192, 4096].  Vector-instruction issue: a SIMD needs about
// 1.0 us per row of 4096 with two or more wavefronts resident (1.4 us with one), 8 rows per SIMD;
// hence four wavefronts per SIMD (at most 128 registers: simple two-operand instructions then issue
// every 2.2 cycles per SIMD, conversions and three-operand ones every 4.3; with three wavefronts
// 2.7 and 5.2) and as few vector instructions per element as the arithmetic allows.  And the memory
// system: 100.7 MB per launch at the 6.6 - 7.0 TB/s that a read + write mix of this size reaches on
// this chip are 14 - 15 us, which is what the span from the first wavefront's start to the last
// one's end measures (15.4 us); prefetching rows, other workgroup sizes and handing rows out
// dynamically all moved work between wavefronts without changing that total.
#include <type_traits>

#include "fwht_device.hpp"

namespace mi {
namespace {

constexpr float kFp8Max = 448.0f;
constexpr float kAmaxFloor = 1e-30f;

// Maximum over the lanes that differ only in their low `bits` lane-index bits (bits <= 6), with
// data-parallel primitives only: quad permutes and row mirrors for 1, 2, 4, 8 (after each step
// the value is uniform over the group already reduced, so a mirror pairs the right groups), then
// v_permlane16_swap / v_permlane32_swap for 16 and 32.  No LDS traffic.
__device__ __forceinline__ float lane_max(float v, uint32_t bits)
{
    auto dpp = [](float x, auto ctrl) {
        return __builtin_bit_cast(
            float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), decltype(ctrl)::value,
                                               0xf, 0xf, false));
    };
    if (bits >= 1u) v = fmaxf(v, dpp(v, std::integral_constant<int, 0xB1>{}));   // quad_perm [1,0,3,2]
    if (bits >= 2u) v = fmaxf(v, dpp(v, std::integral_constant<int, 0x4E>{}));   // quad_perm [2,3,0,1]
    if (bits >= 3u) v = fmaxf(v, dpp(v, std::integral_constant<int, 0x141>{}));  // row_half_mirror
    if (bits >= 4u) v = fmaxf(v, dpp(v, std::integral_constant<int, 0x140>{}));  // row_mirror
    if (bits >= 5u) {
        const uint32_t x = __builtin_bit_cast(uint32_t, v);
        const auto r = __builtin_amdgcn_permlane16_swap(x, x, false, false);
        v = fmaxf(__builtin_bit_cast(float, (uint32_t)r[0]), __builtin_bit_cast(float, (uint32_t)r[1]));
    }
    if (bits >= 6u) {
        const uint32_t x = __builtin_bit_cast(uint32_t, v);
        const auto r = __builtin_amdgcn_permlane32_swap(x, x, false, false);
        v = fmaxf(__builtin_bit_cast(float, (uint32_t)r[0]), __builtin_bit_cast(float, (uint32_t)r[1]));
    }
    return v;
}

// NT tiles per wavefront step; XB cross-tile bits (n = 512 << XB when XB > 0: one step = one row;
// else n <= 512 and the NT tiles are independent).  A wavefront handles the steps first,
// first + stride, ... so the operand and sign-mask set-up is paid once.  MUL = false when the
// transform's output scale is a power of two (folded into the stage-2 operand).
template <int NT, int XB, bool MUL>
__global__ void __launch_bounds__(256)
rht_quant_fp8_kernel(const __bf16* __restrict__ x, const int8_t* __restrict__ sign,
                     uint8_t* __restrict__ q, float* __restrict__ row_scale,
                     __bf16* __restrict__ y_out, uint64_t total, uint64_t num_steps, uint32_t p,
                     int exp2, float mult)
{
    const uint64_t first = (uint64_t)blockIdx.x * 4u + (threadIdx.x >> 6);
    const uint64_t stride = (uint64_t)gridDim.x * 4u;
    __shared__ u32x4 flip_lds[NT][64];
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t n = 1u << p;

    TileOperands<BF16> ops;
    make_tile_operands<BF16, 2>(p, ops, exp2);

    // stage-2 operands that also fold the tile index bits: [s G2; s' G2] for the sign pairs
    // (+,+), (+,-), (-,-), (-,+)
    bf16x8 gfold[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        gfold[0][j] = ops.g2[j]; gfold[0][4 + j] = ops.g2[j];
        gfold[1][j] = ops.g2[j]; gfold[1][4 + j] = -ops.g2[j];
        gfold[2][j] = -ops.g2[j]; gfold[2][4 + j] = -ops.g2[j];
        gfold[3][j] = -ops.g2[j]; gfold[3][4 + j] = ops.g2[j];
    }
    // sign-bit masks of a lane's 8 columns in each tile of a step: the column pattern is the same
    // for every step (a step covers a whole number of rows), so the first wavefront leaves them in
    // LDS for all four
    if (threadIdx.x < 64u) {
#pragma unroll
        for (int c = 0; c < NT; ++c) {
            const uint32_t col = (uint32_t)((first * NT + c) * 512u + 8u * lane) & (n - 1u);
            const u32x2 sg = *reinterpret_cast<const u32x2*>(sign + col);  // 8 int8, +1 / -1
            u32x4 f;
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                const uint32_t s2 = (w < 2 ? sg[0] : sg[1]) >> (16 * (w & 1));
                f[w] = ((s2 & 0x80u) << 8) | ((s2 & 0x8000u) << 16);
            }
            flip_lds[c][lane] = f;
        }
    }
    __syncthreads();
    if (first >= num_steps) return;
    // lanes that share a row: lane bit i carries element bit 3 + i, so the low min(6, p - 3)
    // lane bits index inside a row
    const uint32_t row_lane_bits = p >= 9u ? 6u : p - 3u;

    for (uint64_t step = first; step < num_steps; step += stride) {
        // load + sign flip
        bf16x8 in[NT];
#pragma unroll
        for (int c = 0; c < NT; ++c) {
            const uint64_t off = (step * NT + c) * 512u + 8u * lane;
            u32x4 bits = {0u, 0u, 0u, 0u};
            if (XB > 0 || off + 8u <= total) bits = *reinterpret_cast<const u32x4*>(x + off);
            in[c] = __builtin_bit_cast(bf16x8, bits ^ flip_lds[c][lane]);
        }
        __builtin_amdgcn_sched_barrier(0);

        bf16x8 y[NT];
        float amax[NT];
        if constexpr (XB > 0) {
            const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
            bf16x4 a2[NT][2];
#pragma unroll
            for (int c = 0; c < NT; ++c)
#pragma unroll
                for (int t = 0; t < 2; ++t) a2[c][t] = narrow4<BF16>(BF16::mfma32(in[c], ops.g1[t], zero));
#pragma unroll
            for (int o = 0; o < NT; ++o) {
                float m = 0.0f;
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    f32x4 d = zero;
#pragma unroll
                    for (int pr = 0; pr < NT / 2; ++pr) {
                        bf16x8 A;
#pragma unroll
                        for (int i = 0; i < 4; ++i) { A[i] = a2[2 * pr][t][i]; A[4 + i] = a2[2 * pr + 1][t][i]; }
                        const bool m0 = __builtin_popcount(o & (2 * pr)) & 1, m1 = __builtin_popcount(o & (2 * pr + 1)) & 1;
                        d = BF16::mfma32(A, gfold[(m0 ? 2 : 0) + (m1 != m0 ? 1 : 0)], d);
                    }
                    if (MUL) d = d * mult;
#pragma unroll
                    for (int r = 0; r < 4; ++r) y[o][4 * t + r] = (__bf16)d[r];
                    m = fmaxf(fmaxf(__builtin_fabsf(d[0]), __builtin_fabsf(d[1])), m);
                    m = fmaxf(fmaxf(__builtin_fabsf(d[2]), __builtin_fabsf(d[3])), m);
                }
                amax[o] = m;
            }
        } else {
            f32x4 acc[NT][2];
#pragma unroll
            for (int c = 0; c < NT; ++c) tile_transform<BF16>(in[c], ops, acc[c]);
#pragma unroll
            for (int c = 0; c < NT; ++c) {
                float m = 0.0f;
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    f32x4 v = acc[c][t];
                    if (MUL) v = v * mult;
#pragma unroll
                    for (int r = 0; r < 4; ++r) y[c][4 * t + r] = (__bf16)v[r];
                    m = fmaxf(fmaxf(__builtin_fabsf(v[0]), __builtin_fabsf(v[1])), m);
                    m = fmaxf(fmaxf(__builtin_fabsf(v[2]), __builtin_fabsf(v[3])), m);
                }
                amax[c] = m;
            }
        }
        if (XB > 0) {  // one row spans all NT tiles: fold the tiles, then one lane reduction
            float m = amax[0];
#pragma unroll
            for (int c = 1; c < NT; ++c) m = fmaxf(m, amax[c]);
            m = lane_max(m, 6u);
#pragma unroll
            for (int c = 0; c < NT; ++c) amax[c] = m;
        } else {
#pragma unroll
            for (int c = 0; c < NT; ++c) amax[c] = lane_max(amax[c], row_lane_bits);
        }

        u32x2 codes[NT];
#pragma unroll
        for (int c = 0; c < NT; ++c) {
            const uint64_t off = (step * NT + c) * 512u + 8u * lane;
            if (XB == 0 && off + 8u > total) continue;  // XB > 0: whole rows
            const float a = fmaxf((float)(__bf16)amax[c], kAmaxFloor);
            const float inv = kFp8Max / a;
            // first lane of each row writes the dequantisation factor
            const bool row_head = XB > 0 ? (c == 0 && lane == 0) : ((off & (uint64_t)(n - 1u)) == 0);
            if (row_head) row_scale[off >> p] = a / kFp8Max;
            // |y| <= amax, so y * inv <= 448 * (1 + 2^-23): always inside the round-to-448 interval
            // and the +-448 clamp of the stated convention never changes a finite value; omitted.
            const u32x4 yb = __builtin_bit_cast(u32x4, y[c]);
#pragma unroll
            for (int w = 0; w < 2; ++w) {
                float v[4];
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    v[2 * i] = __builtin_bit_cast(float, yb[2 * w + i] << 16) * inv;
                    v[2 * i + 1] = __builtin_bit_cast(float, yb[2 * w + i] & 0xffff0000u) * inv;
                }
                int pk = __builtin_amdgcn_cvt_pk_fp8_f32(v[0], v[1], 0, false);
                pk = __builtin_amdgcn_cvt_pk_fp8_f32(v[2], v[3], pk, true);
                codes[c][w] = (uint32_t)pk;
            }
            // streaming stores: the codes are not read again here (an exchange between neighbouring
            // lanes would make them 16-byte stores, but costs more vector instructions than it saves)
            __builtin_nontemporal_store(codes[c], reinterpret_cast<u32x2*>(q + off));
            if (y_out) *reinterpret_cast<bf16x8*>(y_out + off) = y[c];
        }
    }
}

template <int NT, int XB>
int launch_quant(const void* x, const int8_t* sign, void* q, float* rs, void* y_out, uint64_t total,
                 uint64_t num_steps, uint32_t p, OutputScale os, hipStream_t s)
{
    // a wavefront's steps must all see the same column pattern: with NT tiles per step a step
    // covers NT * 512 elements, a whole number of rows for every n <= NT * 512 (true here)
    // Grid: the kernel keeps four wavefronts per SIMD (at most 128 registers), 4096 on the chip; one
    // step per wavefront up to that many, and exactly that many wavefronts, each walking its share of
    // the steps, beyond (for [8192, 4096]: two rows per wavefront on every SIMD alike; workgroups
    // that only start when others have finished cost about 1.5 us each at this size).
    uint64_t waves = num_steps;
    const uint64_t resident = 256u * 16u;
    if (waves > resident) waves = resident;
    const uint64_t blocks = (waves + 3u) / 4u;
    if (blocks > 0x7fffffffull) return MI_ERR_SHAPE;
    if (os.mult == 1.0f)
        hipLaunchKernelGGL((rht_quant_fp8_kernel<NT, XB, false>), dim3((uint32_t)blocks), dim3(256), 0,
                           s, static_cast<const __bf16*>(x), sign, static_cast<uint8_t*>(q), rs,
                           static_cast<__bf16*>(y_out), total, num_steps, p, os.exp2, os.mult);
    else
        hipLaunchKernelGGL((rht_quant_fp8_kernel<NT, XB, true>), dim3((uint32_t)blocks), dim3(256), 0,
                           s, static_cast<const __bf16*>(x), sign, static_cast<uint8_t*>(q), rs,
                           static_cast<__bf16*>(y_out), total, num_steps, p, os.exp2, os.mult);
    return launch_status();
}

}  // namespace
}  // namespace mi

extern "C" int mi_rht_quant_fp8(const void* x, const int8_t* sign, void* q, float* row_scale,
                                void* y_out, uint64_t T, uint32_t n, float scale, void* stream)
{
    using namespace mi;
    if (!is_pow2(n) || n < 16u || n > 4096u) return MI_ERR_SIZE;
    if (T == 0) return MI_OK;
    if (!x || !sign || !q || !row_scale) return MI_ERR_NULL;
    if (!aligned16(x) || !aligned16(q) || (y_out && !aligned16(y_out)) ||
        (reinterpret_cast<uintptr_t>(sign) & 7u))
        return MI_ERR_ALIGN;
    const uint32_t p = ilog2(n);
    const uint64_t total = T * (uint64_t)n;
    const OutputScale os = split_output_scale((double)scale, tile_stage_shift<2>(p, false));
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (p <= 9) {
        const uint64_t tiles = (total + 511u) / 512u;
        return launch_quant<1, 0>(x, sign, q, row_scale, y_out, total, tiles, p, os, s);
    }
    switch (p) {
        case 10: return launch_quant<2, 1>(x, sign, q, row_scale, y_out, total, T, p, os, s);
        case 11: return launch_quant<4, 2>(x, sign, q, row_scale, y_out, total, T, p, os, s);
        default: return launch_quant<8, 3>(x, sign, q, row_scale, y_out, total, T, p, os, s);
    }
}
