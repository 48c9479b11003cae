// Stand-alone Walsh-Hadamard transform over the last dimension (mi_fwht), gfx950.
//
// Bandwidth-bound: one 16-byte load and one 16-byte store per 8 (2-byte) or 4 (4-byte) elements,
// everything in between on the matrix cores (tile_transform) plus a few fp32 butterflies.
//
//   n <= 512          : a wavefront transforms NT independent 512-element tiles (several rows
//                       per tile; masked Hadamard operands).
//   1024 <= n <= 4096 : one wavefront per row; n/512 tiles in registers, the tile-index bits by
//                       fp32 butterflies between accumulators.
//   n >= 8192         : one workgroup per row; each wavefront transforms 4096 contiguous
//                       elements as above, then the remaining bits are gathered into registers
//                       through one LDS exchange (write once, read once).
//
// Behaviour replaced: run_fht<dtype>() and its kernels, csrc/main.cu:12-122 and
// HadaCore/hadamard_transform_cuda.cu:90-746 (normalised FWHT, n = 2..2^15).
#include <type_traits>

#include "hadamard_device.hpp"

namespace mi {
namespace {

// ---- register kernel: NT tiles per wavefront step, XB cross-tile bits ----------------------------
// A wavefront handles the steps  first, first + stride, ...  (one step = NT tiles = one row when
// XB > 0), so the operand set-up is paid once per wavefront.  MUL = false when the output scale is
// a power of two (folded into the stage-2 operand).
template <class IO, int NT, int XB, bool MUL>
__global__ void __launch_bounds__(256)
fwht_reg_kernel(const void* in, void* out, uint64_t total, uint64_t num_steps, uint32_t p, int exp2,
                float mult)
{
    const uint32_t wpb = blockDim.x >> 6;  // wavefronts per workgroup: 1, 2 or 4
    const uint64_t first = (uint64_t)blockIdx.x * wpb + (threadIdx.x >> 6);
    const uint64_t stride = (uint64_t)gridDim.x * wpb;
    if (first >= num_steps) return;  // uniform per wavefront

    TileOperands<typename IO::T16> ops;
    make_tile_operands<typename IO::T16, IO::ESIZE>(p, ops, exp2);

    if constexpr (XB > 0 && IO::ESIZE == 2) {
        // whole rows, 16-bit elements: software pipeline, the loads of the wavefront's next row
        // are in flight while this one is transformed and stored (`in` may equal `out`: the next
        // row is a different row)
        typename IO::In cur[NT], nxt[NT];
        wave_fwht_load<IO, NT, false>(in, first, total, cur);
        for (uint64_t step = first; step < num_steps; step += stride) {
            if (step + stride < num_steps) wave_fwht_load<IO, NT, false>(in, step + stride, total, nxt);
            __builtin_amdgcn_sched_barrier(0);
            wave_fwht_finish<IO, NT, XB, false, MUL>(cur, out, step, total, ops, mult);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int c = 0; c < NT; ++c) cur[c] = nxt[c];
        }
        return;
    }
    // Unguarded when every tile of the step lies inside the buffer (always, except for the last
    // step of a ragged n <= 512 problem): no bounds code on the hot path.
    for (uint64_t step = first; step < num_steps; step += stride) {
        if constexpr (XB > 0) {
            wave_fwht_step<IO, NT, XB, false, MUL>(in, out, step, total, ops, mult);
        } else {
            if ((step * NT + NT) * 512u <= total)
                wave_fwht_step<IO, NT, XB, false, MUL>(in, out, step, total, ops, mult);
            else
                wave_fwht_step<IO, NT, XB, true, MUL>(in, out, step, total, ops, mult);
        }
    }
}

// ---- LDS kernel: one workgroup of W = 2^LW wavefronts per row of n = 4096 * W ----------------
// (Persistent workgroups that prefetch their next row before the exchange were measured slower
// than one short-lived workgroup per row on tensors beyond the last-level cache.)
template <class IO, int LW, bool MUL, bool TWO_PHASE>
__global__ void __launch_bounds__(64 << LW)
fwht_lds_kernel(const void* in, void* out, uint64_t rows, int exp2, float mult)
{
    extern __shared__ f32x4 xch[];
    // Consecutive workgroup ids run on different XCDs (id % 8).  On tensors beyond the last-level
    // cache (the streaming variants), XCD x takes the adjacent rows 2x and 2x+1 inside every full
    // group of 16 rows: neutral for n = 8192 and 16384, 2.7 % faster for n = 32768.
    uint64_t row = blockIdx.x;
    if (IO::kStreaming && row < (rows & ~(uint64_t)15u))
        row = (row & ~(uint64_t)15u) + ((row & 7u) * 2u + ((row >> 3) & 1u));
    if (row >= rows) return;
    const uint64_t total = rows << (12 + LW);

    TileOperands<typename IO::T16> ops;
    make_tile_operands<typename IO::T16, IO::ESIZE>(12 + LW, ops, exp2);
    block_fwht_row<IO, LW, MUL, TWO_PHASE>(in, out, row * (8u << LW), total, xch, ops, mult);
}

// ---- host dispatch --------------------------------------------------------------------------------
template <class IO, int NT, int XB>
int launch_reg(const void* in, void* out, uint64_t total, uint64_t num_steps, uint32_t p,
               OutputScale os, hipStream_t s)
{
    if (num_steps == 0) return MI_OK;
    // Up to three steps per wavefront once the chip is filled one and a half times over: the
    // operand set-up is paid once and the next row's loads overlap the current row's arithmetic.
    // (Exactly filled, with the same number of steps for everybody, all wavefronts load, compute
    // and store in phase: 4096 wavefronts of four steps each measured 1 - 2 % slower at
    // [16384, 4096] and [32768, 2048] than 6144 and 10923 wavefronts.)
    // Beyond the 256 MiB Infinity Cache the transform is DRAM-bound, and there one step per
    // (short-lived) wavefront measured 2 - 4 % faster (the sweep through memory stays in order)
    // and non-temporal loads and stores another 5 - 13 % (lines that are never touched again
    // stay out of the caches).
    const bool big = total * (uint64_t)IO::ESIZE > (256ull << 20);
    uint64_t waves = num_steps;
    const uint64_t resident = 256u * 24u;
    const uint64_t per_wave = big ? 1u : 3u;
    if (waves > resident)
        waves = (num_steps + per_wave - 1u) / per_wave > resident ? (num_steps + per_wave - 1u) / per_wave
                                                                  : resident;
    // Workgroup size.  DRAM-bound, the number of contiguous bytes a workgroup covers decides:
    // 16 KB (or 4 KB where four wavefronts do not reach 16) measured 6.1 - 6.3 TB/s for every n
    // and both element sizes, 8 KB and 32 KB 5.4 - 5.9 TB/s (consecutive workgroups run on
    // different XCDs, so this is the stride with which each XCD walks through memory).
    constexpr uint32_t wave_bytes = NT * 512u * IO::ESIZE;
    uint32_t wpb = 4u;
    if (big) wpb = wave_bytes >= 4096u ? (16384u / wave_bytes > 0u ? 16384u / wave_bytes : 1u) : 4096u / wave_bytes;
    if (wpb > 4u) wpb = 4u;
    const uint64_t blocks = (waves + wpb - 1u) / wpb;
    if (blocks > 0x7fffffffull) return MI_ERR_SHAPE;
    using IOB = typename IO::Streaming;
    auto kern = big ? (os.mult == 1.0f ? fwht_reg_kernel<IOB, NT, XB, false> : fwht_reg_kernel<IOB, NT, XB, true>)
                    : (os.mult == 1.0f ? fwht_reg_kernel<IO, NT, XB, false> : fwht_reg_kernel<IO, NT, XB, true>);
    hipLaunchKernelGGL(kern, dim3((uint32_t)blocks), dim3(64u * wpb), 0, s, in, out, total, num_steps, p,
                       os.exp2, os.mult);
    return launch_status();
}

template <class IO, int LW, bool TWO_PHASE>
int launch_lds_as(const void* in, void* out, uint64_t rows, OutputScale os, hipStream_t s)
{
    constexpr size_t lds = sizeof(f32x4) * 64u * (TWO_PHASE ? 8u : 16u) * (1u << LW);
    const bool mul = os.mult != 1.0f;
    auto kern = mul ? fwht_lds_kernel<IO, LW, true, TWO_PHASE> : fwht_lds_kernel<IO, LW, false, TWO_PHASE>;
    if (lds > 64u * 1024u) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
            return MI_ERR_LAUNCH;
    }
    hipLaunchKernelGGL(kern, dim3((uint32_t)rows), dim3(64u << LW), lds, s, in, out, rows, os.exp2,
                       os.mult);
    return launch_status();
}

template <class IO, int LW>
int launch_lds(const void* in, void* out, uint64_t rows, OutputScale os, hipStream_t s)
{
    if (rows == 0) return MI_OK;
    if (rows > 0x7fffffffull) return MI_ERR_SHAPE;
    // While the tensor fits the 256 MiB Infinity Cache, occupancy decides (exchange in two
    // phases, half the LDS).  Once it is DRAM-bound, non-temporal accesses gain 5 - 10 %; with
    // them the single exchange is the faster one for n = 8192 and 16384, the two-phase exchange
    // (two workgroups per compute unit) for n = 32768, where a single-exchange workgroup fills
    // the LDS alone and streaming loads then measured slower than ordinary ones.
    const uint64_t bytes = (rows << (12 + LW)) * (uint64_t)IO::ESIZE;
    if (bytes > (256ull << 20))
        return launch_lds_as<typename IO::Streaming, LW, LW == 3>(in, out, rows, os, s);
    return launch_lds_as<IO, LW, true>(in, out, rows, os, s);
}

template <class IO>
int dispatch(const void* in, void* out, uint64_t rows, uint32_t n, float scale, hipStream_t s)
{
    const uint32_t p = ilog2(n);
    const uint64_t total = rows * (uint64_t)n;
    const OutputScale os = split_output_scale((double)scale, tile_stage_shift<IO::ESIZE>(p, kNarrowRange<typename IO::T16>));
    if (p <= 9) {
        const uint64_t tiles = (total + 511u) / 512u;
        // several independent tiles per step once there is enough work to fill the chip
        if (tiles >= 4u * 16384u)
            return launch_reg<IO, 4, 0>(in, out, total, (tiles + 3u) / 4u, p, os, s);
        return launch_reg<IO, 1, 0>(in, out, total, tiles, p, os, s);
    }
    switch (p) {
        case 10: return launch_reg<IO, 2, 1>(in, out, total, rows, p, os, s);
        case 11: return launch_reg<IO, 4, 2>(in, out, total, rows, p, os, s);
        case 12: return launch_reg<IO, 8, 3>(in, out, total, rows, p, os, s);
        case 13: return launch_lds<IO, 1>(in, out, rows, os, s);
        case 14: return launch_lds<IO, 2>(in, out, rows, os, s);
        case 15: return launch_lds<IO, 3>(in, out, rows, os, s);
        default: return MI_ERR_SIZE;
    }
}

}  // namespace
}  // namespace mi

extern "C" int mi_fwht(const void* in, void* out, uint64_t rows, uint32_t n, int dtype, float scale,
                       void* stream)
{
    using namespace mi;
    if (!is_pow2(n) || n > 32768u) return MI_ERR_SIZE;
    if (rows == 0) return MI_OK;
    if (!in || !out) return MI_ERR_NULL;
    if (!aligned16(in) || !aligned16(out)) return MI_ERR_ALIGN;
    const size_t esize = dtype == MI_F32 ? 4 : 2;
    if (in != out) {
        const uintptr_t a = (uintptr_t)in, b = (uintptr_t)out;
        const uint64_t bytes = rows * (uint64_t)n * esize;
        if (a < b + bytes && b < a + bytes) return MI_ERR_ALIAS;
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (dtype) {
        case MI_F32: return dispatch<Io32>(in, out, rows, n, scale, s);
        case MI_BF16: return dispatch<Io16<BF16>>(in, out, rows, n, scale, s);
        case MI_F16: return dispatch<Io16<F16>>(in, out, rows, n, scale, s);
        default: return MI_ERR_DTYPE;
    }
}
