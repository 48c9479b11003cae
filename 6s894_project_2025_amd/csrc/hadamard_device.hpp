// Device-side embedding API: the Walsh-Hadamard transform as `__device__` building blocks that any
// HIP kernel for gfx950 can call on data it already owns (attention / quantisation epilogues, the
// fused kernels of this library).  Counterpart of the reference's
//   HadamardTransform<dtype,N>::hadamard_transform_device(in, out, sm), T, N_ROWS, SM_BYTES
//   (csrc/hada_handler.cuh:227-264), whose stand-alone kernel is a thin caller (csrc/main.cu:42-53);
// here the stand-alone kernels of mi_fwht are the same kind of thin caller.
//
//   HadamardTransformDevice<IO, LOG_N>      IO = Io16<BF16> | Io16<F16> | Io32,  N = 2^LOG_N
//     ::T          element type in memory
//     ::THREADS    threads that must call together: 64 (one wavefront) for N <= 4096,
//                  N / 64 (N / 4096 wavefronts, one workgroup) above
//     ::N_ROWS     contiguous rows one call transforms: 512 / N for N <= 512, else 1
//     ::LDS_BYTES  dynamic LDS the call needs (0 for N <= 4096)
//     ::prepare(os)                     per-lane Hadamard operands, once per kernel
//     ::hadamard_transform_device(in, out, lds, ops)
//                                       out[0 .. N_ROWS*N) = scale * H_N * in[...] row by row;
//                                       in == out allowed; 16-byte aligned pointers
//   `os` is output_scale<IO, LOG_N>(scale), computed on the host and passed as kernel arguments
//   (a power-of-two scale is folded into the matrix-core operands and costs nothing).
//
// Lower-level pieces for kernels that keep the data in registers (the fused kernels do):
// tile_transform / tile_transform_f32 / cross_tile_butterflies in fwht_device.hpp.
#pragma once

#include "fwht_device.hpp"

namespace mi {

// ---- element I/O -------------------------------------------------------------------------------
// Each IO policy loads a lane's share of one tile into MFMA input form and stores two f32x4
// accumulators back, both guarded against the end of the buffer (`total` elements).

// STREAM = true marks every access non-temporal: for tensors that do not fit the last-level
// cache, where keeping lines that are never touched again only costs bandwidth.
template <class T16_, bool STREAM = false>
struct Io16 {
    using Streaming = Io16<T16_, true>;
    static constexpr bool kStreaming = STREAM;
    using T16 = T16_;
    using E = typename T16::E;
    using Elem = E;
    static constexpr int ESIZE = 2;
    struct In {
        typename T16::V8 a;
    };

    template <bool GUARD>
    static __device__ __forceinline__ In load(const void* base, uint64_t tile, uint64_t total)
    {
        const E* p = static_cast<const E*>(base);
        const uint64_t off = tile * 512u + 8u * (threadIdx.x & 63u);
        In in;
        if (!GUARD || off + 8u <= total) {
            if (STREAM)
                in.a = __builtin_nontemporal_load(reinterpret_cast<const typename T16::V8*>(p + off));
            else
                in.a = *reinterpret_cast<const typename T16::V8*>(p + off);
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j) in.a[j] = (off + j < total) ? p[off + j] : (E)0.0f;
        }
        return in;
    }

    static __device__ __forceinline__ void transform(const In& in, const TileOperands<T16>& ops,
                                                     f32x4 (&acc)[2])
    {
        tile_transform<T16>(in.a, ops, acc);
    }

    template <bool GUARD, bool MUL>
    static __device__ __forceinline__ void store(void* base, uint64_t tile, uint64_t total,
                                                 const f32x4 (&acc)[2], float s)
    {
        E* p = static_cast<E*>(base);
        const uint64_t off = tile * 512u + 8u * (threadIdx.x & 63u);
        typename T16::V8 o;
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) o[4 * t + r] = (E)(MUL ? acc[t][r] * s : acc[t][r]);
        if (!GUARD || off + 8u <= total) {
            if (STREAM)
                __builtin_nontemporal_store(o, reinterpret_cast<typename T16::V8*>(p + off));
            else
                *reinterpret_cast<typename T16::V8*>(p + off) = o;
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j)
                if (off + j < total) p[off + j] = o[j];
        }
    }
};

template <bool STREAM = false>
struct Io32T {
    using Streaming = Io32T<true>;
    static constexpr bool kStreaming = STREAM;
    using T16 = BF16;  // matrix-core type used for the three-piece products
    using Elem = float;
    static constexpr int ESIZE = 4;
    struct In {
        float v[8];
    };

    template <bool GUARD>
    static __device__ __forceinline__ In load(const void* base, uint64_t tile, uint64_t total)
    {
        const float* p = static_cast<const float*>(base);
        In in;
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const uint64_t off = tile * 512u + 256u * t + 4u * (threadIdx.x & 63u);
            if (!GUARD || off + 4u <= total) {
                const f32x4 q = STREAM ? __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(p + off))
                                       : *reinterpret_cast<const f32x4*>(p + off);
#pragma unroll
                for (int r = 0; r < 4; ++r) in.v[4 * t + r] = q[r];
            } else {
#pragma unroll
                for (int r = 0; r < 4; ++r) in.v[4 * t + r] = (off + r < total) ? p[off + r] : 0.0f;
            }
        }
        return in;
    }

    static __device__ __forceinline__ void transform(const In& in, const TileOperands<BF16>& ops,
                                                     f32x4 (&acc)[2])
    {
        tile_transform_f32(in.v, ops, acc);
    }

    template <bool GUARD, bool MUL>
    static __device__ __forceinline__ void store(void* base, uint64_t tile, uint64_t total,
                                                 const f32x4 (&acc)[2], float s)
    {
        float* p = static_cast<float*>(base);
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const uint64_t off = tile * 512u + 256u * t + 4u * (threadIdx.x & 63u);
            const f32x4 o = MUL ? acc[t] * s : acc[t];
            if (!GUARD || off + 4u <= total) {
                if (STREAM)
                    __builtin_nontemporal_store(o, reinterpret_cast<f32x4*>(p + off));
                else
                    *reinterpret_cast<f32x4*>(p + off) = o;
            } else {
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    if (off + r < total) p[off + r] = o[r];
            }
        }
    }
};

using Io32 = Io32T<false>;

// ---- wavefront level: NT tiles of 512 elements, XB cross-tile bits ---------------------------------
// One step = tiles [step*NT, step*NT + NT) of the buffer = one row when XB > 0, several short rows
// otherwise.  `in` may equal `out`: the wavefront reads all tiles of the step before it writes any.
// GUARD = true bounds-checks every access against `total` elements (ragged last step only).
template <class IO, int NT, bool GUARD>
__device__ __forceinline__ void wave_fwht_load(const void* in, uint64_t step, uint64_t total,
                                               typename IO::In (&tin)[NT])
{
#pragma unroll
    for (int c = 0; c < NT; ++c) tin[c] = IO::template load<GUARD>(in, step * NT + c, total);
}

template <class IO, int NT, int XB, bool GUARD, bool MUL>
__device__ __forceinline__ void wave_fwht_finish(const typename IO::In (&tin)[NT], void* out,
                                                 uint64_t step, uint64_t total,
                                                 const TileOperands<typename IO::T16>& ops,
                                                 float mult)
{
    f32x4 acc[NT][2];
#pragma unroll
    for (int c = 0; c < NT; ++c) IO::transform(tin[c], ops, acc[c]);

    cross_tile_butterflies<NT, XB>(acc);

#pragma unroll
    for (int c = 0; c < NT; ++c)
        IO::template store<GUARD, MUL>(out, step * NT + c, total, acc[c], mult);
}

template <class IO, int NT, int XB, bool GUARD, bool MUL>
__device__ __forceinline__ void wave_fwht_step(const void* in, void* out, uint64_t step,
                                               uint64_t total,
                                               const TileOperands<typename IO::T16>& ops, float mult)
{
    typename IO::In tin[NT];
    wave_fwht_load<IO, NT, GUARD>(in, step, total, tin);
    // keep every load of the step in flight before any arithmetic is scheduled
    __builtin_amdgcn_sched_barrier(0);
    wave_fwht_finish<IO, NT, XB, GUARD, MUL>(tin, out, step, total, ops, mult);
}

// ---- workgroup level: W = 2^LW wavefronts transform one row of n = 4096 * W -----------------------
// Pass 1: wavefront w transforms elements [4096w, 4096w+4096) (12 bits).  Exchange: every
// accumulator quad goes to LDS once; wavefront w then gathers, from all W sub-rows, the 8/W tiles
// it owns, runs the LW remaining butterflies in registers and stores.  `xch` holds
// 16 * 64 * 8 * W bytes (TWO_PHASE: the two accumulator halves take turns) or twice that (one
// exchange); all 64*W threads must call (__syncthreads inside).
template <class IO>
__device__ __forceinline__ void block_fwht_load(const void* in, uint64_t tile0, uint64_t total,
                                                typename IO::In (&tin)[8])
{
    const uint32_t w = threadIdx.x >> 6;
#pragma unroll
    for (int c = 0; c < 8; ++c) tin[c] = IO::template load<false>(in, tile0 + w * 8u + c, total);
}

template <class IO, int LW, bool MUL, bool TWO_PHASE = true>
__device__ __forceinline__ void block_fwht_finish(const typename IO::In (&tin)[8], void* out,
                                                  uint64_t tile0, uint64_t total, f32x4* xch,
                                                  const TileOperands<typename IO::T16>& ops, float mult)
{
    constexpr int W = 1 << LW;
    constexpr int OWN = 8 / W;  // tiles per sub-row owned by a wavefront in pass 2
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t w = threadIdx.x >> 6;
    f32x4 acc[8][2];
#pragma unroll
    for (int c = 0; c < 8; ++c) IO::transform(tin[c], ops, acc[c]);
    cross_tile_butterflies<8, 3>(acc);
    f32x4 g[W * OWN][2];  // index s * OWN + c'
    if constexpr (TWO_PHASE) {
        // xch layout: [W sub-rows][8 tiles][64 lanes], used twice (once per accumulator half):
        // half the LDS footprint, so two workgroups share a compute unit at W = 8
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            if (t) __syncthreads();  // every wavefront has read the first half
#pragma unroll
            for (int c = 0; c < 8; ++c) xch[(w * 8u + c) * 64u + lane] = acc[c][t];
            __syncthreads();
#pragma unroll
            for (int s = 0; s < W; ++s)
#pragma unroll
                for (int cc = 0; cc < OWN; ++cc)
                    g[s * OWN + cc][t] = xch[(s * 8u + w * OWN + cc) * 64u + lane];
        }
    } else {
        // xch layout: [W sub-rows][8 tiles][2 halves][64 lanes], one exchange with one barrier
#pragma unroll
        for (int c = 0; c < 8; ++c)
#pragma unroll
            for (int t = 0; t < 2; ++t) xch[((w * 8u + c) * 2u + t) * 64u + lane] = acc[c][t];
        __syncthreads();
#pragma unroll
        for (int s = 0; s < W; ++s)
#pragma unroll
            for (int cc = 0; cc < OWN; ++cc)
#pragma unroll
                for (int t = 0; t < 2; ++t)
                    g[s * OWN + cc][t] = xch[((s * 8u + w * OWN + cc) * 2u + t) * 64u + lane];
    }

    // butterflies over the sub-row index s (element bits 12 .. 12+LW-1)
#pragma unroll
    for (int b = 0; b < LW; ++b)
#pragma unroll
        for (int s = 0; s < W; ++s) {
            if (s & (1 << b)) continue;
#pragma unroll
            for (int cc = 0; cc < OWN; ++cc)
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    const f32x4 x = g[s * OWN + cc][t], y = g[(s | (1 << b)) * OWN + cc][t];
                    g[s * OWN + cc][t] = x + y;
                    g[(s | (1 << b)) * OWN + cc][t] = x - y;
                }
        }

#pragma unroll
    for (int s = 0; s < W; ++s)
#pragma unroll
        for (int cc = 0; cc < OWN; ++cc)
            IO::template store<false, MUL>(out, tile0 + s * 8u + w * OWN + cc, total,
                                           g[s * OWN + cc], mult);
}

template <class IO, int LW, bool MUL, bool TWO_PHASE = true>
__device__ __forceinline__ void block_fwht_row(const void* in, void* out, uint64_t tile0,
                                               uint64_t total, f32x4* xch,
                                               const TileOperands<typename IO::T16>& ops, float mult)
{
    typename IO::In tin[8];
    block_fwht_load<IO>(in, tile0, total, tin);
    block_fwht_finish<IO, LW, MUL, TWO_PHASE>(tin, out, tile0, total, xch, ops, mult);
}

// Host side: the (exp2, mult) pair for a transform of length 2^LOG_N with output factor `scale`.
template <class IO, int LOG_N>
inline OutputScale output_scale(double scale)
{
    return split_output_scale(scale, tile_stage_shift<IO::ESIZE>(LOG_N, kNarrowRange<typename IO::T16>));
}

template <class IO_, int LOG_N>
struct HadamardTransformDevice {
    static_assert(LOG_N >= 0 && LOG_N <= 15, "transform length 1 .. 32768");
    using IO = IO_;
    using T = typename IO::Elem;
    using Operands = TileOperands<typename IO::T16>;
    static constexpr int N = 1 << LOG_N;
    static constexpr int LW = LOG_N > 12 ? LOG_N - 12 : 0;
    static constexpr int THREADS = 64 << LW;
    static constexpr int N_ROWS = LOG_N <= 9 ? (512 >> LOG_N) : 1;
    static constexpr int LDS_BYTES = LOG_N > 12 ? (int)sizeof(f32x4) * 64 * 8 * (1 << LW) : 0;

    static __device__ __forceinline__ Operands prepare(OutputScale os)
    {
        Operands ops;
        make_tile_operands<typename IO::T16, IO::ESIZE>(LOG_N, ops, os.exp2);
        return ops;
    }

    // `lds`: LDS_BYTES of 16-byte aligned LDS (ignored when LDS_BYTES == 0).  The residual factor
    // os.mult is applied at the store (skipped when it is exactly 1).
    static __device__ __forceinline__ void hadamard_transform_device(const T* in, T* out, void* lds,
                                                                     const Operands& ops,
                                                                     OutputScale os)
    {
        constexpr uint64_t kAll = ~0ull;  // the caller owns N_ROWS full rows: nothing to guard
        if constexpr (LOG_N <= 9) {
            if (os.mult == 1.0f) wave_fwht_step<IO, 1, 0, false, false>(in, out, 0, kAll, ops, 1.0f);
            else wave_fwht_step<IO, 1, 0, false, true>(in, out, 0, kAll, ops, os.mult);
        } else if constexpr (LOG_N <= 12) {
            constexpr int XB = LOG_N - 9;
            if (os.mult == 1.0f)
                wave_fwht_step<IO, 1 << XB, XB, false, false>(in, out, 0, kAll, ops, 1.0f);
            else
                wave_fwht_step<IO, 1 << XB, XB, false, true>(in, out, 0, kAll, ops, os.mult);
        } else {
            if (os.mult == 1.0f)
                block_fwht_row<IO, LW, false>(in, out, 0, kAll, static_cast<f32x4*>(lds), ops, 1.0f);
            else
                block_fwht_row<IO, LW, true>(in, out, 0, kAll, static_cast<f32x4*>(lds), ops, os.mult);
        }
    }
};

}  // namespace mi
