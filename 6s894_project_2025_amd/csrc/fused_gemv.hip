// Fused Hadamard + GEMV-batch (mi_fused_ht_gemv), fp32, gfx950:
//     Y[M,B] = W[M,N] * (scale * H_N * X[N,B]),  transform down dimension 0 of X.
//
// A workgroup owns 16 columns of X and a slice of M.
//   prologue : the 16 columns are brought into LDS as T[N][16] (a row is 64 bytes, so the 16
//              column-lanes of a wavefront read global memory contiguously) while radix-16
//              register butterflies run: each thread owns one column and 16 rows per step, so
//              log2(N) stages cost ceil(log2(N)/4) passes over LDS, the first one straight from
//              global memory.  Row positions are XOR-swizzled so every access pattern below
//              touches four different 64-byte bank groups per wavefront.
//   product  : v_mfma_f32_16x16x4_f32 with W as the A operand (one 16-byte load per lane gives
//              four consecutive k for four MFMAs) and T as the B operand; each W element is read
//              once per workgroup instead of once per column.
//
// Behaviour replaced: fused_hadamard_gemv_kernel(_vec), fused_ht/fwht_gemv_fusion.cu:98-244, where
// every column's block re-reads all of W and reduces with warp shuffles.
#include "common.hpp"

namespace mi {
namespace {

constexpr int kCols = 16;
constexpr int kThreads = 256;
constexpr int kRowsPerWave = 32;                        // two 16-row MFMA blocks
constexpr int kRowsPerBlock = kRowsPerWave * kThreads / 64;  // 128

// physical row of logical row r in the LDS tile: low two bits mixed with bits 2-3 and 4-5
__device__ __forceinline__ uint32_t prow(uint32_t r)
{
    return r ^ ((r >> 2) & 3u) ^ ((r >> 4) & 3u);
}

template <int WBITS>
__device__ __forceinline__ void butterfly_regs(float (&v)[16])
{
#pragma unroll
    for (int b = 0; b < WBITS; ++b)
#pragma unroll
        for (int i = 0; i < (1 << WBITS); ++i) {
            if (i & (1 << b)) continue;
            const float x = v[i], y = v[i | (1 << b)];
            v[i] = x + y;
            v[i | (1 << b)] = x - y;
        }
}

// One radix-2^WBITS pass over index bits [shift, shift + WBITS).  FROM_GLOBAL: read X, else LDS.
template <int WBITS, bool FROM_GLOBAL>
__device__ __forceinline__ void pass(const float* __restrict__ X, float* tile, uint32_t N,
                                     uint32_t B, uint32_t b0, uint32_t shift, float mul)
{
    const uint32_t c = threadIdx.x & 15u, g = threadIdx.x >> 4;
    const uint32_t stride = 1u << shift;
    const uint32_t sets = N >> WBITS;
    const bool col_ok = b0 + c < B;
    for (uint32_t s = g; s < sets; s += kThreads / 16) {
        const uint32_t base = ((s >> shift) << (shift + WBITS)) | (s & (stride - 1u));
        float v[16];
#pragma unroll
        for (int i = 0; i < (1 << WBITS); ++i) {
            const uint32_t r = base + (uint32_t)i * stride;
            if (FROM_GLOBAL)
                v[i] = col_ok ? X[(uint64_t)r * B + b0 + c] : 0.0f;
            else
                v[i] = tile[prow(r) * kCols + c];
        }
        butterfly_regs<WBITS>(v);
#pragma unroll
        for (int i = 0; i < (1 << WBITS); ++i) {
            const uint32_t r = base + (uint32_t)i * stride;
            tile[prow(r) * kCols + c] = v[i] * mul;
        }
    }
}

template <bool FROM_GLOBAL>
__device__ __forceinline__ void pass_w(int wbits, const float* __restrict__ X, float* tile,
                                       uint32_t N, uint32_t B, uint32_t b0, uint32_t shift,
                                       float mul)
{
    switch (wbits) {
        case 1: pass<1, FROM_GLOBAL>(X, tile, N, B, b0, shift, mul); break;
        case 2: pass<2, FROM_GLOBAL>(X, tile, N, B, b0, shift, mul); break;
        case 3: pass<3, FROM_GLOBAL>(X, tile, N, B, b0, shift, mul); break;
        default: pass<4, FROM_GLOBAL>(X, tile, N, B, b0, shift, mul); break;
    }
}

__global__ void __launch_bounds__(kThreads)
fused_ht_gemv_kernel(const float* __restrict__ W, const float* __restrict__ X,
                     float* __restrict__ Y, uint32_t M, uint32_t N, uint32_t B, uint32_t logN,
                     float scale)
{
    extern __shared__ __attribute__((aligned(16))) float tile[];  // [N][16], rows swizzled
    const uint32_t b0 = blockIdx.x * kCols;

    // ---- prologue: T = scale * H_N * X[:, b0:b0+16] --------------------------------------------
    {
        uint32_t done = 0;
        bool first = true;
        while (done < logN) {
            const int wbits = (int)min(4u, logN - done);
            const float mul = (done + wbits == logN) ? scale : 1.0f;
            if (first)
                pass_w<true>(wbits, X, tile, N, B, b0, done, mul);
            else
                pass_w<false>(wbits, X, tile, N, B, b0, done, mul);
            first = false;
            done += wbits;
            __syncthreads();
        }
    }

    // ---- product ----------------------------------------------------------------------------------
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint32_t lo = lane & 15u, hi = lane >> 4;
    const uint32_t mb = blockIdx.y * kRowsPerBlock + wave * kRowsPerWave;
    if (mb >= M) return;

    f32x4 acc[2] = {f32x4{0.f, 0.f, 0.f, 0.f}, f32x4{0.f, 0.f, 0.f, 0.f}};
    const float* wrow[2];
#pragma unroll
    for (int mi = 0; mi < 2; ++mi) {
        const uint32_t m = min(mb + 16u * mi + lo, M - 1u);
        wrow[mi] = W + (uint64_t)m * N + 4u * hi;
    }
    if (N >= 16u) {
        const uint32_t ksteps = N >> 4;
        f32x4 acur[2], anext[2];
#pragma unroll
        for (int mi = 0; mi < 2; ++mi) acur[mi] = *reinterpret_cast<const f32x4*>(wrow[mi]);
        for (uint32_t kk = 0; kk < ksteps; ++kk) {
            if (kk + 1 < ksteps) {
#pragma unroll
                for (int mi = 0; mi < 2; ++mi)
                    anext[mi] = *reinterpret_cast<const f32x4*>(wrow[mi] + 16u * (kk + 1));
            }
            float bv[4];
#pragma unroll
            for (int s = 0; s < 4; ++s) bv[s] = tile[prow(16u * kk + 4u * hi + s) * kCols + lo];
#pragma unroll
            for (int s = 0; s < 4; ++s)
#pragma unroll
                for (int mi = 0; mi < 2; ++mi)
                    acc[mi] = __builtin_amdgcn_mfma_f32_16x16x4f32(acur[mi][s], bv[s], acc[mi], 0, 0,
                                                                   0);
#pragma unroll
            for (int mi = 0; mi < 2; ++mi) acur[mi] = anext[mi];
        }
    } else {
        // N = 2, 4, 8: one partial step, lanes with k >= N contribute zero
#pragma unroll
        for (int mi = 0; mi < 2; ++mi) {
            const uint32_t m = min(mb + 16u * mi + lo, M - 1u);
            const float a = hi < N ? W[(uint64_t)m * N + hi] : 0.0f;
            const float b = hi < N ? tile[prow(hi) * kCols + lo] : 0.0f;
            acc[mi] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, acc[mi], 0, 0, 0);
            if (N == 8u) {
                const float a2 = W[(uint64_t)m * N + 4u + hi];
                const float b2 = tile[prow(4u + hi) * kCols + lo];
                acc[mi] = __builtin_amdgcn_mfma_f32_16x16x4f32(a2, b2, acc[mi], 0, 0, 0);
            }
        }
    }

    // D[m'][n']: n' = lo is the column, m' = 4*hi + r the row inside the 16-row block
    if (b0 + lo < B) {
#pragma unroll
        for (int mi = 0; mi < 2; ++mi)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const uint32_t m = mb + 16u * mi + 4u * hi + r;
                if (m < M) Y[(uint64_t)m * B + b0 + lo] = acc[mi][r];
            }
    }
}

}  // namespace
}  // namespace mi

extern "C" int mi_fused_ht_gemv(const void* W, const void* X, void* Y, uint32_t M, uint32_t N,
                                uint32_t B, int dtype, float scale, void* stream)
{
    using namespace mi;
    if (dtype != MI_F32) return MI_ERR_DTYPE;
    if (!is_pow2(N) || N < 2u || N > 2048u) return MI_ERR_SIZE;
    if (M == 0 || B == 0) return MI_OK;
    if (!W || !X || !Y) return MI_ERR_NULL;
    if (!aligned16(W) || !aligned16(X) || !aligned16(Y)) return MI_ERR_ALIGN;
    const size_t lds = (size_t)N * kCols * sizeof(float);
    auto kern = fused_ht_gemv_kernel;
    if (lds > 64u * 1024u) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
            return MI_ERR_LAUNCH;
    }
    const dim3 grid((B + kCols - 1) / kCols, (M + kRowsPerBlock - 1) / kRowsPerBlock);
    hipLaunchKernelGGL(kern, grid, dim3(kThreads), lds, static_cast<hipStream_t>(stream),
                       static_cast<const float*>(W), static_cast<const float*>(X),
                       static_cast<float*>(Y), M, N, B, ilog2(N), scale);
    return launch_status();
}
