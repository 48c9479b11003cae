// Fused Hadamard + GEMV-batch (mi_fused_ht_gemv), fp32, gfx950:
//     Y[M,B] = W[M,N] * (scale * H_N * X[N,B]),  transform down dimension 0 of X.
//
// A workgroup owns 16 columns of X and 16, 32 or 64 rows of W.
//   prologue : the 16 columns are brought into LDS as T[N][16] (a row is 64 bytes, so the 16
//              column-lanes of a wavefront read global memory contiguously) while radix-16
//              register butterflies run: each thread owns one column and 16 rows per step, so
//              log2(N) stages cost ceil(log2(N)/4) passes over LDS, the first one straight from
//              global memory.  Row positions are XOR-swizzled so every access pattern below
//              touches four different 64-byte bank groups per wavefront.
//   product  : v_mfma_f32_16x16x4_f32 with W as the A operand (one 16-byte load per lane gives
//              four consecutive k for four MFMAs) and T as the B operand; each W element is read
//              once per workgroup instead of once per column.  The four wavefronts each take a
//              quarter of the K range with four K steps of loads in flight (the loop is
//              latency-bound otherwise), and their partial sums are added through LDS.
//
// Behaviour replaced: fused_hadamard_gemv_kernel(_vec), fused_ht/fwht_gemv_fusion.cu:98-244, where
// every column's block re-reads all of W and reduces with warp shuffles.
#include "common.hpp"

namespace mi {
namespace {

constexpr int kCols = 16;
constexpr int kThreads = 256;

// physical row of logical row r in the LDS tile: low two bits mixed with bits 2-3 and 4-5
__device__ __forceinline__ uint32_t prow(uint32_t r)
{
    return r ^ ((r >> 2) & 3u) ^ ((r >> 4) & 3u);
}

template <int WBITS>
__device__ __forceinline__ void butterfly_regs(float (&v)[32])
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
// Each thread owns one column and works on SETS butterfly sets at a time, all of their loads
// issued before any arithmetic (the pass from global memory is latency-bound otherwise).
template <int WBITS, bool FROM_GLOBAL>
__device__ __forceinline__ void pass(const float* __restrict__ X, float* tile, uint32_t N,
                                     uint32_t B, uint32_t b0, uint32_t shift, float mul)
{
    constexpr int R = 1 << WBITS;
    constexpr int SETS = (FROM_GLOBAL ? 4 : 2) / (WBITS == 5 ? 2 : 1);
    const uint32_t c = threadIdx.x & 15u, g = threadIdx.x >> 4;
    const uint32_t stride = 1u << shift;
    const uint32_t sets = N >> WBITS;
    const bool col_ok = b0 + c < B;
    constexpr uint32_t G = kThreads / 16;
    for (uint32_t s0 = g; s0 < sets; s0 += G * SETS) {
        float v[SETS][32];
        uint32_t base[SETS];
#pragma unroll
        for (int u = 0; u < SETS; ++u) {
            const uint32_t s = s0 + (uint32_t)u * G;
            base[u] = ((s >> shift) << (shift + WBITS)) | (s & (stride - 1u));
            if (s < sets) {
#pragma unroll
                for (int i = 0; i < R; ++i) {
                    const uint32_t r = base[u] + (uint32_t)i * stride;
                    if (FROM_GLOBAL)
                        v[u][i] = col_ok ? X[(uint64_t)r * B + b0 + c] : 0.0f;
                    else
                        v[u][i] = tile[prow(r) * kCols + c];
                }
            }
        }
#pragma unroll
        for (int u = 0; u < SETS; ++u) {
            const uint32_t s = s0 + (uint32_t)u * G;
            if (s < sets) {
                butterfly_regs<WBITS>(v[u]);
#pragma unroll
                for (int i = 0; i < R; ++i) {
                    const uint32_t r = base[u] + (uint32_t)i * stride;
                    tile[prow(r) * kCols + c] = v[u][i] * mul;
                }
            }
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
        case 4: pass<4, FROM_GLOBAL>(X, tile, N, B, b0, shift, mul); break;
        default: pass<5, FROM_GLOBAL>(X, tile, N, B, b0, shift, mul); break;
    }
}

// MI = 16-row blocks of W per workgroup (16, 32 or 64 rows).  The four wavefronts split the K range
// of the product between them (every wavefront covers all MI row blocks over a quarter of N), so
// each one streams a short, deeply prefetched run of W, and the partial sums meet in LDS.
template <int MI>
__global__ void __launch_bounds__(kThreads)
fused_ht_gemv_kernel(const float* __restrict__ W, const float* __restrict__ X,
                     float* __restrict__ Y, uint32_t M, uint32_t N, uint32_t B, uint32_t logN,
                     float scale, uint32_t rows_per_group)
{
    extern __shared__ __attribute__((aligned(16))) float tile[];  // [N][16] rows swizzled, then sums
    const uint32_t b0 = blockIdx.x * kCols;
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint32_t lo = lane & 15u, hi = lane >> 4;
    // this workgroup's rows: [m_first, m_last), a multiple of 16 * MI except at the end of W
    const uint32_t m_first = blockIdx.y * rows_per_group;
    const uint32_t m_last = min(M, m_first + rows_per_group);

    constexpr int PF = 4;  // K steps (of 16) in flight per wavefront
    const uint32_t total = N >> 4;
    const uint32_t quarter = (total + 3u) / 4u;
    const uint32_t k_begin = min(wave * quarter, total), k_end = min(k_begin + quarter, total);
    const float* wrow[MI];
    f32x4 a[PF][MI];
    auto start_block = [&](uint32_t mb) {
#pragma unroll
        for (int mi = 0; mi < MI; ++mi) {
            const uint32_t m = min(mb + 16u * mi + lo, M - 1u);
            wrow[mi] = W + (uint64_t)m * N + 4u * hi;
        }
#pragma unroll
        for (int j = 0; j < PF; ++j)
            if (k_begin + j < k_end) {
#pragma unroll
                for (int mi = 0; mi < MI; ++mi)
                    a[j][mi] = *reinterpret_cast<const f32x4*>(wrow[mi] + 16u * (k_begin + j));
            }
    };
    // The first W fragments do not depend on the transform: start them before the prologue.
    start_block(m_first);

    // ---- prologue: T = scale * H_N * X[:, b0:b0+16] --------------------------------------------
    {
        uint32_t done = 0;
        bool first = true;
        uint32_t passes_left = (logN + 4u) / 5u;  // fewest radix-32 passes, bits spread evenly
        while (done < logN) {
            const int wbits = (int)((logN - done + passes_left - 1u) / passes_left);
            --passes_left;
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
    f32x4* red = reinterpret_cast<f32x4*>(tile + (size_t)N * kCols);  // [4 wavefronts][MI][64 lanes]

    for (uint32_t mb = m_first; mb < m_last; mb += 16u * MI) {
        if (mb != m_first) start_block(mb);
        // ---- product ------------------------------------------------------------------------------
        f32x4 acc[MI];
#pragma unroll
        for (int mi = 0; mi < MI; ++mi) acc[mi] = f32x4{0.f, 0.f, 0.f, 0.f};
        if (N >= 16u) {
            for (uint32_t kk = k_begin; kk < k_end; kk += PF) {
#pragma unroll
                for (int j = 0; j < PF; ++j) {
                    if (kk + j < k_end) {  // wavefront-uniform
                        f32x4 cur[MI];
#pragma unroll
                        for (int mi = 0; mi < MI; ++mi) cur[mi] = a[j][mi];
                        if (kk + j + PF < k_end) {
#pragma unroll
                            for (int mi = 0; mi < MI; ++mi)
                                a[j][mi] = *reinterpret_cast<const f32x4*>(wrow[mi] +
                                                                           16u * (kk + j + PF));
                        }
                        float bv[4];
#pragma unroll
                        for (int s = 0; s < 4; ++s)
                            bv[s] = tile[prow(16u * (kk + j) + 4u * hi + s) * kCols + lo];
#pragma unroll
                        for (int s = 0; s < 4; ++s)
#pragma unroll
                            for (int mi = 0; mi < MI; ++mi)
                                acc[mi] = __builtin_amdgcn_mfma_f32_16x16x4f32(cur[mi][s], bv[s],
                                                                               acc[mi], 0, 0, 0);
                    }
                }
            }
        } else if (wave == 0) {
            // N = 2, 4, 8: one partial step, lanes with k >= N contribute zero
#pragma unroll
            for (int mi = 0; mi < MI; ++mi) {
                const uint32_t m = min(mb + 16u * mi + lo, M - 1u);
                const float av = hi < N ? W[(uint64_t)m * N + hi] : 0.0f;
                const float b = hi < N ? tile[prow(hi) * kCols + lo] : 0.0f;
                acc[mi] = __builtin_amdgcn_mfma_f32_16x16x4f32(av, b, acc[mi], 0, 0, 0);
                if (N == 8u) {
                    const float a2 = W[(uint64_t)m * N + 4u + hi];
                    const float b2 = tile[prow(4u + hi) * kCols + lo];
                    acc[mi] = __builtin_amdgcn_mfma_f32_16x16x4f32(a2, b2, acc[mi], 0, 0, 0);
                }
            }
        }

        // ---- meet the four K quarters in LDS ------------------------------------------------------
        __syncthreads();  // the previous block's sums have been read
#pragma unroll
        for (int mi = 0; mi < MI; ++mi) red[(wave * MI + mi) * 64u + lane] = acc[mi];
        __syncthreads();
        // D[m'][n']: n' = lo is the column, m' = 4*hi + r the row inside the 16-row block
        for (uint32_t mi = wave; mi < (uint32_t)MI; mi += 4u) {
            f32x4 sum = red[mi * 64u + lane];
#pragma unroll
            for (uint32_t w = 1; w < 4u; ++w) sum += red[(w * MI + mi) * 64u + lane];
            if (b0 + lo < B) {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const uint32_t m = mb + 16u * mi + 4u * hi + r;
                    if (m < M) Y[(uint64_t)m * B + b0 + lo] = sum[r];
                }
            }
        }
    }
}

template <int MI>
int launch_gemv(const float* W, const float* X, float* Y, uint32_t M, uint32_t N, uint32_t B,
                float scale, hipStream_t s)
{
    const size_t lds = (size_t)N * kCols * sizeof(float) + 4u * MI * 64u * sizeof(f32x4);
    auto kern = fused_ht_gemv_kernel<MI>;
    if (lds > 64u * 1024u) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
            return MI_ERR_LAUNCH;
    }
    // A workgroup keeps its transformed tile for several row blocks once there are more row
    // blocks than it takes to give every compute unit two workgroups.
    constexpr uint32_t kBlock = 16u * MI;
    const uint32_t col_groups = (B + kCols - 1) / kCols;
    const uint32_t row_blocks = (M + kBlock - 1) / kBlock;
    uint32_t groups_y = (512u + col_groups - 1) / col_groups;
    if (groups_y > row_blocks) groups_y = row_blocks;
    const uint32_t rows_per_group = ((row_blocks + groups_y - 1) / groups_y) * kBlock;
    const dim3 grid(col_groups, (M + rows_per_group - 1) / rows_per_group);
    hipLaunchKernelGGL(kern, grid, dim3(kThreads), lds, s, W, X, Y, M, N, B, ilog2(N), scale,
                       rows_per_group);
    return launch_status();
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
    hipStream_t s = static_cast<hipStream_t>(stream);
    const float* w = static_cast<const float*>(W);
    const float* x = static_cast<const float*>(X);
    float* y = static_cast<float*>(Y);
    // 64-row workgroups once that still gives every compute unit a workgroup; 32-row ones for
    // small problems, where more (shorter) workgroups matter more than the repeated transform,
    // and 16-row ones for the smallest (M = N = 1024, B <= 64: 12.2 -> 11.1 us)
    const uint64_t groups64 = (uint64_t)((B + kCols - 1) / kCols) * ((M + 63u) / 64u);
    if (groups64 >= 256u) return launch_gemv<4>(w, x, y, M, N, B, scale, s);
    if (groups64 < 128u) return launch_gemv<1>(w, x, y, M, N, B, scale, s);
    return launch_gemv<2>(w, x, y, M, N, B, scale, s);
}
