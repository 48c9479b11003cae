// Fused Hadamard + GEMV-batch (mi_fused_ht_gemv), fp32, gfx950:
//     Y[M,B] = W[M,N] * (scale * H_N * X[N,B]),  transform down dimension 0 of X.
//
// This file: the entry point, and the kernel for every shape but the large ones with N >= 512 (those
// that give every compute unit a 64-row workgroup go to fused_gemv_stream.hip).  A workgroup owns
// 16 columns of X and 16, 32 or 64 rows of W at a time; it keeps its transformed columns in LDS for
// several row blocks when there are more row blocks than compute units to spread them over.
//   prologue, N >= 512: gemv_common.hpp (the columns are brought into LDS column by column and
//              transformed there by the exact fp32 tile transform on the matrix cores), read by the
//              product as 16-byte B fragments.  N = 1024 measured 10.4 us per workgroup for the
//              register-butterfly prologue below (every LDS access 4 bytes, 128 of them per thread
//              and pass) against 4 us of loading and 6 us of transform for twice the columns there.
//   prologue, N < 512: the 16 columns are brought into LDS as T[N][16] (a row is 64 bytes, so the 16
//              column-lanes of a wavefront read global memory contiguously) while radix-16
//              register butterflies run: each thread owns one column and 16 rows per step, so
//              log2(N) stages cost ceil(log2(N)/4) passes over LDS, the first one straight from
//              global memory.  Row positions are XOR-swizzled so every access pattern below
//              touches four different 64-byte bank groups per wavefront.
//   product  : v_mfma_f32_16x16x4_f32 (32 cycles each) with W as the A operand (one 16-byte load
//              per lane gives four consecutive k for four MFMAs) and T as the B operand; each W
//              element is read once per workgroup instead of once per column.  The four wavefronts
//              each take a quarter of the K steps with four steps of loads in flight, the B
//              fragments of a step read one step early, and their partial sums are added through
//              LDS.  A load instruction of this form touches 16 rows of W and 64 bytes of each; the
//              vector cache handles a request per 128-byte line however little of it is asked for,
//              which bounds this loop at 16 - 17 bytes per clock and compute unit, half of what the
//              matrix cores could take with 16 columns: fused_gemv_stream.hip is the answer to that.
//   placement: workgroups are numbered so that the column groups sharing a slice of W run on one
//              XCD (one L2), or the row groups sharing a column tile.
//
// Behaviour replaced: fused_hadamard_gemv_kernel(_vec), fused_ht/fwht_gemv_fusion.cu:98-244, where
// every column's block re-reads all of W and reduces with warp shuffles.
#include "gemv_common.hpp"

namespace mi {
namespace {

constexpr int kCols = 16;
constexpr int kThreads = 256;

using gemv::GemvPlan;
using gemv::kPad;
using gemv::kXcds;
using gemv::lds_barrier;
using gemv::plan_gemv;

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

// One radix-2^WBITS pass over index bits [shift, shift + WBITS).  FROM: 0 the LDS tile, 1 X[N][B] in
// global memory, 2 X given column by column (Xt[B][N], the layout of mi_fused_ht_gemm).
// Each thread owns one column and works on SETS butterfly sets at a time, all of their loads
// issued before any arithmetic (the pass from global memory is latency-bound otherwise).
template <int WBITS, int FROM>
__device__ __forceinline__ void pass(const float* __restrict__ X, float* tile, uint32_t N,
                                     uint32_t B, uint32_t b0, uint32_t shift, float mul)
{
    constexpr int R = 1 << WBITS;
    constexpr bool FROM_GLOBAL = FROM != 0;
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
                    if (FROM == 1)
                        v[u][i] = col_ok ? X[(uint64_t)r * B + b0 + c] : 0.0f;
                    else if (FROM == 2)
                        v[u][i] = col_ok ? X[(uint64_t)(b0 + c) * N + r] : 0.0f;
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

template <int FROM>
__device__ __forceinline__ void pass_w(int wbits, const float* __restrict__ X, float* tile,
                                       uint32_t N, uint32_t B, uint32_t b0, uint32_t shift,
                                       float mul)
{
    switch (wbits) {
        case 1: pass<1, FROM>(X, tile, N, B, b0, shift, mul); break;
        case 2: pass<2, FROM>(X, tile, N, B, b0, shift, mul); break;
        case 3: pass<3, FROM>(X, tile, N, B, b0, shift, mul); break;
        case 4: pass<4, FROM>(X, tile, N, B, b0, shift, mul); break;
        default: pass<5, FROM>(X, tile, N, B, b0, shift, mul); break;
    }
}

// MI = 16-row blocks of W per workgroup (16, 32 or 64 rows).  The four wavefronts split the K range
// of the product between them (every wavefront covers all MI row blocks over a quarter of N), so
// each one streams a short, deeply prefetched run of W, and the partial sums meet in LDS.
// (Eight wavefronts per workgroup, two per SIMD, measured no faster where a compute unit holds one
// workgroup anyway: the transform of a column costs a SIMD about 1 400 cycles of MFMA and vector
// issue whoever issues them.  M = N = 1024: B = 64 8.7 instead of 9.2 us, B = 8 8.9 instead of 8.5.)
// XT: X is given column by column (Xt[B][N]); the register-butterfly prologue only.
template <int MI, bool TILED, bool XT>
__global__ void __launch_bounds__(kThreads)
fused_ht_gemv_kernel(const float* __restrict__ W, const float* __restrict__ X,
                     float* __restrict__ Y, uint32_t M, uint32_t N, uint32_t B, uint32_t logN,
                     float scale, uint32_t rows_per_group, uint32_t col_groups, uint32_t row_groups,
                     uint32_t per_xcd, bool col_major)
{
    static_assert(!(TILED && XT), "the column-major staging reads X[N][B]");
    constexpr int NC = kCols, WAVES = kThreads / 64;
    constexpr int PF = 4;        // K steps (of 16) in flight per wavefront
    constexpr int NF = NC / 16;  // 16-column fragments of the product per workgroup
    extern __shared__ __attribute__((aligned(16))) float tile[];  // [N][16] rows swizzled, then sums
    // Workgroups are handed to the eight XCDs in turn, each with an L2 of its own.  Position
    // (XCD, slot) takes place XCD * per_xcd + slot of an order of the tiles in which neighbours
    // share data: row-group-major (the column groups that share a slice of W side by side on one
    // XCD, which reads the slice once from beyond its L2 and all of X it needs) or, col_major,
    // column-group-major (the row groups that share a column tile side by side: little of X per
    // XCD, all of W).  The launcher picks the second when the first would have every XCD fetch
    // more than 2 MB of X at once: the column tiles are wanted all at the same moment, at the
    // start, while W is streamed over the whole K loop ((1024, 1024, 2048): 52.7 -> 48.7 us).
    const uint32_t place = (blockIdx.x % kXcds) * per_xcd + blockIdx.x / kXcds;
    if (place >= col_groups * row_groups) return;
    const uint32_t b0 = (col_major ? place / row_groups : place % col_groups) * NC;
    // the wavefront's index as a scalar: everything derived from it (its K range above all) then
    // steers branches instead of lane masks
    const uint32_t lane = threadIdx.x & 63u, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t lo = lane & 15u, hi = lane >> 4;
    // this workgroup's rows: [m_first, m_last), a multiple of 16 * MI except at the end of W
    const uint32_t m_first = (col_major ? place % row_groups : place / col_groups) * rows_per_group;
    const uint32_t m_last = min(M, m_first + rows_per_group);

    const uint32_t total = N >> 4;
    const uint32_t quarter = (total + (uint32_t)WAVES - 1u) / (uint32_t)WAVES;  // a wavefront's share of the K steps
    const uint32_t k_begin = min(wave * quarter, total), k_end = min(k_begin + quarter, total);
    // The wavefront's i-th K step.  TILED (N >= 512, so the steps divide evenly): steps 2p and
    // 2p+1 of a wavefront are the two 64-byte halves of one 128-byte line of each row of W, asked
    // for together, and the four wavefronts take adjacent lines.  (With a quarter of the K range
    // each, the halves of a line were asked for a step apart, with 256 other lines of rows a
    // multiple of 4 KB apart in between.  Measured: N = 2048, 33.6 -> 31.4 thousand cycles per
    // row block; N = 1024, no change.)
    auto kof = [&](uint32_t i) { return TILED ? (i >> 1) * (2u * WAVES) + 2u * wave + (i & 1u) : k_begin + i; };
    const float* wrow[MI];
    f32x4 a[PF][MI];
    auto rows_of = [&](uint32_t mb, const float* (&rows)[MI]) {
#pragma unroll
        for (int mi = 0; mi < MI; ++mi) {
            const uint32_t m = min(mb + 16u * mi + lo, M - 1u);
            rows[mi] = W + (uint64_t)m * N + 4u * hi;
        }
    };
    auto start_block = [&](uint32_t mb) {
        rows_of(mb, wrow);
        if constexpr (TILED) {
#pragma unroll
            for (int j = 0; j < PF; j += 2)
#pragma unroll
                for (int mi = 0; mi < MI; ++mi) {
                    a[j][mi] = *reinterpret_cast<const f32x4*>(wrow[mi] + 16u * kof(j));
                    a[j + 1][mi] = *reinterpret_cast<const f32x4*>(wrow[mi] + 16u * kof(j + 1));
                }
        } else {
#pragma unroll
            for (int j = 0; j < PF; ++j)
                if (k_begin + j < k_end) {
#pragma unroll
                    for (int mi = 0; mi < MI; ++mi)
                        a[j][mi] = *reinterpret_cast<const f32x4*>(wrow[mi] + 16u * kof(j));
                }
        }
    };
    // The first W fragments do not depend on the transform.  N < 512: start them before the
    // prologue; N >= 512: behind the loads of the column tile, which the prologue waits for first.
    if constexpr (!TILED) start_block(m_first);

    // ---- prologue: T = scale * H_N * X[:, b0:b0+16] --------------------------------------------
    const uint32_t cstride = N + kPad;  // TILED: floats per column of TT
    if constexpr (TILED) {
        gemv::stage_column_tile<NC, WAVES>(X, tile, N, B, b0, lane, wave, gemv::first_row_of(blockIdx.x));
        start_block(m_first);
        lds_barrier();
        gemv::transform_column_tile<NC, WAVES>(tile, N, B, b0, scale, lane, wave);
        lds_barrier();
    } else {
        uint32_t done = 0;
        bool first = true;
        uint32_t passes_left = (logN + 4u) / 5u;  // fewest radix-32 passes, bits spread evenly
        while (done < logN) {
            const int wbits = (int)((logN - done + passes_left - 1u) / passes_left);
            --passes_left;
            const float mul = (done + wbits == logN) ? scale : 1.0f;
            if (first)
                pass_w<XT ? 2 : 1>(wbits, X, tile, N, B, b0, done, mul);
            else
                pass_w<0>(wbits, X, tile, N, B, b0, done, mul);
            first = false;
            done += wbits;
            __syncthreads();
        }
    }
    // [MI * NF fragments][3 other wavefronts][64 lanes]
    f32x4* red = reinterpret_cast<f32x4*>(tile + (size_t)(TILED ? cstride : N) * NC);

    for (uint32_t mb = m_first; mb < m_last; mb += 16u * MI) {
        // TILED: the previous block's last steps have already started this block's first loads
        const bool has_next = mb + 16u * MI < m_last;
        const float* wnext[MI];
        if constexpr (TILED) {
            if (has_next) rows_of(mb + 16u * MI, wnext);
        } else {
            if (mb != m_first) start_block(mb);
        }
        // ---- product ------------------------------------------------------------------------------
        f32x4 acc[MI * NF];  // fragment g = mi * NF + f: rows 16 mi .., columns 16 f ..
#pragma unroll
        for (int g = 0; g < MI * NF; ++g) acc[g] = f32x4{0.f, 0.f, 0.f, 0.f};
        // One K step (16 columns of W) for all fragments.  refill: start the W loads PF steps ahead;
        // more (TILED): read the next step's B fragments now, a step before their MFMAs.
        f32x4 bq[2][NF];
        auto read_b = [&](uint32_t k, f32x4 (&o)[NF]) __attribute__((always_inline)) {
            if constexpr (TILED) {
                const f32x4* const tile4 = reinterpret_cast<const f32x4*>(tile);
#pragma unroll
                for (int f = 0; f < NF; ++f) o[f] = tile4[(16u * f + lo) * (cstride / 4u) + 4u * k + hi];
            } else {
#pragma unroll
                for (int s = 0; s < 4; ++s) o[0][s] = tile[prow(16u * k + 4u * hi + s) * kCols + lo];
            }
        };
        auto k_step = [&](uint32_t i, int j, int refill, bool more) __attribute__((always_inline)) {
            const uint32_t k = kof(i);
            if (TILED && more) {
                read_b(kof(i + 1u), bq[(j + 1) & 1]);
                __builtin_amdgcn_sched_barrier(0);  // ahead of this step's MFMAs, not behind them
            }
            if (!TILED) read_b(k, bq[j & 1]);
#pragma unroll
            for (int s = 0; s < 4; ++s)
#pragma unroll
                for (int mi = 0; mi < MI; ++mi)
#pragma unroll
                    for (int f = 0; f < NF; ++f)
                        acc[mi * NF + f] = __builtin_amdgcn_mfma_f32_16x16x4f32(
                            a[j][mi][s], bq[j & 1][f][s], acc[mi * NF + f], 0, 0, 0);
            if constexpr (TILED) {
                // steps 2p and 2p+1 are the halves of a 128-byte line: ask for both together
                if (refill != 0 && (j & 1)) {
                    const float* const* src = refill == 1 ? wrow : wnext;  // 2: the next row block
                    const uint32_t at = refill == 1 ? i + PF : (uint32_t)j;
#pragma unroll
                    for (int mi = 0; mi < MI; ++mi) {
                        a[j - 1][mi] = *reinterpret_cast<const f32x4*>(src[mi] + 16u * kof(at - 1u));
                        a[j][mi] = *reinterpret_cast<const f32x4*>(src[mi] + 16u * kof(at));
                    }
                }
            } else if (refill == 1) {
#pragma unroll
                for (int mi = 0; mi < MI; ++mi)
                    a[j][mi] = *reinterpret_cast<const f32x4*>(wrow[mi] + 16u * kof(i + PF));
            }
            // keep every step's loads in the step: left to itself the scheduler gathers the loads
            // of a round behind its last MFMA and waits for all of them before the next one
            __builtin_amdgcn_sched_barrier(0);
        };
        if constexpr (TILED) {
            // every wavefront has a whole number of PF-step rounds: all but the last refill the ring
            read_b(kof(0), bq[0]);
            for (uint32_t ii = 0; ii + PF < quarter; ii += PF) {
#pragma unroll
                for (int j = 0; j < PF; ++j) k_step(ii + j, j, 1, true);
            }
            if (has_next) {
#pragma unroll
                for (int j = 0; j < PF; ++j) k_step(quarter - PF + j, j, 2, j + 1 < PF);
#pragma unroll
                for (int mi = 0; mi < MI; ++mi) wrow[mi] = wnext[mi];
            } else {
#pragma unroll
                for (int j = 0; j < PF; ++j) k_step(quarter - PF + j, j, 0, j + 1 < PF);
            }
        } else if (N >= 16u) {
            for (uint32_t ii = 0; k_begin + ii < k_end; ii += PF) {
#pragma unroll
                for (int j = 0; j < PF; ++j)
                    if (k_begin + ii + j < k_end) k_step(ii + j, j, k_begin + ii + j + PF < k_end ? 1 : 0, false);
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

        // ---- meet the wavefronts' K shares in LDS ------------------------------------------------
        // Fragment g is finished by wavefront g % WAVES, which keeps its own partial sum in
        // registers: only the others go through LDS (12 KB instead of 16 for 64 rows by 16 columns
        // and four wavefronts, which is what lets two such workgroups with N = 1024 share a compute
        // unit).  The sum is taken in the order of the wavefronts, whoever holds which part.
        constexpr int G = MI * NF;
        // D[m'][n']: n' = lo is the column, m' = 4*hi + r the row inside the 16-row block
        lds_barrier();  // the sums of the row block before have been read
#pragma unroll
        for (int g = 0; g < G; ++g) {
            const uint32_t owner = (uint32_t)(g % WAVES);
            if (wave != owner) red[((uint32_t)g * (WAVES - 1) + (wave < owner ? wave : wave - 1u)) * 64u + lane] = acc[g];
        }
        lds_barrier();
#pragma unroll
        for (int g = 0; g < G; ++g) {
            const int owner = g % WAVES;
            if (wave != (uint32_t)owner) continue;
            f32x4 sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int w = 0; w < WAVES; ++w) {
                const f32x4 part = w == owner ? acc[g] : red[(g * (WAVES - 1) + (w < owner ? w : w - 1)) * 64 + lane];
                sum = w == 0 ? part : sum + part;
            }
            const uint32_t col = b0 + 16u * (uint32_t)(g % NF) + lo;
            if (col < B) {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const uint32_t m = mb + 16u * (uint32_t)(g / NF) + 4u * hi + r;
                    if (m < M) Y[(uint64_t)m * B + col] = sum[r];
                }
            }
        }
    }
}

inline size_t gemv_lds_bytes(uint32_t N, bool tiled, uint32_t nc, uint32_t mi, uint32_t waves)
{
    return (size_t)(N + (tiled ? kPad : 0u)) * nc * sizeof(float) + (size_t)(waves - 1u) * mi * (nc / 16u) * 64u * sizeof(f32x4);
}

template <int MI, bool TILED, bool XT>
int launch_gemv_as(const float* W, const float* X, float* Y, uint32_t M, uint32_t N, uint32_t B,
                   float scale, hipStream_t s)
{
    constexpr uint32_t NC = kCols, WAVES = kThreads / 64;
    const size_t lds = gemv_lds_bytes(N, TILED, NC, MI, WAVES);
    // the tile transform's two MFMA stages attenuate by a power of two that the scale takes back
    if (TILED) scale = (float)((double)scale * (double)(1u << tile_stage_shift<4>(9u, false)));
    auto kern = fused_ht_gemv_kernel<MI, TILED, XT>;
    if (lds > 64u * 1024u) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
            return MI_ERR_LAUNCH;
    }
    const GemvPlan p = plan_gemv(M, B, NC, 16u * MI, lds);
    const uint32_t per_xcd = (p.workgroups() + kXcds - 1) / kXcds;
    // bytes of X an XCD needs under the row-group-major order: its column groups' tiles
    const uint64_t x_per_xcd = (uint64_t)(p.col_groups < per_xcd ? p.col_groups : per_xcd) * NC * N * sizeof(float);
    const bool col_major = x_per_xcd > (2ull << 20);
    hipLaunchKernelGGL(kern, dim3(per_xcd * kXcds), dim3(64 * WAVES), lds, s, W, X, Y, M, N, B,
                       ilog2(N), scale, p.rows_per_group, p.col_groups, p.row_groups, per_xcd, col_major);
    return launch_status();
}

template <int MI>
int launch_gemv(const float* W, const float* X, float* Y, uint32_t M, uint32_t N, uint32_t B,
                float scale, bool xt, hipStream_t s)
{
    if (N < 512u)
        return xt ? launch_gemv_as<MI, false, true>(W, X, Y, M, N, B, scale, s)
                  : launch_gemv_as<MI, false, false>(W, X, Y, M, N, B, scale, s);
    if (xt) return MI_ERR_SIZE;  // (no caller: mi_fused_ht_gemm sends N >= 512 here only on large shapes)
    return launch_gemv_as<MI, true, false>(W, X, Y, M, N, B, scale, s);
}

}  // namespace

namespace gemv {

// The kernel for a shape; arguments already validated.  `columns_contiguous`: X is given as Xt[B][N]
// (mi_fused_ht_gemm's layout) instead of X[N][B].
int launch_any(const float* w, const float* x, float* y, uint32_t M, uint32_t N, uint32_t B, float scale,
               bool columns_contiguous, hipStream_t s)
{
    // N >= 512 on shapes that give every compute unit a 64-row, 16-column workgroup: the kernels that
    // hold the transformed columns in registers and stream W through the LDS in whole lines.
    //   N = 512, 1024 (fused_gemv_rows.hip: every wavefront holds all of K, the wavefronts split the
    //   rows): (1024, 1024, 256) 14.4 -> 11.7 us, (1024, 1024, 512) 19.1 -> 16.1, (1024, 1024, 2048)
    //   48.0 -> 40.3, (4096, 1024, 4096) 300 -> 257, (512, 512, 1024) 11.6 -> 10.0, (4096, 512, 4096)
    //   171 -> 139 against this file's kernel with 16 or 32 columns in LDS;
    //   N = 2048 (fused_gemv_stream.hip: the wavefronts split K): (2048, 2048, 512) 73 -> 46.
    const uint64_t groups64 = (uint64_t)((B + kCols - 1) / kCols) * ((M + 63u) / 64u);
    //   N = 256 (the same kernel with 64 columns per workgroup, which is what 256 registers hold of
    //   such columns) from 128 pairs of 64 columns x 64 rows on: (1024, 256, 1024) 15.5 -> 11.3 us,
    //   (2048, 256, 2048) 46.4 -> 24.7, (4096, 256, 4096) 153 -> 72, (1024, 256, 512) 13.6 -> 11.1,
    //   (512, 256, 1024) 11.0 -> 11.1, (512, 256, 512) 10.7 -> 10.9.
    if (N == 256u && (uint64_t)((B + 63u) / 64u) * ((M + 63u) / 64u) >= 128u)
        return launch_rows(w, x, y, M, N, B, scale, columns_contiguous, s);
    if (groups64 >= 256u) {
        if (N == 512u || N == 1024u) return launch_rows(w, x, y, M, N, B, scale, columns_contiguous, s);
        if (N == 2048u) return launch_stream_2048(w, x, y, M, B, scale, columns_contiguous, s);
    }
    // otherwise 64-row workgroups once that still gives every compute unit a workgroup; 32-row ones
    // for small problems, where more (shorter) workgroups matter more than the repeated transform,
    // and 16-row ones for the smallest (M = N = 1024, B <= 64: 12.2 -> 11.1 us)
    if (groups64 >= 256u) return launch_gemv<4>(w, x, y, M, N, B, scale, columns_contiguous, s);
    if (groups64 < 128u) return launch_gemv<1>(w, x, y, M, N, B, scale, columns_contiguous, s);
    return launch_gemv<2>(w, x, y, M, N, B, scale, columns_contiguous, s);
}

}  // namespace gemv
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
    return gemv::launch_any(w, x, y, M, N, B, scale, false, s);
}
