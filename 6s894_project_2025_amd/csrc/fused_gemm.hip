// Fused Hadamard -> GEMM (mi_fused_ht_gemm), gfx950:  C[M,N] = W[M,K] * (scale * H_K * X[K,N]),
// X given as Xt[N,K].  The transformed operand lives only in LDS.
//
// This file: the dispatcher and the LDS-resident variant, used for K = 32 .. 256 (64 columns per
// workgroup, a column at most half a 512-element tile).  K >= 512 goes to the register-resident
// variants in fused_gemm_xreg.hip and fused_gemm_xreg_k2048.hip, which hold more columns per
// compute unit.
//
// Structure ("X-stationary"): a workgroup owns BN columns of X for the whole K extent.
//   prologue : its wavefronts transform those BN rows of Xt on the matrix cores (tile_transform,
//              the stand-alone kernel's building block), round to the 16-bit type and park
//              them in LDS as Y[BN][K] (16-byte chunks XOR-swizzled so that both the prologue's
//              writes and the main loop's fragment reads are bank-conflict free);
//   main loop: each wavefront takes 64-row blocks of W inside the workgroup's M range.  W is
//              read from global memory with four adjacent lanes covering 64 contiguous bytes of
//              a row (the pattern the L1 coalesces; one lane per row runs at a quarter of the
//              rate), prefetched several K steps ahead into registers, and turned into MFMA
//              operand order (lane = row) through a 4 KB wavefront-private LDS staging area
//              (ds_write_b128 / ds_read_b128, both conflict-free under an XOR swizzle;
//              ds_bpermute moves only 4 bytes per lane and measured 3x slower).  It is contracted
//              against Y fragments read from LDS with v_mfma_f32_16x16x32; Y is the A operand and
//              W the B operand, so a lane ends up with 16 consecutive output columns of one row.
//   epilogue : the 64 x BN result block goes through the same staging area so that eight adjacent
//              lanes store 128 contiguous bytes of a row of C.
// The M range is split over gridDim.y workgroups so that the chip is filled.
//
// Behaviour replaced: fused_ht_gemm_pipelined, fused_ht/fusion_pipelined.cu:306-563 (cp.async
// double-buffered X tile + in-smem butterfly + scalar-FMA GEMM; fp32 only, compile-time dims).
#include <type_traits>

#include "fwht_device.hpp"
#include "lds_layout.hpp"

namespace mi {

// K = 512 ... 4096 with the transformed operand in registers: fused_gemm_xreg.hip
int fused_gemm16_xreg(const void* W, const void* Xt, void* C, uint32_t M, uint32_t N, uint32_t K,
                      int in_dtype, int out_f32, float scale, hipStream_t s);

namespace {

constexpr int kGemmThreads = 512;
constexpr int kGemmWaves = kGemmThreads / 64;
constexpr int kWaveRows = 64;   // rows of W per wavefront block
constexpr int kMI = kWaveRows / 16;
constexpr int kStageBytes = kWaveRows * 64;  // per-wavefront LDS staging: rows x 32 K x 2 B

// Byte offset of 16-byte chunk q of column n in the swizzled Y[BN][K] LDS image.
// `col_bytes` = bytes per column, LOG_NB = log2(16-column fragments per block): the fragment
// read of lane `lo` touches column NB*lo + nb, so the swizzle key is n / NB.
template <int LOG_NB>
__host__ __device__ constexpr uint32_t y_chunk_offset(uint32_t n, uint32_t q, uint32_t col_bytes,
                                                      uint32_t swz_mask)
{
    // built as (16-byte chunk index) << 4 so that the 16-byte alignment is visible to the compiler
    // and every access becomes a single ds_read_b128 / ds_write_b128
    return (n * (col_bytes >> 4) + (q ^ ((n >> LOG_NB) & swz_mask))) << 4;
}

// Per-wavefront staging of a 64-row x 32-K sub-step of W: row r (64 bytes), 16-byte chunk c stored
// at position c ^ ((r >> 1) & 3).  Writer lane l holds row l / 4, chunk l % 4 (coalescable global
// loads); reader lane (hi, lo) takes row lo, chunk hi (MFMA operand order).
__host__ __device__ constexpr uint32_t stage_write_offset(uint32_t lane)
{
    return (lane >> 2) * 64u + (((lane & 3u) ^ ((lane >> 3) & 3u)) << 4);
}
__host__ __device__ constexpr uint32_t stage_read_offset(uint32_t lane)
{
    return (lane & 15u) * 64u + (((lane >> 4) ^ (((lane & 15u) >> 1) & 3u)) << 4);
}
template <int LOG_NB>
constexpr bool y_patterns_conflict_free()
{
    // K >= 64 (at K = 32 a column is four chunks and the four-way key cannot separate eight lanes;
    // that size is a single step with no loop to protect)
    for (uint32_t K = 64; K <= 4096; K *= 2) {
        const uint32_t chunks = K >> 3, mask = (chunks >= 16u ? 16u : chunks) - 1u;
        // prologue write: lane l of tile t holds elements 512 t + 8 l ..: column e / K, chunk (e % K) / 8
        for (uint32_t t = 0; t < 4; ++t)
            if (!lds::conflict_free_b128([=](uint32_t lane) {
                    const uint32_t e = 512u * t + 8u * lane;
                    return y_chunk_offset<LOG_NB>(e / K, (e % K) >> 3, K * 2u, mask);
                }))
                return false;
        // fragment read: lane (hi, lo) takes column NB lo + nb, chunk q0 + hi (the pattern repeats
        // every 16 chunks)
        for (uint32_t nb = 0; nb < (1u << LOG_NB); ++nb)
            for (uint32_t q0 = 0; q0 < chunks && q0 < 16u; q0 += 4)
                if (!lds::conflict_free_b128([=](uint32_t lane) {
                        return y_chunk_offset<LOG_NB>(((lane & 15u) << LOG_NB) + nb, q0 + (lane >> 4), K * 2u, mask);
                    }))
                    return false;
    }
    return true;
}
static_assert(lds::conflict_free_b128(stage_write_offset) && lds::conflict_free_b128(stage_read_offset),
              "the W staging pattern would serialise");
static_assert(y_patterns_conflict_free<0>() && y_patterns_conflict_free<1>() && y_patterns_conflict_free<2>(),
              "an access pattern of the transformed tile would serialise");

template <class T16, int BN>
__global__ void __launch_bounds__(kGemmThreads)
fused_ht_gemm16_kernel(const typename T16::E* __restrict__ W, const typename T16::E* __restrict__ Xt,
                       void* __restrict__ C, uint32_t M, uint32_t N, uint32_t K, uint32_t logK,
                       uint32_t m_per_block, uint32_t msplit, int out_f32, float fscale)
{
    using E = typename T16::E;
    using V8 = typename T16::V8;
    constexpr int NB = BN / 16;  // 16-column fragments of Y (A-operand blocks)
    constexpr int LOG_NB = NB == 4 ? 2 : (NB == 2 ? 1 : 0);
    extern __shared__ __attribute__((aligned(16))) unsigned char ylds[];

    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint32_t lo = lane & 15u, hi = lane >> 4;
    // 1-D grid, M-slice index fastest: consecutive workgroup ids go to different XCDs, so every
    // XCD keeps working on the same few M slices of W and that slice stays in its L2.
    const uint32_t n0 = (blockIdx.x / msplit) * BN;
    const uint32_t m_begin = (blockIdx.x % msplit) * m_per_block;
    const uint32_t chunks_per_col = K >> 3;
    const uint32_t swz_mask = (chunks_per_col >= 16u ? 16u : chunks_per_col) - 1u;

    const uint32_t m_end = min(M, m_begin + m_per_block);
    unsigned char* stage = ylds + (size_t)BN * K * 2u + wave * kStageBytes;

    // ---- W stream state of this wavefront's current 64-row block ---------------------------------
    // Load pattern: for row block mi and half h, lane l reads the 16 bytes at row 16*mi + l/4,
    // k = 64*ks + 32*h + 8*(l%4): four adjacent lanes cover 64 contiguous bytes.
    constexpr int kDepth = 1;  // K64 steps of W in flight in registers (deeper measured slower)
    const uint32_t ksteps = K >> 6;
    // The workgroups of one XCD stream the same rows of W in lockstep; each starts its K loop at a
    // different step (the sum over k is order independent) so that they hit different L2 lines.
    const uint32_t krot = (blockIdx.x / msplit) & (ksteps - 1u);
    auto kmap = [&](uint32_t ks) { return (ks + krot) & (ksteps - 1u); };
    const E* wld[kMI];
    u32x4 wraw[kDepth][kMI][2];
    auto preload = [&](uint32_t mb) {
#pragma unroll
        for (int mi = 0; mi < kMI; ++mi) {
            const uint32_t m = min(mb + 16u * mi + (lane >> 2), M - 1u);  // masked at the store
            wld[mi] = W + (uint64_t)m * K + 8u * (lane & 3u);
        }
#pragma unroll
        for (int d = 0; d < kDepth; ++d)
            if ((uint32_t)d < ksteps) {
#pragma unroll
                for (int mi = 0; mi < kMI; ++mi)
#pragma unroll
                    for (int h = 0; h < 2; ++h)
                        wraw[d][mi][h] =
                            *reinterpret_cast<const u32x4*>(wld[mi] + 64u * kmap(d) + 32u * h);
            }
    };
    uint32_t mb = m_begin + wave * kWaveRows;
    // the first W loads do not depend on the transformed tile: put them in flight before the prologue
    if (mb < m_end && K >= 64u) preload(mb);

    // ---- prologue: Y = bf16(scale * H_K * X[:, n0:n0+BN]) into LDS -------------------------------
    {
        TileOperands<T16> ops;
        make_tile_operands<T16, 2>(logK, ops);
        constexpr int BATCH = 16;                         // tiles in flight per wavefront
        const uint32_t block_tiles = (BN * K) >> 9;       // 512-element tiles in this block
        const uint64_t total = (uint64_t)N * K;           // elements in Xt
        const uint64_t tile_base = ((uint64_t)n0 * K) >> 9;
        // GUARD = false: the block lies inside Xt and holds a whole number of batches
        auto run = [&](auto guard_tag) {
            constexpr bool GUARD = decltype(guard_tag)::value;
            for (uint32_t t0 = wave * BATCH; t0 < block_tiles; t0 += kGemmWaves * BATCH) {
                V8 in[BATCH];
#pragma unroll
                for (int c = 0; c < BATCH; ++c) {
                    const uint64_t off = (tile_base + t0 + c) * 512u + 8u * lane;
                    if (GUARD) {
#pragma unroll
                        for (int j = 0; j < 8; ++j) in[c][j] = (E)0.0f;  // past N / past the block
                        if (t0 + c < block_tiles && off + 8u <= total)
                            in[c] = *reinterpret_cast<const V8*>(Xt + off);
                    } else {
                        in[c] = *reinterpret_cast<const V8*>(Xt + off);
                    }
                }
#pragma unroll
                for (int g = 0; g < BATCH; ++g) {   // a tile holds 512 / K whole columns
                    if (GUARD && t0 + g >= block_tiles) continue;
                    f32x4 acc[2];
                    tile_transform<T16>(in[g], ops, acc);
                    V8 o;
#pragma unroll
                    for (int t = 0; t < 2; ++t)
#pragma unroll
                        for (int r = 0; r < 4; ++r) o[4 * t + r] = (E)(acc[t][r] * fscale);
                    const uint32_t e = (t0 + g) * 512u + 8u * lane;  // offset in the block
                    const uint32_t n = e >> logK, q = (e & (K - 1u)) >> 3;
                    *reinterpret_cast<V8*>(ylds + y_chunk_offset<LOG_NB>(n, q, K * 2u, swz_mask)) = o;
                }
            }
        };
        if (n0 + BN <= N && block_tiles % (kGemmWaves * BATCH) == 0)
            run(std::false_type{});
        else
            run(std::true_type{});
    }
    __syncthreads();

    // ---- main loop ------------------------------------------------------------------------------
    // staging layout for a 64-row x 32-K sub-step: row r (64 bytes), 16-byte chunk c stored at
    // position c ^ ((r >> 1) & 3) (measured conflict-free for both access orders).  Writer lane l
    // holds row 16*mi + l/4, chunk l%4; reader lane (hi, lo) takes row 16*mi + lo, chunk hi.
    const uint32_t wr_off = stage_write_offset(lane);
    const uint32_t rd_off = stage_read_offset(lane);

    while (mb < m_end) {
        f32x4 acc[NB][kMI];
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
            for (int mi = 0; mi < kMI; ++mi) acc[nb][mi] = f32x4{0.f, 0.f, 0.f, 0.f};

        if (K >= 64u) {
            // Software pipeline over 32-wide sub-steps: the LDS traffic of sub-step s+1 (staging
            // write, W fragment reads, Y fragment reads) is issued before the MFMAs of sub-step s.
            // Operand order: lane (hi, lo) needs row 16*mi + lo, k = 64*ks + 32*h + 8*hi + j; the Y
            // fragments use the same k assignment (chunk 8*ks + 4*h + hi).  LDS operations of one
            // wavefront complete in order, so the single staging area is safe: the reads of s were
            // issued before the writes of s+1.
            V8 a_nx[NB], b_nx[kMI];
            auto fetch = [&](const u32x4 (&src)[kMI][2], int h, uint32_t ks) {
#pragma unroll
                for (int mi = 0; mi < kMI; ++mi)
                    *reinterpret_cast<u32x4*>(stage + mi * 1024u + wr_off) = src[mi][h];
#pragma unroll
                for (int nb = 0; nb < NB; ++nb)
                    a_nx[nb] = *reinterpret_cast<const V8*>(
                        ylds + y_chunk_offset<LOG_NB>(NB * lo + nb, 8u * kmap(ks) + 4u * h + hi,
                                                      K * 2u, swz_mask));
#pragma unroll
                for (int mi = 0; mi < kMI; ++mi)
                    b_nx[mi] = *reinterpret_cast<const V8*>(stage + mi * 1024u + rd_off);
            };
            fetch(wraw[0], 0, 0);
            for (uint32_t ks0 = 0; ks0 < ksteps; ks0 += kDepth) {
#pragma unroll
                for (int d = 0; d < kDepth; ++d) {
                    const uint32_t ks = ks0 + d;
                    if (ks < ksteps) {
#pragma unroll
                        for (int h = 0; h < 2; ++h) {
                            V8 a_cu[NB], b_cu[kMI];
#pragma unroll
                            for (int nb = 0; nb < NB; ++nb) a_cu[nb] = a_nx[nb];
#pragma unroll
                            for (int mi = 0; mi < kMI; ++mi) b_cu[mi] = b_nx[mi];
                            if (h == 0) {
                                fetch(wraw[d], 1, ks);
                                // both halves of wraw[d] are now on their way to LDS: refill it
                                if (ks + kDepth < ksteps) {
#pragma unroll
                                    for (int mi = 0; mi < kMI; ++mi)
#pragma unroll
                                        for (int hh = 0; hh < 2; ++hh)
                                            wraw[d][mi][hh] = *reinterpret_cast<const u32x4*>(
                                                wld[mi] + 64u * kmap(ks + kDepth) + 32u * hh);
                                }
                            } else if (ks + 1 < ksteps) {
                                fetch(wraw[(d + 1) % kDepth], 0, ks + 1);
                            }
#pragma unroll
                            for (int mi = 0; mi < kMI; ++mi)
#pragma unroll
                                for (int nb = 0; nb < NB; ++nb)
                                    acc[nb][mi] = T16::mfma32(a_cu[nb], b_cu[mi], acc[nb][mi]);
                            // spread this sub-step's LDS and global traffic between its MFMAs
                            // instead of issuing it in one burst
#pragma unroll
                            for (int i = 0; i < 4; ++i) {
                                __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);  // DS write
                                __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);  // MFMA
                                __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);  // DS read
                                __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);  // MFMA
                                if (h == 0) __builtin_amdgcn_sched_group_barrier(0x020, 2, 0);  // VMEM read
                            }
                        }
                    }
                }
            }
        } else {
            // K = 32: a single 32-wide step, operands straight from global memory
            V8 a[NB];
#pragma unroll
            for (int nb = 0; nb < NB; ++nb)
                a[nb] = *reinterpret_cast<const V8*>(
                    ylds + y_chunk_offset<LOG_NB>(NB * lo + nb, hi, K * 2u, swz_mask));
#pragma unroll
            for (int mi = 0; mi < kMI; ++mi) {
                const uint32_t m = min(mb + 16u * mi + lo, M - 1u);
                const V8 bw = *reinterpret_cast<const V8*>(W + (uint64_t)m * K + 8u * hi);
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) acc[nb][mi] = T16::mfma32(a[nb], bw, acc[nb][mi]);
            }
        }

        // the next block's first W loads go out before this block's result is stored
        const uint32_t mb_next = mb + kGemmWaves * kWaveRows;
        if (mb_next < m_end && K >= 64u) preload(mb_next);

        // ---- epilogue ----------------------------------------------------------------------------
        // D[m'][n']: n' = lo is the row of W; m' = 4*hi + r is the A-operand lane, which carried
        // column NB*m' + nb.  So lane (hi, lo) owns, for row 16*mi + lo, the contiguous run of 4*NB
        // columns starting at 4*NB*hi, in the order v[NB*r + nb].
        if constexpr (NB == 4) {
            // Through the staging area, so that adjacent lanes store adjacent 16-byte pieces of a
            // row of C.  One round covers kStageBytes / (64 columns * element size) rows.
            const bool vec_ok = out_f32 ? ((N & 3u) == 0) : ((N & 7u) == 0);
            if (!out_f32) {
#pragma unroll
                for (int p = 0; p < kMI / 2; ++p) {  // 32 rows x 128 bytes per round
#pragma unroll
                    for (int mm = 0; mm < 2; ++mm) {
                        const int mi = 2 * p + mm;
                        const uint32_t rl = 16u * mm + lo;
#pragma unroll
                        for (int q = 0; q < 2; ++q) {
                            V8 o;
#pragma unroll
                            for (int i = 0; i < 8; ++i) {
                                const int idx = 8 * q + i;  // = NB*r + nb
                                o[i] = (E)acc[idx & 3][mi][idx >> 2];
                            }
                            *reinterpret_cast<V8*>(stage + rl * 128u +
                                                   (((2u * hi + q) ^ (rl & 7u)) << 4)) = o;
                        }
                    }
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const uint32_t rl = 8u * i + (lane >> 3), ch = lane & 7u;
                        const V8 o = *reinterpret_cast<const V8*>(stage + rl * 128u +
                                                                  ((ch ^ (rl & 7u)) << 4));
                        const uint32_t m = mb + 32u * p + rl, col = n0 + 8u * ch;
                        if (m < m_end && col < N) {
                            E* dst = static_cast<E*>(C) + (uint64_t)m * N + col;
                            if (vec_ok && col + 8u <= N) {
                                __builtin_nontemporal_store(o, reinterpret_cast<V8*>(dst));
                            } else {
#pragma unroll
                                for (int j = 0; j < 8; ++j)
                                    if (col + j < N) dst[j] = o[j];
                            }
                        }
                    }
                }
            } else {
#pragma unroll
                for (int mi = 0; mi < kMI; ++mi) {  // 16 rows x 256 bytes per round
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        f32x4 o;
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            const int idx = 4 * q + i;
                            o[i] = acc[idx & 3][mi][idx >> 2];
                        }
                        *reinterpret_cast<f32x4*>(stage + lo * 256u + (((4u * hi + q) ^ lo) << 4)) = o;
                    }
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const uint32_t rl = 4u * i + (lane >> 4), ch = lane & 15u;
                        const f32x4 o =
                            *reinterpret_cast<const f32x4*>(stage + rl * 256u + ((ch ^ rl) << 4));
                        const uint32_t m = mb + 16u * mi + rl, col = n0 + 4u * ch;
                        if (m < m_end && col < N) {
                            float* dst = static_cast<float*>(C) + (uint64_t)m * N + col;
                            if (vec_ok && col + 4u <= N) {
                                __builtin_nontemporal_store(o, reinterpret_cast<f32x4*>(dst));
                            } else {
#pragma unroll
                                for (int j = 0; j < 4; ++j)
                                    if (col + j < N) dst[j] = o[j];
                            }
                        }
                    }
                }
            }
        } else {
            // narrower tiles (K >= 2048): direct element-wise stores
#pragma unroll
            for (int mi = 0; mi < kMI; ++mi) {
                const uint32_t m = mb + 16u * mi + lo;
                if (m >= m_end) continue;
                const uint32_t col0 = n0 + (4u * NB) * hi;
#pragma unroll
                for (int r = 0; r < 4; ++r)
#pragma unroll
                    for (int nb = 0; nb < NB; ++nb) {
                        const uint32_t col = col0 + NB * r + nb;
                        if (col >= N) continue;
                        if (out_f32)
                            static_cast<float*>(C)[(uint64_t)m * N + col] = acc[nb][mi][r];
                        else
                            static_cast<E*>(C)[(uint64_t)m * N + col] = (E)acc[nb][mi][r];
                    }
            }
        }
        mb = mb_next;
    }
}

template <class T16, int BN>
int launch_gemm16(const void* W, const void* Xt, void* C, uint32_t M, uint32_t N, uint32_t K,
                  int out_f32, float scale, hipStream_t s)
{
    const uint32_t logK = ilog2(K);
    const int shift = tile_stage_shift<2>(logK, kNarrowRange<T16>);
    const float fscale = (float)((double)scale * (double)(1u << shift));
    const uint32_t n_tiles = (N + BN - 1) / BN;
    // split M so that about one workgroup per compute unit exists; each covers a multiple of
    // 512 rows (wavefronts x rows per wavefront block)
    const uint32_t row_blocks = (M + 511u) / 512u;
    uint32_t msplit = (256u + n_tiles - 1u) / n_tiles;
    if (msplit < 1u) msplit = 1u;
    if (msplit > row_blocks) msplit = row_blocks;
    const uint32_t m_per_block = ((row_blocks + msplit - 1u) / msplit) * 512u;
    msplit = (M + m_per_block - 1u) / m_per_block;
    const size_t lds = (size_t)BN * K * 2u + (size_t)kGemmWaves * kStageBytes;
    auto kern = fused_ht_gemm16_kernel<T16, BN>;
    if (lds > 64u * 1024u) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
            return MI_ERR_LAUNCH;
    }
    hipLaunchKernelGGL(kern, dim3(n_tiles * msplit), dim3(kGemmThreads), lds, s,
                       static_cast<const typename T16::E*>(W),
                       static_cast<const typename T16::E*>(Xt), C, M, N, K, logK, m_per_block, msplit,
                       out_f32, fscale);
    return launch_status();
}

template <class T16>
int dispatch_gemm16(const void* W, const void* Xt, void* C, uint32_t M, uint32_t N, uint32_t K,
                    int out_f32, float scale, hipStream_t s)
{
    switch (K) {
        case 32:
        case 64:
        case 128:
        case 256: return launch_gemm16<T16, 64>(W, Xt, C, M, N, K, out_f32, scale, s);
        case 512:
        case 1024:
        case 2048:
        case 4096: return fused_gemm16_xreg(W, Xt, C, M, N, K, T16::kCode, out_f32, scale, s);
        default: return MI_ERR_SIZE;
    }
}

}  // namespace

int fused_gemm_f32(const float* W, const float* Xt, float* C, uint32_t M, uint32_t N, uint32_t K,
                   float scale, hipStream_t s);  // fused_gemm_f32.hip

}  // namespace mi

extern "C" int mi_fused_ht_gemm(const void* W, const void* Xt, void* C, uint32_t M, uint32_t N,
                                uint32_t K, int in_dtype, int out_dtype, float scale, void* stream)
{
    using namespace mi;
    if (!is_pow2(K) || K < 32u || K > 4096u) return MI_ERR_SIZE;
    if (M == 0 || N == 0) return MI_OK;
    if (!W || !Xt || !C) return MI_ERR_NULL;
    if (!aligned16(W) || !aligned16(Xt) || !aligned16(C)) return MI_ERR_ALIGN;
    if (out_dtype != MI_F32 && out_dtype != in_dtype) return MI_ERR_DTYPE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (in_dtype) {
        case MI_F32:
            return fused_gemm_f32(static_cast<const float*>(W), static_cast<const float*>(Xt),
                                  static_cast<float*>(C), M, N, K, scale, s);
        case MI_BF16: return dispatch_gemm16<BF16>(W, Xt, C, M, N, K, out_dtype == MI_F32, scale, s);
        case MI_F16: return dispatch_gemm16<F16>(W, Xt, C, M, N, K, out_dtype == MI_F32, scale, s);
        default: return MI_ERR_DTYPE;
    }
}
