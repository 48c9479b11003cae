// The prologue of the fused Hadamard + GEMV kernels for N >= 512 (fused_gemv.hip,
// fused_gemv_stream.hip): a tile of NC columns of X[N, B] is brought into LDS column by column and
// transformed there, TT = scale * H_N * X[:, b0 .. b0 + NC - 1].
//
// Column c of the tile lives at TT + c * (N + kPad) floats.  With a row stride of 16 bytes modulo
// 128 the 16-byte accesses of eight adjacent lanes (eight columns, the same k) fall into eight
// different 16-byte columns of the LDS row, as do those of eight lanes on consecutive k of one
// column.
//
// Behaviour replaced: the shared-memory butterflies of fused_hadamard_gemv_kernel,
// fused_ht/fwht_gemv_fusion.cu:118-133.
#pragma once

#include <type_traits>

#include "fwht_device.hpp"

namespace mi {
namespace gemv {

constexpr uint32_t kPad = 4;
constexpr uint32_t kXcds = 8;

// Workgroup barrier for data exchanged through LDS only.  __syncthreads() also waits for every
// outstanding global load (a release at workgroup scope), which would end the flight of the W
// fragments requested ahead of the prologue and of the next row block at exactly the points
// where they are meant to overlap other work; nothing here passes data between wavefronts through
// global memory.
__device__ __forceinline__ void lds_barrier()
{
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// Where workgroup `id` of a launch starts reading its column tile: 64-row steps, neighbours in time
// (ids run over the XCDs first) far apart.
__device__ __forceinline__ uint32_t first_row_of(uint32_t id) { return 64u * (id * 5u); }

// X[:, b0 .. b0+NC-1] -> TT: a thread reads four adjacent columns of a row.  A wavefront covers 16
// rows by 16 columns, so that its four-byte LDS writes (bank = 16 * (column / 4) + row modulo 64)
// never meet in a bank.  Columns past the end of X are filled with zeros.  The caller puts a
// workgroup barrier between this and the transform.
// ROWS_AHEAD = rows in flight per thread (0: as many as make a round of 512 rows).  A round waits out
// one latency of the memory system, about 2.5 us when every workgroup of a launch starts here at
// once, so a kernel with the registers to spare asks for the whole tile at once.
// `first_row`: the row the workgroup starts with (it wraps around at N).  Workgroups that start a
// launch together and all walk down the rows of X from row 0 ask the memory system for the same
// few rows at the same moment; spread over the rows the tile of M = N = 2048, B = 512 arrives in
// 3.6 us instead of 10.
template <int NC, int WAVES, int ROWS_AHEAD = 0>
__device__ __forceinline__ void stage_column_tile(const float* __restrict__ X, float* tile, uint32_t N, uint32_t B,
                                                  uint32_t b0, uint32_t lane, uint32_t wave, uint32_t first_row)
{
    const uint32_t cstride = N + kPad;
    constexpr uint32_t WQ = NC / 16;                     // wavefronts side by side along a row
    constexpr uint32_t RP = 16u * (uint32_t)WAVES / WQ;  // rows per pass of the workgroup
    const uint32_t q4 = (lane & 3u) + 4u * (wave % WQ), r0 = (lane >> 2) + 16u * (wave / WQ);
    // this thread's four columns: all inside X and 16-byte loadable, some, or none
    const uint32_t c4 = b0 + 4u * q4;
    const bool vec_ok = c4 + 4u <= B && (B & 3u) == 0;
    const bool any = c4 < B;
    // DEPTH rows in flight per thread (DEPTH * RP divides N): the tile is NC * 4 bytes of each of N
    // rows, from the L2
    constexpr int DEPTH = ROWS_AHEAD ? ROWS_AHEAD : 512u / RP;
    static_assert(DEPTH >= 1 && DEPTH <= 32 && (DEPTH * RP) % 256u == 0, "a round of DEPTH passes covers whole (half) tiles of rows");
    for (uint32_t rb = r0; rb < N; rb += (uint32_t)DEPTH * RP) {
        f32x4 v[DEPTH];
#pragma unroll
        for (int u = 0; u < DEPTH; ++u) {
            const uint32_t r = (rb + (uint32_t)u * RP + first_row) & (N - 1u);  // N is a power of two
            v[u] = f32x4{0.f, 0.f, 0.f, 0.f};
            const uint64_t at = (uint64_t)r * B + c4;
            if (vec_ok) {
                v[u] = *reinterpret_cast<const f32x4*>(X + at);
            } else if (any) {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (c4 + e < B) v[u][e] = X[at + e];
            }
        }
#pragma unroll
        for (int u = 0; u < DEPTH; ++u) {
            const uint32_t r = (rb + (uint32_t)u * RP + first_row) & (N - 1u);  // N is a power of two
#pragma unroll
            for (int e = 0; e < 4; ++e) tile[(4u * q4 + e) * cstride + r] = v[u][e];
        }
    }
}

// The same tile from X given column by column (Xt[B][N], each column of X contiguous: the layout of
// mi_fused_ht_gemm): a straight copy, 16 bytes per thread and access, every load of the tile in
// flight at once.  Columns past the end of X are filled with zeros.
template <int NC, int WAVES, int N>
__device__ __forceinline__ void stage_column_tile_xt(const float* __restrict__ Xt, float* tile, uint32_t B, uint32_t b0,
                                                     uint32_t tid)
{
    constexpr uint32_t cstride = N + kPad, kPerColumn = N / 4u;     // 16-byte chunks per column
    constexpr int PER_THREAD = NC * (int)kPerColumn / (64 * WAVES);  // chunks per thread
    static_assert(PER_THREAD >= 1 && PER_THREAD <= 32 && NC * kPerColumn % (64u * WAVES) == 0u, "whole rounds of the workgroup");
    f32x4 v[PER_THREAD];
#pragma unroll
    for (int u = 0; u < PER_THREAD; ++u) {
        const uint32_t at = tid + (uint32_t)u * 64u * WAVES, c = at / kPerColumn, q = at % kPerColumn;
        v[u] = b0 + c < B ? *reinterpret_cast<const f32x4*>(Xt + ((uint64_t)(b0 + c) * N + 4u * q)) : f32x4{0.f, 0.f, 0.f, 0.f};
    }
#pragma unroll
    for (int u = 0; u < PER_THREAD; ++u) {
        const uint32_t at = tid + (uint32_t)u * 64u * WAVES, c = at / kPerColumn, q = at % kPerColumn;
        *reinterpret_cast<f32x4*>(tile + c * cstride + 4u * q) = v[u];
    }
}

// Wavefront w transforms columns w, w + WAVES, w + 2 WAVES, ... of the tile, those that exist in X
// (a last or only column group may hold fewer than NC: with B = 8 every wavefront has two columns
// to do, not four for two of them and four columns of zeros for the others).  Its tiles (NT = N /
// 512 per column) are taken in pairs whose MFMA chains interleave, the next pair's LDS reads and
// three-way splits sitting in the shadow of this pair's MFMAs (one wavefront per SIMD may be all
// there is); the tiles of a column are then joined by fp32 butterflies in registers.  Columns past
// the end of X are left as they are: a column of the B operand reaches only its own column of the
// product, which is not stored.  `scale` carries the power of two that the two MFMA stages take
// out (tile_stage_shift<4>(9, false)).
// (A pair of tiles is 28 MFMAs and about 136 other instructions, and a wavefront that has its SIMD
// to itself issues one instruction per eight cycles: 1 300 cycles of issue before any wait, whatever
// the order.  Handing the next pair's split out evenly between the MFMAs with scheduling groups,
// three vector instructions behind each bf16 MFMA and five behind each fp32 one, changed nothing;
// nor did stage 1 on the fp32 matrix cores, eight MFMAs of 32 cycles on the unsplit data instead of
// three of 16 on the pieces: 48 MFMAs a pair, 1 536 cycles, the same 0.8 us; with a column's
// butterflies, scale and write-back handed out between the next column's MFMAs as well, N = 1024
// went from 3.2 to 2.9 us per four columns and N = 2048 from 6.5 to 7.2; one tile of a pair in each
// form, 1 120 cycles of matrix core beside a hundred other instructions, measured 3.2 and 6.8.)
template <int NT, int NC, int WAVES>
__device__ __forceinline__ void transform_column_tile_as(float* tile, uint32_t N, uint32_t B, uint32_t b0,
                                                         float scale, uint32_t lane, uint32_t wave)
{
    const uint32_t cstride = N + kPad;
    TileOperands<BF16> ops;
    make_tile_operands<BF16, 4>(9, ops);
    constexpr int XB = NT == 4 ? 2 : (NT == 2 ? 1 : 0);
    constexpr int HOLD = NT > 2 ? NT : 2;  // tiles of a unit: a column, or two of one tile
    constexpr int UPAIRS = HOLD / 2;       // pairs of tiles per unit
    const uint32_t ncols = min((uint32_t)NC, B - b0);
    const uint32_t mine = ncols > wave ? (ncols - wave + WAVES - 1u) / WAVES : 0u;  // columns of this wavefront
    const uint32_t units = NT == 1 ? (mine + 1u) / 2u : mine;
    // tile t of unit u: NT > 1: tile t of the wavefront's u-th column; NT = 1: column 2u + t
    auto at = [&](uint32_t u, int t) {
        const uint32_t j = NT == 1 ? 2u * u + (uint32_t)t : u;
        const uint32_t c = min(wave + (uint32_t)WAVES * j, (uint32_t)NC - 1u);  // (NT = 1, odd count: a spare column)
        return tile + c * cstride + (NT == 1 ? 0u : 512u * (uint32_t)t);
    };
    auto fetch = [&](uint32_t u, int t, SplitTileF32& o) __attribute__((always_inline)) {
        float in[8];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const f32x4 q = *reinterpret_cast<const f32x4*>(at(u, t) + 256u * h + 4u * lane);
#pragma unroll
            for (int r = 0; r < 4; ++r) in[4 * h + r] = q[r];
        }
        split_tile_f32(in, o);
    };
    if (units == 0u) return;
    SplitTileF32 cur[2], nxt[2];
    fetch(0u, 0, cur[0]);
    fetch(0u, 1, cur[1]);
    auto unit = [&](uint32_t u, bool more) __attribute__((always_inline)) {
        f32x4 held[HOLD][2];
#pragma unroll
        for (int q = 0; q < UPAIRS; ++q) {
            if (q + 1 < UPAIRS) {
                fetch(u, 2 * q + 2, nxt[0]);
                fetch(u, 2 * q + 3, nxt[1]);
            } else if (more) {
                fetch(u + 1u, 0, nxt[0]);
                fetch(u + 1u, 1, nxt[1]);
            }
            f32x4 a[2][2];
            tile_pair_mfma_f32(cur, ops, a);
#pragma unroll
            for (int c = 0; c < 2; ++c)
#pragma unroll
                for (int h = 0; h < 2; ++h) held[2 * q + c][h] = a[c][h];
            cur[0] = nxt[0];
            cur[1] = nxt[1];
        }
        if constexpr (NT > 1) cross_tile_butterflies<NT, XB>(held);
#pragma unroll
        for (int i = 0; i < HOLD; ++i)
#pragma unroll
            for (int h = 0; h < 2; ++h)
                *reinterpret_cast<f32x4*>(at(u, i) + 256u * h + 4u * lane) = held[i][h] * scale;
    };
    // a full tile: the same number of units for every wavefront, one straight-line sequence
    constexpr uint32_t FULL_UNITS = (NC / WAVES) / (NT == 1 ? 2 : 1);
    if (ncols == (uint32_t)NC) {
#pragma unroll
        for (uint32_t u = 0; u < FULL_UNITS; ++u) unit(u, u + 1u < FULL_UNITS);
    } else {
        for (uint32_t u = 0; u < units; ++u) unit(u, u + 1u < units);
    }
}

// N = 256: a 512-element tile is two adjacent columns (the operands leave the tile's upper index bit
// alone).  Wavefront w takes the column pairs w, w + WAVES, ..., two pairs at a time; every column of
// the tile is transformed, present in X or not (a tile this narrow is only used on large batches).
template <int NC, int WAVES>
__device__ __forceinline__ void transform_column_pairs_256(float* tile, float scale, uint32_t lane, uint32_t wave)
{
    constexpr uint32_t cstride = 256u + kPad;
    constexpr int PER_WAVE = NC / 2 / WAVES;  // column pairs per wavefront
    static_assert(PER_WAVE >= 2 && PER_WAVE % 2 == 0, "pairs are taken two at a time");
    TileOperands<BF16> ops;
    make_tile_operands<BF16, 4>(8, ops);
    auto column = [&](int j, int h) { return tile + (2u * (wave + (uint32_t)WAVES * j) + h) * cstride + 4u * lane; };
    auto fetch = [&](int j, SplitTileF32& o) __attribute__((always_inline)) {
        float in[8];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const f32x4 q = *reinterpret_cast<const f32x4*>(column(j, h));
#pragma unroll
            for (int r = 0; r < 4; ++r) in[4 * h + r] = q[r];
        }
        split_tile_f32(in, o);
    };
    SplitTileF32 cur[2], nxt[2];
    fetch(0, cur[0]);
    fetch(1, cur[1]);
#pragma unroll
    for (int u = 0; u < PER_WAVE / 2; ++u) {
        if (u + 1 < PER_WAVE / 2) {
            fetch(2 * u + 2, nxt[0]);
            fetch(2 * u + 3, nxt[1]);
        }
        f32x4 a[2][2];
        tile_pair_mfma_f32(cur, ops, a);
#pragma unroll
        for (int c = 0; c < 2; ++c)
#pragma unroll
            for (int h = 0; h < 2; ++h) *reinterpret_cast<f32x4*>(column(2 * u + c, h)) = a[c][h] * scale;
        cur[0] = nxt[0];
        cur[1] = nxt[1];
    }
}

// N = 512, 1024 or 2048
template <int NC, int WAVES>
__device__ __forceinline__ void transform_column_tile(float* tile, uint32_t N, uint32_t B, uint32_t b0, float scale,
                                                      uint32_t lane, uint32_t wave)
{
    if (N == 512u)
        transform_column_tile_as<1, NC, WAVES>(tile, N, B, b0, scale, lane, wave);
    else if (N == 1024u)
        transform_column_tile_as<2, NC, WAVES>(tile, N, B, b0, scale, lane, wave);
    else
        transform_column_tile_as<4, NC, WAVES>(tile, N, B, b0, scale, lane, wave);
}

// How the tiles of Y are spread: a workgroup keeps its transformed tile for several row blocks once
// there are more row blocks than it takes to give every compute unit as many workgroups as fit its
// LDS (two are counted on where they fit).
struct GemvPlan {
    uint32_t col_groups, rows_per_group, row_groups;
    uint32_t workgroups() const { return col_groups * row_groups; }
};
inline GemvPlan plan_gemv(uint32_t M, uint32_t B, uint32_t nc, uint32_t block_rows, size_t lds)
{
    GemvPlan p;
    p.col_groups = (B + nc - 1u) / nc;
    const uint32_t row_blocks = (M + block_rows - 1u) / block_rows;
    uint32_t groups_y = ((lds <= 80u * 1024u ? 512u : 256u) + p.col_groups - 1u) / p.col_groups;
    if (groups_y > row_blocks) groups_y = row_blocks;
    p.rows_per_group = ((row_blocks + groups_y - 1u) / groups_y) * block_rows;
    p.row_groups = (M + p.rows_per_group - 1u) / p.rows_per_group;
    return p;
}

// The same for a kernel of which a compute unit holds one workgroup (fused_gemv_stream.hip): the
// launch runs in rounds of 256 workgroups, each costing one prologue plus a time per 64-row block
// (measured about 12 us and 9 us: 4 : 3), so the number of row groups is the one that minimises
// rounds x (prologue + row blocks per group).  33 column groups over 32 row blocks: seven row groups
// of five blocks (231 workgroups, one round) instead of eight of four (264: a second round for eight
// workgroups, 104 us instead of 60 for M = N = 2048, B = 528).
inline GemvPlan plan_gemv_rounds(uint32_t M, uint32_t B, uint32_t nc, uint32_t block_rows)
{
    GemvPlan p;
    p.col_groups = (B + nc - 1u) / nc;
    const uint32_t row_blocks = (M + block_rows - 1u) / block_rows;
    uint64_t best = ~0ull;
    uint32_t best_per_group = row_blocks;
    for (uint32_t per_group = 1; per_group <= row_blocks; ++per_group) {
        const uint64_t groups = (row_blocks + per_group - 1u) / per_group;
        const uint64_t rounds = (groups * p.col_groups + 255u) / 256u;
        const uint64_t cost = rounds * (4u + 3ull * per_group);
        if (cost < best) {
            best = cost;
            best_per_group = per_group;
        }
        if (rounds == 1u) break;  // longer groups only cost more from here on
    }
    p.rows_per_group = best_per_group * block_rows;
    p.row_groups = (M + p.rows_per_group - 1u) / p.rows_per_group;
    return p;
}

// N = 2048 with W streamed through LDS and each wavefront's quarter of the transformed columns in its
// registers (fused_gemv_stream.hip); same contract as the kernels of fused_gemv.hip.
// `columns_contiguous`: X is given as Xt[B][N] (the layout of mi_fused_ht_gemm) instead of X[N][B].
int launch_stream_2048(const float* W, const float* X, float* Y, uint32_t M, uint32_t B, float scale,
                       bool columns_contiguous, hipStream_t s);

// N = 256, 512 and 1024 with the whole B operand in every wavefront's registers, the wavefronts
// splitting the rows (fused_gemv_rows.hip: 64 columns per workgroup for N = 256, 16 otherwise); same
// contract.
int launch_rows(const float* W, const float* X, float* Y, uint32_t M, uint32_t N, uint32_t B, float scale,
                bool columns_contiguous, hipStream_t s);

// The GEMV kernel for a shape (fused_gemv.hip), arguments already validated; `columns_contiguous` as
// above (supported for N < 512 and for the shapes the two kernels above take).
int launch_any(const float* W, const float* X, float* Y, uint32_t M, uint32_t N, uint32_t B, float scale,
               bool columns_contiguous, hipStream_t s);

}  // namespace gemv
}  // namespace mi
