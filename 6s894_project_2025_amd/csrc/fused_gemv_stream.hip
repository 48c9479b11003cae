// Fused Hadamard + GEMV-batch for the shapes that fill the chip, fp32, gfx950:
//     Y[M,B] = W[M,N] * (scale * H_N * X[N,B]),  N = 2048 (16 columns per workgroup).
//
// The kernel of fused_gemv.hip keeps the transformed columns in LDS and takes W straight from global
// memory into registers, a 16-byte piece per lane: a load instruction then touches 16 rows of W and 64
// bytes of each, and the compute unit's vector cache, which handles one 128-byte line per request
// however little of it is asked for, passes 16 - 17 bytes per clock where the fp32 matrix cores of a
// 16-column workgroup consume 32.  Here the two operands change places:
//   * after the same prologue (gemv_common.hpp: the column tile staged into LDS and transformed
//     there) every wavefront copies the B fragments of its quarter of the K range into registers
//     (16 columns x N / 4 values = N / 16 registers per lane), which frees all of the LDS;
//   * W is then streamed through the LDS by direct global -> LDS transfers that ask for whole
//     128-byte lines (a transfer covers 8 rows x 128 bytes), each wavefront through a ring of its own
//     (four stages of 64 rows x 128 bytes, three stages requested ahead), and read back as A
//     fragments; the wavefronts never wait for each other inside a row block;
//   * the four partial sums of a row block meet in LDS as in fused_gemv.hip.
//
// Behaviour replaced: fused_hadamard_gemv_kernel(_vec), fused_ht/fwht_gemv_fusion.cu:98-244, on the
// large shapes of its benchmark list (:643-653).
#include "gemv_common.hpp"
#include "lds_layout.hpp"
#include "xreg_common.hpp"

namespace mi {
namespace {

using gemv::kPad;
using gemv::kXcds;
using gemv::lds_barrier;

constexpr int kWaves = 4;
constexpr uint32_t kBlockRows = 64;                             // rows of W per row block
constexpr uint32_t kLineBytes = 128;                            // two K steps (2 x 16 floats) of a row
constexpr uint32_t kStageBytes = kBlockRows * kLineBytes;       // 8 KB
constexpr int kSlots = 4;                                       // stages in a wavefront's ring
constexpr int kAhead = 3;                                       // stages requested ahead of the MFMAs
constexpr int kPieces = kStageBytes / 1024;                     // transfers (64 lanes x 16 bytes) per stage
constexpr uint32_t kRingBytes = kWaves * kSlots * kStageBytes;  // 128 KB

// LDS image of a stage: [64 rows][128 bytes], the 16-byte chunk q of row r stored at q ^ (r & 7).
// A transfer puts lane l's bytes at 16 l of its kilobyte, so lane l asks for row l / 8 of the
// transfer's eight rows and chunk (l % 8) ^ (l / 8); a fragment read (lane (hi, lo): row 16 mb + lo,
// chunk 4 half + hi) then finds eight different 16-byte columns under eight adjacent lanes.
__host__ __device__ constexpr uint32_t stage_chunk_offset(uint32_t row, uint32_t q)
{
    return row * kLineBytes + ((q ^ (row & 7u)) << 4);
}
constexpr bool stage_patterns_ok()
{
    for (uint32_t i = 0; i < (uint32_t)kPieces; ++i)  // the transfers fill every slot of the stage exactly once
        for (uint32_t l = 0; l < 64; ++l)
            if (stage_chunk_offset(8u * i + l / 8u, (l % 8u) ^ (l / 8u)) != 1024u * i + 16u * l) return false;
    for (uint32_t mb = 0; mb < 4; ++mb)
        for (uint32_t half = 0; half < 2; ++half)
            if (!lds::conflict_free_b128(
                    [=](uint32_t lane) { return stage_chunk_offset(16u * mb + (lane & 15u), 4u * half + (lane >> 4)); }))
                return false;
    return true;
}
static_assert(stage_patterns_ok(), "the W stage layout does not match its transfers or its reads would serialise");

template <int N, int NC>
struct StreamGeom {
    static_assert(N % 512 == 0 && NC % 16 == 0, "whole tiles, whole fragments");
    static constexpr int NF = NC / 16;                    // 16-column fragments
    static constexpr int STEPS = N / 16 / kWaves;         // K steps (of 16) per wavefront and row block
    static constexpr int STAGES = STEPS / 2;              // a stage is two K steps: one 128-byte line per row
    static constexpr int G = 4 * NF;                      // accumulator fragments per wavefront
    static constexpr uint32_t kTileBytes = (uint32_t)NC * (N + kPad) * 4u;
    static constexpr uint32_t kRedBytes = (kWaves - 1) * G * 64u * 16u;
    static constexpr uint32_t kLdsBytes = kRingBytes + kRedBytes;
    static_assert(STAGES % kSlots == 0, "stage g of every row block lives in ring slot g % 4");
    static_assert(kTileBytes <= kLdsBytes && kLdsBytes <= 160u * 1024u, "the tile and later the ring fit the LDS");
    static_assert(STEPS * NF * 4 <= 256, "the B fragments of a wavefront fit its registers");
};

// XT: X is given column by column (Xt[B][N]).
template <int N, int NC, bool XT>
__global__ void __launch_bounds__(64 * kWaves)
fused_ht_gemv_stream_kernel(const float* __restrict__ W, const float* __restrict__ X, float* __restrict__ Y,
                            uint32_t M, uint32_t B, float scale, uint32_t rows_per_group, uint32_t col_groups,
                            uint32_t row_groups, uint32_t per_xcd, bool col_major)
{
    using Geo = StreamGeom<N, NC>;
    constexpr int NF = Geo::NF, STEPS = Geo::STEPS, STAGES = Geo::STAGES, G = Geo::G;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    float* const tile = reinterpret_cast<float*>(lds);
    // placement as in fused_gemv.hip: (XCD, slot) takes place XCD * per_xcd + slot of an order of the
    // tiles in which neighbours share a slice of W or, col_major, a column tile
    const uint32_t place = (blockIdx.x % kXcds) * per_xcd + blockIdx.x / kXcds;
    if (place >= col_groups * row_groups) return;  // workgroup-uniform, before any barrier
    const uint32_t b0 = (col_major ? place / row_groups : place % col_groups) * NC;
    const uint32_t lane = threadIdx.x & 63u, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t lo = lane & 15u, hi = lane >> 4;
    const uint32_t m_first = (col_major ? place % row_groups : place / col_groups) * rows_per_group;
    const uint32_t m_last = min(M, m_first + rows_per_group);

    // ---- prologue: TT = scale * H_N * X[:, b0 .. b0 + NC - 1] in LDS ------------------------------
    // (all N rows of the tile requested before the first is waited for: 128 registers per lane that
    // nothing else needs yet)
    if constexpr (XT)
        gemv::stage_column_tile_xt<NC, kWaves, N>(X, tile, B, b0, threadIdx.x);
    else
        gemv::stage_column_tile<NC, kWaves, N / (16 * kWaves / (NC / 16))>(X, tile, N, B, b0, lane, wave,
                                                                          gemv::first_row_of(blockIdx.x));
    lds_barrier();
    gemv::transform_column_tile<NC, kWaves>(tile, N, B, b0, scale, lane, wave);
    lds_barrier();
    // The wavefront's i-th K step is step (i / 2) * 8 + 2 * wave + i % 2 of the row: steps 2p and
    // 2p + 1 are the two halves of the wavefront's 128-byte line in the p-th 512 bytes of every row.
    // Lane (hi, lo) holds k = 16 step + 4 hi + s of column 16 f + lo for the MFMA with index s.
    float bf[STEPS][NF][4];
    {
        constexpr uint32_t cstride4 = (N + kPad) / 4u;
        const f32x4* const tile4 = reinterpret_cast<const f32x4*>(tile);
#pragma unroll
        for (int i = 0; i < STEPS; ++i)
#pragma unroll
            for (int f = 0; f < NF; ++f) {
                const f32x4 q = tile4[(16u * f + lo) * cstride4 + 4u * ((uint32_t)(i >> 1) * 8u + 2u * wave + (i & 1)) + hi];
#pragma unroll
                for (int e = 0; e < 4; ++e) bf[i][f][e] = q[e];
            }
    }
    lds_barrier();  // every wavefront has its fragments: the LDS now belongs to the W stream

    // ---- W stream -----------------------------------------------------------------------------------
    const uint32_t ring = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(xreg::lptr_t)lds) +
                          wave * (uint32_t)(kSlots * kStageBytes);
    const unsigned char* const ring_ptr = lds + wave * (uint32_t)(kSlots * kStageBytes);
    f32x4* const red = reinterpret_cast<f32x4*>(lds + kRingBytes);
    const uint32_t trow = lane >> 3, tq = (lane & 7u) ^ trow;
    uint32_t voff[kPieces];  // lane part of a transfer's address inside the row block being requested
    auto aim = [&](uint32_t mb) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < kPieces; ++i)
            voff[i] = (min(mb + 8u * i + trow, M - 1u) - mb) * (uint32_t)(N * 4) + (tq << 4);
    };
    // the wavefront's line in the first 512 bytes of a row block's first row (derived from the block's
    // first row every time, not carried around the row-block loop as a pointer: the transfer takes its
    // base from scalar registers, which the compiler grants a value it can see to be uniform)
    auto line_of = [&](uint32_t mb) __attribute__((always_inline)) {
        return reinterpret_cast<const unsigned char*>(W) + (uint64_t)mb * (N * 4) + wave * kLineBytes;
    };
    auto request = [&](const unsigned char* line, int stage, int piece) __attribute__((always_inline)) {
        xreg::global_to_lds16(voff[piece], line + stage * 512, ring, (stage % kSlots) * (int)kStageBytes + piece * 1024);
    };
    // lane part of a fragment read, by half of the line
    uint32_t frag_at[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) frag_at[h] = stage_chunk_offset(lo, 4u * h + hi);
    f32x4 fr[2][4];
    auto read_frags = [&](int step, f32x4 (&o)[4]) __attribute__((always_inline)) {
#pragma unroll
        for (int mb = 0; mb < 4; ++mb)
            o[mb] = *reinterpret_cast<const f32x4*>(ring_ptr + frag_at[step & 1] +
                                                    ((step >> 1) % kSlots) * kStageBytes + mb * 16u * kLineBytes);
    };

    aim(m_first);
#pragma unroll
    for (int g = 0; g < kAhead; ++g)
#pragma unroll
        for (int i = 0; i < kPieces; ++i) request(line_of(m_first), g, i);
    // Transfers complete in order among themselves, but not relative to stores, so every count
    // below is the number of *transfers* requested after the stage that is needed: pending stores
    // of Y can only make a wait longer.
    xreg::wait_vm(kPieces * (kAhead - 1));
    read_frags(0, fr[0]);

    // One row block.  LAST: no row block follows, the stream ends with this block's last stage.
    auto row_block = [&](auto last_tag, uint32_t mb) __attribute__((always_inline)) {
        constexpr bool LAST = decltype(last_tag)::value;
        const unsigned char* const line = line_of(mb);
        const unsigned char* const next_line = line_of(mb + kBlockRows);
        f32x4 acc[G];
#pragma unroll
        for (int g = 0; g < G; ++g) acc[g] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int t = 0; t < STEPS; ++t) {
            const int stage = t >> 1;
            // the fragments of the next step (of the next block's first step), a step ahead
            if (t + 1 < STEPS || !LAST) {
                if (t & 1) {
                    // stage + 1 must have landed; requested after it: stages + 2, + 3 where they exist
                    const int later = LAST ? (STAGES - 2 - stage < kAhead - 1 ? STAGES - 2 - stage : kAhead - 1) : kAhead - 1;
                    xreg::wait_vm(kPieces * (later > 0 ? later : 0));
                }
                read_frags((t + 1) % STEPS, fr[(t + 1) & 1]);
            }
            __builtin_amdgcn_sched_barrier(0);
            // from its third-last stage on a block requests the next block's first stages
            const int ask = stage + kAhead;
            if (!(t & 1) && ask == STAGES && !LAST) aim(mb + kBlockRows);
#pragma unroll
            for (int s = 0; s < 4; ++s) {
#pragma unroll
                for (int mi = 0; mi < 4; ++mi)
#pragma unroll
                    for (int f = 0; f < NF; ++f)
                        acc[mi * NF + f] = __builtin_amdgcn_mfma_f32_16x16x4f32(fr[t & 1][mi][s], bf[t][f][s],
                                                                                acc[mi * NF + f], 0, 0, 0);
                // the stage's eight transfers behind the MFMAs of its first step, two per group
                if (!(t & 1) && (ask < STAGES || !LAST)) {
                    request(ask < STAGES ? line : next_line, ask % STAGES, 2 * s);
                    request(ask < STAGES ? line : next_line, ask % STAGES, 2 * s + 1);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        // ---- meet the wavefronts' K shares in LDS: fragment g is finished by wavefront g % 4, which
        // keeps its own part in registers; the sum is taken in the order of the wavefronts ---------
        lds_barrier();  // the sums of the row block before have been read
#pragma unroll
        for (int g = 0; g < G; ++g) {
            const uint32_t owner = (uint32_t)(g % kWaves);
            if (wave != owner) red[((uint32_t)g * (kWaves - 1) + (wave < owner ? wave : wave - 1u)) * 64u + lane] = acc[g];
        }
        lds_barrier();
#pragma unroll
        for (int g = 0; g < G; ++g) {
            const int owner = g % kWaves;
            if (wave != (uint32_t)owner) continue;
            f32x4 sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int w = 0; w < kWaves; ++w) {
                const f32x4 part = w == owner ? acc[g] : red[(g * (kWaves - 1) + (w < owner ? w : w - 1)) * 64 + lane];
                sum = w == 0 ? part : sum + part;
            }
            // D[m'][n']: n' = lo is the column, m' = 4 hi + r the row inside the 16-row fragment
            const uint32_t col = b0 + 16u * (uint32_t)(g % NF) + lo;
            if (col < B) {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const uint32_t m = mb + 16u * (uint32_t)(g / NF) + 4u * hi + r;
                    if (m < M) Y[(uint64_t)m * B + col] = sum[r];
                }
            }
        }
    };
#pragma unroll 1
    for (uint32_t mb = m_first; mb < m_last; mb += kBlockRows) {
        if (mb + kBlockRows < m_last)
            row_block(std::false_type{}, mb);
        else
            row_block(std::true_type{}, mb);
    }
}

}  // namespace

namespace gemv {

namespace {

template <int N, int NC, bool XT>
int launch_stream_as(const float* W, const float* X, float* Y, uint32_t M, uint32_t B, float scale, hipStream_t s)
{
    using Geo = StreamGeom<N, NC>;
    // the tile transform's two MFMA stages attenuate by a power of two that the scale takes back
    scale = (float)((double)scale * (double)(1u << tile_stage_shift<4>(9u, false)));
    auto kern = fused_ht_gemv_stream_kernel<N, NC, XT>;
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)Geo::kLdsBytes) != hipSuccess)
        return MI_ERR_LAUNCH;
    const GemvPlan p = plan_gemv_rounds(M, B, NC, kBlockRows);
    const uint32_t per_xcd = (p.workgroups() + kXcds - 1) / kXcds;
    // bytes of X an XCD needs under the row-group-major order: its column groups' tiles
    const uint64_t x_per_xcd = (uint64_t)(p.col_groups < per_xcd ? p.col_groups : per_xcd) * NC * N * sizeof(float);
    const bool col_major = x_per_xcd > (2ull << 20);
    hipLaunchKernelGGL(kern, dim3(per_xcd * kXcds), dim3(64 * kWaves), Geo::kLdsBytes, s, W, X, Y, M, B, scale,
                       p.rows_per_group, p.col_groups, p.row_groups, per_xcd, col_major);
    return launch_status();
}

}  // namespace

// Launched by mi_fused_ht_gemv (fused_gemv.hip) for N = 2048 on the shapes that give every compute
// unit a 64-row workgroup.
int launch_stream_2048(const float* W, const float* X, float* Y, uint32_t M, uint32_t B, float scale,
                       bool columns_contiguous, hipStream_t s)
{
    return columns_contiguous ? launch_stream_as<2048, 16, true>(W, X, Y, M, B, scale, s)
                              : launch_stream_as<2048, 16, false>(W, X, Y, M, B, scale, s);
}

}  // namespace gemv
}  // namespace mi
