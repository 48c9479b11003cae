// Fused Hadamard + GEMV-batch for N = 512 and 1024 on the shapes that fill the chip, fp32, gfx950:
//     Y[M,B] = W[M,N] * (scale * H_N * X[N,B]),  16 columns per workgroup.
//
// All N values of 16 transformed columns are 4 N bytes per lane, at most the 256 registers of a
// wavefront's accumulation file, so here every wavefront keeps the whole B operand and the four
// wavefronts of a workgroup split the *rows* of a 64-row block instead of the K range:
//   * no partial sums, no barrier and no LDS traffic between the wavefronts after the prologue;
//   * a workgroup transforms 16 columns, not 32 (half the prologue of the K-split kernel of
//     fused_gemv_stream.hip for the same number of workgroups);
//   * W is streamed through LDS as there, by direct global -> LDS transfers of whole lines: a
//     wavefront's stage is its 16 rows x 512 bytes (eight K steps), a transfer covers 2 rows x 512
//     bytes, the ring has four stages with three requested ahead, and the first two stages are
//     requested before the prologue, into the part of the LDS that the column tile leaves free.
// The matrix cores see 16 columns per workgroup, which asks 32 bytes per clock of the W stream;
// whole-line transfers deliver that (the 16-byte loads of fused_gemv.hip: 16 - 17).
//
// Behaviour replaced: fused_hadamard_gemv_kernel(_vec), fused_ht/fwht_gemv_fusion.cu:98-244.
#include "gemv_common.hpp"
#include "lds_layout.hpp"
#include "xreg_common.hpp"

namespace mi {
namespace {

using gemv::kPad;
using gemv::kXcds;
using gemv::lds_barrier;

constexpr int kWaves = 4;
constexpr uint32_t kBlockRows = 64;  // rows of W per row block: 16 per wavefront
constexpr int kSlots = 4;            // stages in a wavefront's ring
constexpr int kAhead = 3;            // stages requested ahead of the MFMAs

// A wavefront's stage: its 16 rows x SS K steps (64 SS bytes of each row: 512 for N >= 512, 256 for
// N = 256, so that a row block is a multiple of four stages).
// LDS image: [16 rows][64 SS bytes], the 16-byte chunk q of row r stored at q ^ (r & 7).  A transfer
// puts lane l's bytes at 16 l of its kilobyte, so lane l asks for row l / (4 SS) of the transfer's
// rows and chunk (l % (4 SS)) ^ (row & 7): whole 128-byte lines of W.  A fragment read (lane (hi, lo):
// row lo, chunk 4 ks + hi) then finds eight different 16-byte columns under eight adjacent lanes.
template <int SS>
struct Stage {
    static constexpr uint32_t kRowBytes = 64u * SS;
    static constexpr uint32_t kBytes = 16u * kRowBytes;
    static constexpr int kPieces = kBytes / 1024;            // transfers (64 lanes x 16 bytes) per stage
    static constexpr uint32_t kRowsPerPiece = 1024u / kRowBytes;
    static constexpr uint32_t kSlotBytes = kWaves * kBytes;  // ring slot s of wavefront w: s * kSlotBytes + w * kBytes
    static constexpr uint32_t kRingBytes = kSlots * kSlotBytes;
    static constexpr uint32_t kTileBase = 2 * kSlotBytes;    // the column tile lives on top of slots 2 and 3
    static_assert(kPieces <= SS, "one transfer of the stage three ahead per K step");
    static __host__ __device__ constexpr uint32_t chunk_offset(uint32_t row, uint32_t q)
    {
        return row * kRowBytes + ((q ^ (row & 7u)) << 4);
    }
    static constexpr bool patterns_ok()
    {
        for (uint32_t i = 0; i < (uint32_t)kPieces; ++i)  // the transfers fill every slot of the stage exactly once
            for (uint32_t l = 0; l < 64; ++l) {
                const uint32_t row = kRowsPerPiece * i + l / (4u * SS);
                if (chunk_offset(row, (l % (4u * SS)) ^ (row & 7u)) != 1024u * i + 16u * l) return false;
            }
        for (uint32_t ks = 0; ks < (uint32_t)SS; ++ks)
            if (!lds::conflict_free_b128([=](uint32_t lane) { return chunk_offset(lane & 15u, 4u * ks + (lane >> 4)); }))
                return false;
        return true;
    }
};
static_assert(Stage<8>::patterns_ok() && Stage<4>::patterns_ok(),
              "the W stage layout does not match its transfers or its reads would serialise");

// acc (+)= A(16 x 4) * B(4 x 16) with B straight from the accumulation-register file.  Opaque
// statements: the compiler would otherwise copy every B value into an ordinary register right before
// its MFMA (N = 1024: a hundred copies per row block, none of them hidden behind the MFMAs: 9 570
// cycles per block instead of 8 650).  It then knows nothing of the instruction's timing: whoever
// reads `c` with anything but the next MFMA waits out the pipeline first (xreg::mfma_delay), and the
// build checks the generated ISA (build.py, ISA_CHECKED).
__device__ __forceinline__ void xmfma_first(f32x4& c, float a, float b)
{
    asm volatile("v_mfma_f32_16x16x4_f32 %0, %1, %2, 0" : "=v"(c) : "v"(a), "a"(b));
}
__device__ __forceinline__ void xmfma_next(f32x4& c, float a, float b)
{
    asm volatile("v_mfma_f32_16x16x4_f32 %0, %1, %2, %0" : "+v"(c) : "v"(a), "a"(b));
}

template <int N, int NC>
struct RowsGeom {
    static_assert(N % 256 == 0 && NC % 16 == 0, "whole half tiles, whole fragments");
    static constexpr int SS = N >= 512 ? 8 : 4;           // K steps per stage
    using St = Stage<SS>;
    static constexpr int NF = NC / 16;                    // 16-column fragments
    static constexpr int STEPS = N / 16;                  // K steps (of 16) per row block
    static constexpr int STAGES = STEPS / SS;
    static constexpr uint32_t kTileBytes = (uint32_t)NC * (N + kPad) * 4u;
    static constexpr uint32_t kLdsBytes = St::kTileBase + kTileBytes > St::kRingBytes ? St::kTileBase + kTileBytes : St::kRingBytes;
    static_assert(STAGES % kSlots == 0, "stage g of every row block lives in ring slot g % 4");
    static_assert(kLdsBytes <= 160u * 1024u, "the tile on top of the last two ring slots fits the LDS");
    static_assert(STEPS * NF * 4 <= 256, "the B operand of a wavefront fits its registers");
};

// XT: X is given column by column (Xt[B][N]).
template <int N, int NC, bool XT>
__global__ void __launch_bounds__(64 * kWaves)
fused_ht_gemv_rows_kernel(const float* __restrict__ W, const float* __restrict__ X, float* __restrict__ Y,
                          uint32_t M, uint32_t B, float scale, uint32_t rows_per_group, uint32_t col_groups,
                          uint32_t row_groups, uint32_t per_xcd, bool col_major)
{
    using Geo = RowsGeom<N, NC>;
    using St = typename Geo::St;
    constexpr int NF = Geo::NF, STEPS = Geo::STEPS, STAGES = Geo::STAGES, kStageSteps = Geo::SS, kPieces = St::kPieces;
    constexpr uint32_t kStageBytes = St::kBytes, kSlotBytes = St::kSlotBytes, kStageRowBytes = St::kRowBytes;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    float* const tile = reinterpret_cast<float*>(lds + St::kTileBase);
    // placement as in fused_gemv.hip: (XCD, slot) takes place XCD * per_xcd + slot of an order of the
    // tiles in which neighbours share a slice of W or, col_major, a column tile
    const uint32_t place = (blockIdx.x % kXcds) * per_xcd + blockIdx.x / kXcds;
    if (place >= col_groups * row_groups) return;  // workgroup-uniform, before any barrier
    const uint32_t b0 = (col_major ? place / row_groups : place % col_groups) * NC;
    const uint32_t lane = threadIdx.x & 63u, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t lo = lane & 15u, hi = lane >> 4;
    const uint32_t m_first = (col_major ? place % row_groups : place / col_groups) * rows_per_group;
    const uint32_t m_last = min(M, m_first + rows_per_group);

    // ---- W stream -----------------------------------------------------------------------------------
    const uint32_t ring = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(xreg::lptr_t)lds) + wave * kStageBytes;
    const unsigned char* const ring_ptr = lds + wave * kStageBytes;
    constexpr uint32_t kLanesPerRow = 4u * kStageSteps;  // 16-byte chunks of a row in a stage
    const uint32_t trow = lane / kLanesPerRow;
    uint32_t voff[kPieces];  // lane part of a transfer's address inside the row block being requested
    auto aim = [&](uint32_t mb) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < kPieces; ++i) {
            const uint32_t row = St::kRowsPerPiece * i + trow;  // of the wavefront's 16
            voff[i] = (min(mb + 16u * wave + row, M - 1u) - mb) * (uint32_t)(N * 4) +
                      (((lane % kLanesPerRow) ^ (row & 7u)) << 4);
        }
    };
    // the first 512 bytes of a row block's first row (derived from the block's first row every time,
    // not carried around the row-block loop as a pointer: the transfer takes its base from scalar
    // registers, which the compiler grants a value it can see to be uniform)
    auto block_of = [&](uint32_t mb) __attribute__((always_inline)) {
        return reinterpret_cast<const unsigned char*>(W) + (uint64_t)mb * (N * 4);
    };
    auto request = [&](const unsigned char* block, int stage, int piece) __attribute__((always_inline)) {
        xreg::global_to_lds16(voff[piece], block + stage * (int)kStageRowBytes, ring,
                              (stage % kSlots) * (int)kSlotBytes + piece * 1024);
    };
    // the first two stages do not depend on the transform, and their ring slots lie below the tile
    aim(m_first);
#pragma unroll
    for (int g = 0; g < 2; ++g)
#pragma unroll
        for (int i = 0; i < kPieces; ++i) request(block_of(m_first), g, i);

    // ---- prologue: TT = scale * H_N * X[:, b0 .. b0 + NC - 1] in LDS ------------------------------
    // (all N rows of the tile requested before the first is waited for)
    if constexpr (XT)
        gemv::stage_column_tile_xt<NC, kWaves, N>(X, tile, B, b0, threadIdx.x);
    else
        gemv::stage_column_tile<NC, kWaves, N / (16 * kWaves / (NC / 16))>(X, tile, N, B, b0, lane, wave,
                                                                          gemv::first_row_of(blockIdx.x));
    lds_barrier();
    if constexpr (N == 256)
        gemv::transform_column_pairs_256<NC, kWaves>(tile, scale, lane, wave);
    else
        gemv::transform_column_tile<NC, kWaves>(tile, N, B, b0, scale, lane, wave);
    lds_barrier();
    // Lane (hi, lo) holds k = 16 step + 4 hi + s of column 16 f + lo for the MFMA with index s.
    float bf[STEPS][NF][4];
    {
        constexpr uint32_t cstride4 = (N + kPad) / 4u;
        const f32x4* const tile4 = reinterpret_cast<const f32x4*>(tile);
#pragma unroll
        for (int i = 0; i < STEPS; ++i)
#pragma unroll
            for (int f = 0; f < NF; ++f) {
                const f32x4 q = tile4[(16u * f + lo) * cstride4 + 4u * i + hi];
#pragma unroll
                for (int e = 0; e < 4; ++e) bf[i][f][e] = q[e];
            }
    }
    lds_barrier();  // every wavefront has the B operand: the rest of the LDS now belongs to the W stream
#pragma unroll
    for (int i = 0; i < kPieces; ++i) request(block_of(m_first), 2, i);

    // lane part of a fragment read, by parity of the K step inside its stage
    uint32_t frag_at[2];
#pragma unroll
    for (int p = 0; p < 2; ++p) frag_at[p] = St::chunk_offset(lo, 4u * p + hi);
    auto read_frag = [&](int step) __attribute__((always_inline)) {
        const int ks = step % kStageSteps, stage = step / kStageSteps;
        return *reinterpret_cast<const f32x4*>(ring_ptr + frag_at[ks & 1] + (stage % kSlots) * kSlotBytes + (ks >> 1) * 128u);
    };
    // Transfers complete in order among themselves, but not relative to stores, so every count
    // below is the number of *transfers* requested after the stage that is needed: pending stores
    // of Y can only make a wait longer.
    xreg::wait_vm(kPieces * (kAhead - 1));
    // fragments are read kFragAhead K steps before their MFMAs (a step is four MFMAs, 128 cycles: one
    // step ahead left the loop waiting for LDS, 0.78 of the matrix cores' rate)
    // (a ring of eight: the entry a read overwrites was last an MFMA operand five steps ago, and the
    // ring index runs on over the edge between two row blocks)
    constexpr int kFragAhead = 3, kFragRing = 8;
    static_assert(STEPS % kFragRing == 0 && kFragRing > kFragAhead + 1, "step t of every block uses ring entry t % 8");
    f32x4 fr[kFragRing];
#pragma unroll
    for (int t = 0; t < kFragAhead; ++t) fr[t] = read_frag(t);

    // a lane's place in a row block of Y: row 16 wave + 4 hi (+ r), column lo (+ 16 f); 32-bit while
    // 64 rows of Y stay below 4 GB
    const bool cols_full = b0 + NC <= B && B < (1u << 24);
    const uint32_t y_lane = ((16u * wave + 4u * hi) * B + lo) * 4u;

    // One row block.  LAST: no row block follows, the stream ends with this block's last stage.
    auto row_block = [&](auto last_tag, uint32_t mb) __attribute__((always_inline)) {
        constexpr bool LAST = decltype(last_tag)::value;
        const unsigned char* const block = block_of(mb);
        const unsigned char* const next_block = block_of(mb + kBlockRows);
        // two accumulators per fragment take turns, so that no MFMA waits for the one before it
        f32x4 acc[NF][2];
#pragma unroll
        for (int t = 0; t < STEPS; ++t) {
            const int stage = t / kStageSteps, ks = t % kStageSteps;
            // the fragment of step t + kFragAhead (of the next block's first steps)
            if (t + kFragAhead < STEPS || !LAST) {
                const int ahead = (t + kFragAhead) % STEPS;
                if (ahead % kStageSteps == 0) {
                    // its stage (this step's stage + 1) must have landed; requested after it: stage
                    // + 2 and, so far, ks transfers of stage + 3, where those stages exist
                    const int left = STAGES - 1 - (stage + 1);  // stages of this block after stage + 1
                    const int after = LAST ? (left >= 2 ? kPieces + ks : (left > 0 ? left : 0) * kPieces) : kPieces + ks;
                    xreg::wait_vm(after);
                }
                fr[(t + kFragAhead) % kFragRing] = read_frag(ahead);
            }
            __builtin_amdgcn_sched_barrier(0);
            // one transfer of stage + 3 per step; from its third-last stage on a block requests the
            // next block's first stages
            const int ask = stage + kAhead;
            if (ks == 0 && ask == STAGES && !LAST) aim(mb + kBlockRows);
#pragma unroll
            for (int s = 0; s < 4; ++s)
#pragma unroll
                for (int f = 0; f < NF; ++f)
                    if (t == 0 && s < 2)
                        xmfma_first(acc[f][s & 1], fr[t % kFragRing][s], bf[t][f][s]);
                    else
                        xmfma_next(acc[f][s & 1], fr[t % kFragRing][s], bf[t][f][s]);
            if (ks < kPieces && (ask < STAGES || !LAST)) request(ask < STAGES ? block : next_block, ask % STAGES, ks);
            __builtin_amdgcn_sched_barrier(0);
        }
        // D[m'][n']: n' = lo is the column, m' = 4 hi + r the row inside the wavefront's 16
        xreg::mfma_delay();
#pragma unroll
        for (int f = 0; f < NF; ++f) asm volatile("" : "+v"(acc[f][0]), "+v"(acc[f][1]));
        if (mb + kBlockRows <= M && cols_full) {
            // a whole block inside Y: scalar base + the lane's fixed offset, no masks.  (Summing a
            // block's results into spare registers and storing them behind the first MFMAs of the
            // next block measured slower, 8 860 cycles per block instead of 8 800: the wait for the
            // matrix cores stays, and the stores cost the MFMA stream what they cost here.)
            unsigned char* const yb = reinterpret_cast<unsigned char*>(Y) + ((uint64_t)mb * B + b0) * 4u;
#pragma unroll
            for (int f = 0; f < NF; ++f)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float v = acc[f][0][r] + acc[f][1][r];
                    xreg::cached_store4(y_lane, __float_as_uint(v), yb + ((uint64_t)r * B + 16u * f) * 4u);
                }
        } else {
#pragma unroll
            for (int f = 0; f < NF; ++f) {
                const uint32_t col = b0 + 16u * (uint32_t)f + lo;
                if (col < B) {
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const uint32_t m = mb + 16u * wave + 4u * hi + r;
                        if (m < M) Y[(uint64_t)m * B + col] = acc[f][0][r] + acc[f][1][r];
                    }
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

template <int N, int NC, bool XT>
int launch_rows_as(const float* W, const float* X, float* Y, uint32_t M, uint32_t B, float scale, hipStream_t s)
{
    using Geo = RowsGeom<N, NC>;
    // the tile transform's two MFMA stages attenuate by a power of two that the scale takes back
    scale = (float)((double)scale * (double)(1u << tile_stage_shift<4>(N >= 512 ? 9u : 8u, false)));
    auto kern = fused_ht_gemv_rows_kernel<N, NC, XT>;
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)Geo::kLdsBytes) != hipSuccess)
        return MI_ERR_LAUNCH;
    const gemv::GemvPlan p = gemv::plan_gemv_rounds(M, B, NC, kBlockRows);
    const uint32_t per_xcd = (p.workgroups() + kXcds - 1) / kXcds;
    // bytes of X an XCD needs under the row-group-major order: its column groups' tiles
    const uint64_t x_per_xcd = (uint64_t)(p.col_groups < per_xcd ? p.col_groups : per_xcd) * NC * N * sizeof(float);
    const bool col_major = x_per_xcd > (2ull << 20);
    hipLaunchKernelGGL(kern, dim3(per_xcd * kXcds), dim3(64 * kWaves), Geo::kLdsBytes, s, W, X, Y, M, B, scale,
                       p.rows_per_group, p.col_groups, p.row_groups, per_xcd, col_major);
    return launch_status();
}

}  // namespace

namespace gemv {

int launch_rows(const float* W, const float* X, float* Y, uint32_t M, uint32_t N, uint32_t B, float scale,
                bool columns_contiguous, hipStream_t s)
{
    if (N == 1024u)
        return columns_contiguous ? launch_rows_as<1024, 16, true>(W, X, Y, M, B, scale, s)
                                  : launch_rows_as<1024, 16, false>(W, X, Y, M, B, scale, s);
    if (N == 512u)
        return columns_contiguous ? launch_rows_as<512, 16, true>(W, X, Y, M, B, scale, s)
                                  : launch_rows_as<512, 16, false>(W, X, Y, M, B, scale, s);
    if (N == 256u)
        return columns_contiguous ? launch_rows_as<256, 64, true>(W, X, Y, M, B, scale, s)
                                  : launch_rows_as<256, 64, false>(W, X, Y, M, B, scale, s);
    return MI_ERR_SIZE;
}

}  // namespace gemv
}  // namespace mi
