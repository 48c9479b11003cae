// Fused Hadamard -> GEMM in fp32 (the reference's precision) with the transformed operand held in
// registers, gfx950:
//     C[M,N] = W[M,K] * (scale * H_K * X[K,N]),  X given as Xt[N,K],  K = 512 ... 4096, fp32 in and out
// (described for K = 1024).
//
// Same structure as the 16-bit kernel of fused_gemm_xreg.hip (one wavefront per SIMD, W streamed
// global -> LDS directly through a ring of four 32 KB stages, fragments broadcast to the four
// wavefronts through LDS, results stored behind the next block's MFMAs); what differs:
//   * a wavefront's 256 accumulation registers hold 16 columns x 1024 k as fp32 (64 columns per
//     workgroup, where the transformed tile in LDS allowed 32);
//   * the prologue is the exact fp32 transform on the bf16 matrix cores (tile_transform_f32:
//     three-piece operands), two tiles per column and one fp32 butterfly between them, passed
//     through the LDS area four columns at a time;
//   * the contraction is v_mfma_f32_16x16x4_f32: a 16-byte fragment per lane carries four
//     consecutive k for four MFMAs (lane (hi, lo) of fragment kk holds k = 16 kk + 4 hi + s), a
//     stage of 64 rows x 512 bytes is 128 k, and sixteen MFMAs of 32 cycles stand behind every four
//     fragment reads: the loop is bound by the fp32 matrix-core rate and by nothing else.
//
// Behaviour replaced: fused_ht_gemm_pipelined (fp32), fused_ht/fusion_pipelined.cu:306-563.
#include <type_traits>

#include "xreg_common.hpp"

namespace mi {
namespace xreg {

// acc (+)= A(16 x 4) * B(4 x 16), B straight from the accumulation-register file (see XMfma in
// fused_gemm_xreg.hip for why this is an opaque statement and what that implies for readers of c)
__device__ __forceinline__ void xmfma_f32_first(f32x4& c, float a, float b)
{
    asm volatile("v_mfma_f32_16x16x4_f32 %0, %1, %2, 0" : "=v"(c) : "v"(a), "a"(b));
}
__device__ __forceinline__ void xmfma_f32_next(f32x4& c, float a, float b)
{
    asm volatile("v_mfma_f32_16x16x4_f32 %0, %1, %2, %0" : "+v"(c) : "v"(a), "a"(b));
}

// Geometry by K: a wavefront's 256 accumulation registers hold 16 NBF columns x K values.
template <int K>
struct GeomF32 {
    // (K = 256 would be 64 columns per wavefront; mi_fused_ht_gemm sends it to the GEMV kernels instead,
    // which are faster on every shape: fused_gemm_f32.hip)
    static_assert(K == 512 || K == 1024, "16 NBF columns x K fp32 values = 256 registers per lane");
    static constexpr int NBF = 1024 / K;      // 16-column fragments per wavefront
    static constexpr int CPW = 16 * NBF;      // columns per wavefront
    static constexpr int COLS = 4 * CPW;      // columns per workgroup
    static constexpr int KSTEPS = K / 16;     // 16-byte fragments (4 k per lane, 16 k per step) per column
    static constexpr int SPB = K / 128;       // W stages (64 rows x 128 k) per row block
    static constexpr int AHEAD = SPB >= 3 ? 3 : SPB;  // stages the W stream runs ahead of the MFMAs
    static constexpr int NM = 16 * NBF;       // MFMAs per K step: 4 row fragments x 4 k x NBF
    static constexpr int RCOLS = 4 * NBF;     // columns that pass through the LDS area together
};

// The prologue's LDS area of a wavefront (16 KB): [4 NBF columns][K / 4 chunks], chunk q of column
// c stored at q ^ 2 (c / NBF).  Every lane writes one chunk of a column (consecutive lanes,
// consecutive chunks); in round p only the lanes with lo / 4 == p read, chunk 4 s + hi of the
// columns NBF (lo % 4) + f.
template <int K>
__host__ __device__ constexpr uint32_t area_f32_offset(uint32_t c, uint32_t q)
{
    return c * (uint32_t)K * 4u + ((q ^ (2u * (c / (uint32_t)GeomF32<K>::NBF))) << 4);
}
template <int K>
constexpr bool area_f32_conflict_free()
{
    constexpr uint32_t NBF = GeomF32<K>::NBF;
    for (uint32_t c = 0; c < 4u * NBF; ++c)
        for (uint32_t t = 0; t < (uint32_t)K / 256u; ++t)
            if (!lds::conflict_free_b128([=](uint32_t lane) { return area_f32_offset<K>(c, 64u * t + lane); }))
                return false;
    for (uint32_t f = 0; f < NBF; ++f)
        for (uint32_t p = 0; p < 4; ++p)
            for (uint32_t s = 0; s < (uint32_t)K / 16u; ++s)
                if (!lds::conflict_free_b128_masked(
                        [=](uint32_t lane) { return area_f32_offset<K>(NBF * (lane & 3u) + f, 4u * s + (lane >> 4)); },
                        [=](uint32_t lane) { return ((lane & 15u) >> 2) == p; }))
                    return false;
    return true;
}
static_assert(area_f32_conflict_free<512>() && area_f32_conflict_free<1024>(),
              "an LDS access pattern of the fp32 prologue would serialise");

template <int K>
__global__ void __launch_bounds__(kThreads)
fused_ht_gemm_xreg_f32_kernel(const float* __restrict__ W, const float* __restrict__ Xt,
                              float* __restrict__ C, uint32_t M, uint32_t N, uint32_t m_per_block,
                              uint32_t msplit, uint32_t mpx, uint32_t cgx, uint32_t nrect, float fscale)
{
    using G = GeomF32<K>;
    constexpr int NBF = G::NBF, KSTEPS = G::KSTEPS, SPB = G::SPB, AHEAD = G::AHEAD, NM = G::NM;
    constexpr uint32_t kCols = G::COLS, CPW = G::CPW;
    static_assert(kSlots == 4 && AHEAD <= SPB && AHEAD >= 1, "stage g of the stream lives in buffer g % 4");
    static_assert(G::RCOLS * K * 4 == kAreaBytes, "a round of columns fills the wavefront's LDS area");
    constexpr uint32_t ROW_BYTES = K * 4u;

    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t lo = lane & 15u, hi = lane >> 4;

    uint32_t cg, ms;
    if (!tile_of_workgroup(blockIdx.x, msplit, mpx, cgx, nrect, cg, ms)) return;  // uniform, before any barrier
    const uint32_t n0 = cg * kCols;
    const uint32_t m_begin = ms * m_per_block;
    if (m_begin >= M || n0 >= N) return;  // workgroup-uniform, before any barrier
    const uint32_t m_end = min(M, m_begin + m_per_block);
    const uint32_t nrb = (m_end - m_begin + kRows - 1u) / kRows;
    auto row_block = [&](uint32_t rbi) __attribute__((always_inline)) {  // clamped: rbi <= nrb
        return rbi < nrb ? rbi : 0u;
    };

    // ---- W stream: as in the 16-bit kernel, with 4-byte elements (a stage row is 128 k) ------------
    const unsigned char* Wb = reinterpret_cast<const unsigned char*>(W);
    const uint32_t lds_base = (uint32_t)(uintptr_t)(lptr_t)lds;
    const uint32_t lrow = lane >> 5, lq = lane & 31u;
    uint32_t voff[8];
    auto set_voff = [&](uint32_t rbi) __attribute__((always_inline)) {
        const uint32_t r0 = m_begin + row_block(rbi) * kRows + 16u * wave + lrow;
#pragma unroll
        for (int i = 0; i < 8; ++i)
            voff[i] = min(r0 + 2u * i, M - 1u) * ROW_BYTES + ((lq ^ (2u * i + lrow)) << 4);
    };
    const uint32_t lds_wave_base = lds_base + 16u * wave * 512u;  // this wavefront's rows of a stage
    auto w_issue = [&](int kq, int slot, int i) __attribute__((always_inline)) {
        global_to_lds16(voff[i], Wb + kq * 512, lds_wave_base, slot * kStageBytes + 2 * i * 512);
    };
    set_voff(0);

    // ---- prologue: column f of lane (., lo) = column n0 + CPW w + NBF lo + f ------------------------
    // The wavefront's columns pass through its LDS area in four rounds of 4 NBF columns = eight
    // 512-element tiles (K = 1024: two tiles and one butterfly per column; K = 512: a tile per
    // column).
    // (yf is an array of scalars, not of 4-vectors: an MFMA names one register, and the compiler
    // keeps a vector's elements in the accumulation-register file only as a whole; with vectors
    // it copied every element into one scratch register right before use, while the previous MFMA
    // was still reading that register)
    float yf[NBF][KSTEPS][4];
    {
        unsigned char* area = lds + kAreaBase + wave * kAreaBytes;
        TileOperands<BF16> ops;
        make_tile_operands<BF16, 4>(9, ops);
        float in[8][8];
        auto load_tile = [&](int p4, int i) {
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                const uint32_t o = 512u * i + 256u * t;  // offset inside the round's columns
                const uint32_t col = min(n0 + CPW * wave + (uint32_t)(G::RCOLS * p4) + o / K, N - 1u);
                const f32x4 q = *reinterpret_cast<const f32x4*>(Xt + ((uint64_t)col * K + o % K + 4u * lane));
#pragma unroll
                for (int r = 0; r < 4; ++r) in[i][4 * t + r] = q[r];
            }
        };
        auto w_first = [&](int i) {  // the first AHEAD stages of W, behind the last round of X
#pragma unroll
            for (int u = 0; u < AHEAD; ++u) {
                const int pc = AHEAD * i + u;
                w_issue(pc >> 3, pc >> 3, pc & 7);
            }
        };
        auto put = [&](uint32_t c, uint32_t q, f32x4 v) {
            *reinterpret_cast<f32x4*>(area + area_f32_offset<K>(c, q)) = v * fscale;
        };
#pragma unroll
        for (int i = 0; i < 8; ++i) load_tile(0, i);
        // Pairs of tiles, software-pipelined by hand (one wavefront per SIMD hides nothing by
        // itself): while the MFMA chains of pair p run, the vector unit splits pair p + 1 into its
        // bf16 pieces, and the loads of the next round's pair p are already on their way.
        SplitTileF32 cur[2], nxt[2];
        split_tile_f32(in[0], cur[0]);
        split_tile_f32(in[1], cur[1]);
#pragma unroll
        for (int p4 = 0; p4 < 4; ++p4) {
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                if (p4 + 1 < 4) {  // in[2 p], in[2 p + 1] are split already: refill them for the next round
                    load_tile(p4 + 1, 2 * p);
                    load_tile(p4 + 1, 2 * p + 1);
                } else {
                    w_first(2 * p);
                    w_first(2 * p + 1);
                }
                // (the loads stay here, a round ahead of their use: left alone, the scheduler
                // sinks them to the use and the wavefront waits out every one)
                __builtin_amdgcn_sched_barrier(0);
                if (!(p4 == 3 && p == 3)) {
                    split_tile_f32(in[(2 * p + 2) & 7], nxt[0]);
                    split_tile_f32(in[(2 * p + 3) & 7], nxt[1]);
                }
                f32x4 a[2][2];
                tile_pair_mfma_f32(cur, ops, a);
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    if constexpr (K == 1024) {
                        // column p: element 512 half + 256 t + 4 lane + r = chunk 128 half + 64 t + lane
                        put(p, 64u * t + lane, a[0][t] + a[1][t]);
                        put(p, 128u + 64u * t + lane, a[0][t] - a[1][t]);
                    } else {
                        // columns 2 p, 2 p + 1: element 256 t + 4 lane + r
                        put(2 * p, 64u * t + lane, a[0][t]);
                        put(2 * p + 1, 64u * t + lane, a[1][t]);
                    }
                }
                cur[0] = nxt[0];
                cur[1] = nxt[1];
            }
            if ((int)(lo >> 2) == p4) {
#pragma unroll
                for (int f = 0; f < NBF; ++f)
#pragma unroll
                    for (int s = 0; s < KSTEPS; ++s) {
                        const f32x4 q = *reinterpret_cast<const f32x4*>(
                            area + area_f32_offset<K>(NBF * (lo & 3u) + f, 4u * s + hi));
#pragma unroll
                        for (int e = 0; e < 4; ++e) yf[f][s][e] = q[e];
                    }
            }
        }
    }

    wait_vm(8 * (AHEAD - 1));
    wait_lds();
    __builtin_amdgcn_s_barrier();

    auto frag = [&](uint32_t slot, int mb, int ks) __attribute__((always_inline)) -> f32x4 {
        return *reinterpret_cast<const f32x4*>(lds + slot * kStageBytes +
                                               stage_offset(16u * mb + lo, 4u * ks + hi));
    };
    f32x4 fr[4][4];  // [K step % 4][mb]
#pragma unroll
    for (int mb = 0; mb < 4; ++mb) {
        fr[0][mb] = frag(0, mb, 0);
        fr[1][mb] = frag(0, mb, 1);
    }

    // lane (hi, lo) of a row block owns rows 16 mb + 4 hi + r of columns col0 .. col0 + NBF - 1
    const uint32_t col0 = n0 + CPW * wave + NBF * lo;
    const uint32_t lane_off = (4u * hi * N + col0) * 4u;  // inside the row block, < 2^32
    unsigned char* const Cb = reinterpret_cast<unsigned char*>(C);
    const bool cols_full = n0 + kCols <= N && N % NBF == 0u;  // vector stores need aligned rows
    auto store_one = [&](const f32x4 (&acc)[4][NBF], uint64_t block_base, int mb, int r)
        __attribute__((always_inline)) {
        unsigned char* row_ptr = Cb + (block_base + (uint64_t)((16u * mb + r) * N) * 4u);  // scalar
        // (locals: a bit cast applied to a vector element expression itself reads element 0)
        const float v0 = acc[mb][0][r];
        if constexpr (NBF == 1) {
            stream_store4(lane_off, __float_as_uint(v0), row_ptr);
        } else {
            const float v1 = acc[mb][1][r];
            stream_store8(lane_off, u32x2{__float_as_uint(v0), __float_as_uint(v1)}, row_ptr);
        }
    };
    auto store_edge = [&](const f32x4 (&acc)[4][NBF], uint32_t row_base) __attribute__((always_inline)) {
#pragma unroll
        for (int f = 0; f < NBF; ++f) {
            if (col0 + f >= N) continue;
#pragma unroll
            for (int mb = 0; mb < 4; ++mb)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const uint32_t row = row_base + 16u * mb + 4u * hi + r;
                    if (row < m_end) C[(uint64_t)row * N + col0 + f] = acc[mb][f][r];
                }
        }
    };

    // One row block: SPB stages of 8 K steps of NM MFMAs.  `second`: the block is the odd one of a
    // pair (its stages start at buffer SPB % 4).  `prev_full`: `prev` holds the finished previous
    // block, stored behind the MFMAs of K step 6.
    auto row_block_body = [&](auto prev_tag, auto second_tag, f32x4 (&acc)[4][NBF], const f32x4 (&prev)[4][NBF],
                              uint64_t prev_base, uint32_t rbi) __attribute__((always_inline)) {
        constexpr bool prev_full = decltype(prev_tag)::value;
        constexpr int slot_base = decltype(second_tag)::value ? (SPB & 3) : 0;
        const bool last = rbi + 1u == nrb;
#pragma unroll
        for (int kq = 0; kq < SPB; ++kq) {
            constexpr int kPieceAt[7] = {0, 2, 4, 5, 6, 7, 8};
            // (everything below folds to constants once the loops are unrolled)
            const int cur_slot = (slot_base + kq) & 3, next_slot = (slot_base + kq + 1) & 3;
            const int fill_slot = (slot_base + kq + AHEAD) & 3;
            const int fill_kq = (kq + AHEAD) % SPB;
            const bool fill_own_block = kq + AHEAD < SPB;
#pragma unroll
            for (int ks = 0; ks < kStepsPerStage; ++ks) {
                if (kq == SPB - AHEAD && ks == 0 && !last) set_voff(rbi + 1u);
                const int kk = kq * kStepsPerStage + ks;
#pragma unroll
                for (int m = 0; m < NM; ++m) {
                    // consecutive MFMAs go to different accumulators
                    const int s = m / (4 * NBF), mb = m & 3, f = (m >> 2) % NBF;
                    if (kk == 0 && s == 0)
                        xmfma_f32_first(acc[mb][f], fr[ks & 3][mb][s], yf[f][0][s]);
                    else
                        xmfma_f32_next(acc[mb][f], fr[ks & 3][mb][s], yf[f][kk][s]);
                    // one memory instruction in the shadow of an MFMA: fragments two K steps ahead
                    // (the last four MFMAs: their registers were last read by the MFMAs of two
                    // steps ago), up to two transfer pieces, the previous block's sixteen stores
                    if (m >= NM - 4)
                        fr[(ks + 2) & 3][m - (NM - 4)] = ks < 6 ? frag(cur_slot, m - (NM - 4), ks + 2)
                                                                : frag(next_slot, m - (NM - 4), ks - 6);
                    else if (m >= 4 && m < 6) {
                        if (ks < 6 && (fill_own_block || !last)) {
                            const int i = kPieceAt[ks] + (m - 4);
                            if (i < kPieceAt[ks + 1]) w_issue(fill_kq, fill_slot, i);
                        }
                    }
                    if (prev_full && kk == 6 && m < 16) store_one(prev, prev_base, m >> 2, m & 3);
                    __builtin_amdgcn_sched_barrier(0);
                }
                // keep the previous step's fragment registers allocated while the matrix core may
                // still be reading them (see the 16-bit kernel)
                asm volatile("" ::"v"(fr[(ks + 3) & 3][0]), "v"(fr[(ks + 3) & 3][1]),
                             "v"(fr[(ks + 3) & 3][2]), "v"(fr[(ks + 3) & 3][3]));
                if (ks == 5) {
                    const int later = SPB - kq - 2 < AHEAD - 1 ? SPB - kq - 2 : AHEAD - 1;
                    const int after_last = kq == SPB - 1 ? -1 : 8 * (later > 0 ? later : 0);
                    if (last)
                        wait_vm(after_last);
                    else
                        wait_vm(8 * (AHEAD - 1));
                    wait_lds();
                    __builtin_amdgcn_s_barrier();
                }
            }
        }
    };

    auto store_block = [&](f32x4 (&acc)[4][NBF], uint64_t base) __attribute__((always_inline)) {
        drain_mfma(acc);
#pragma unroll
        for (int mb = 0; mb < 4; ++mb)
#pragma unroll
            for (int r = 0; r < 4; ++r) store_one(acc, base, mb, r);
    };
    auto finish = [&](f32x4 (&acc)[4][NBF], uint32_t rbi, bool& full, uint64_t& base)
        __attribute__((always_inline)) {
        const uint32_t row_base = m_begin + row_block(rbi) * kRows;
        full = cols_full && row_base + kRows <= m_end;
        base = (uint64_t)row_base * N * 4u;
        if (!full) {
            drain_mfma(acc);
            store_edge(acc, row_base);
        }
    };
    {
        // two accumulator sets: a finished block is stored behind the MFMAs of the next one
        f32x4 accA[4][NBF], accB[4][NBF];
        bool pend = false;        // accB holds a finished full row block that is not stored yet
        uint64_t pend_base = 0;
        auto run = [&](bool prev_full, auto second_tag, f32x4 (&acc)[4][NBF], const f32x4 (&prev)[4][NBF],
                       uint64_t prev_base, uint32_t rbi) __attribute__((always_inline)) {
            if (prev_full)
                row_block_body(std::true_type{}, second_tag, acc, prev, prev_base, rbi);
            else
                row_block_body(std::false_type{}, second_tag, acc, prev, prev_base, rbi);
        };
#pragma unroll 1
        for (uint32_t rbi = 0; rbi < nrb; rbi += 2u) {
            run(pend, std::false_type{}, accA, accB, pend_base, rbi);
            bool fullA;
            uint64_t baseA;
            finish(accA, rbi, fullA, baseA);
            if (rbi + 1u < nrb) {
                run(fullA, std::true_type{}, accB, accA, baseA, rbi + 1u);
                finish(accB, rbi + 1u, pend, pend_base);
            } else {
                pend = false;
                if (fullA) store_block(accA, baseA);
            }
        }
        if (pend) store_block(accB, pend_base);
    }
}

// ---- K = 2048, 4096: the K range split over pairs of wavefronts ---------------------------------
// A wavefront's registers hold 16 columns x 1024 values and the matrix core is 16 columns wide, so
// for larger K wavefront (cs, kp) = (wave / 2, wave % 2) holds one 1024-value quarter of the
// transformed columns 16 cs .. 16 cs + 15 (32 columns per workgroup).  With T_i the 1024-point
// transform of quarter i of a column x, H_K x has the quarters
//     K = 2048:  Y_0 = T_0 + T_1,  Y_1 = T_0 - T_1
//     K = 4096:  Y_j = sum_i (-1)^popcount(i & j) T_i
// K = 4096 runs two phases, one launch each: in phase ph the pair holds Y_{2 ph} and Y_{2 ph + 1}
// and walks all of its row blocks; phase 1 adds what phase 0 stored.  (One launch with a loop over
// the phases made the compiler carry values of the prologue across the main loop, and with them
// some of the transformed operand out of the accumulation registers.)
// W is streamed as two streams (the K ranges of the pair's two quarters), each through its own
// ring of four 16 KB stages (64 rows x 64 k); a wavefront reads the fragments of its own stream
// only.  At the end of a row block each wavefront of a pair hands the partner two of its four
// 16-row accumulator fragments through LDS and finishes (adds, stores) the other two.
// The prologue is shared inside a pair: per round, wavefront kp transforms column 2 r + kp of the
// set, all quarters of it, and writes the two quarters of this phase into the pair's LDS region;
// after a barrier each wavefront reads its own quarter of both columns.
namespace k2 {
constexpr int kStage = 16 * 1024;      // 64 rows x 256 B
constexpr int kSteps = 4;              // K steps of 16 per stage
constexpr int SPB = 16;                // stages per row block and stream
constexpr int AHEAD = 3;
// 128 KB: the prologue's regions [column set][quarter of the pair][column parity][4 KB], later the
// exchange buffers
constexpr uint32_t kAreaBase = 8 * kStage;
static_assert(kAreaBase + 2 * 2 * 2 * 4096 == (uint32_t)kLdsBytes, "rings and regions fill the 160 KB");
// LDS image of a stage: [64 rows][256 B], the 16-byte chunk q of row r stored at q ^ (r & 15)
__host__ __device__ constexpr uint32_t stage_offset(uint32_t row, uint32_t q)
{
    return row * 256u + ((q ^ (row & 15u)) << 4);
}
// a quarter's two columns: [2 columns][256 chunks], chunk q of column c stored at q ^ 2c
__host__ __device__ constexpr uint32_t area_offset(uint32_t c, uint32_t q) { return c * 4096u + ((q ^ (2u * c)) << 4); }
// the same for q = 4 s + hi, hi < 4, as a base and a multiple of s: the swizzle leaves the bits of s alone
__host__ __device__ constexpr uint32_t area_read_base(uint32_t c, uint32_t hi) { return c * 4096u + ((hi ^ (2u * c)) << 4); }
constexpr bool patterns_conflict_free()
{
    for (uint32_t c = 0; c < 2; ++c)
        for (uint32_t hi = 0; hi < 4; ++hi)
            for (uint32_t s = 0; s < 64; ++s)
                if (area_read_base(c, hi) + 64u * s != area_offset(c, 4u * s + hi)) return false;
    for (uint32_t mb = 0; mb < 4; ++mb)
        for (uint32_t ks = 0; ks < 4; ++ks)
            if (!lds::conflict_free_b128(
                    [=](uint32_t lane) { return stage_offset(16u * mb + (lane & 15u), 4u * ks + (lane >> 4)); }))
                return false;
    for (uint32_t c = 0; c < 2; ++c)
        for (uint32_t t = 0; t < 4; ++t)
            if (!lds::conflict_free_b128([=](uint32_t lane) { return area_offset(c, 64u * t + lane); })) return false;
    for (uint32_t p = 0; p < 8; ++p)
        for (uint32_t s = 0; s < 64; ++s)
            if (!lds::conflict_free_b128_masked(
                    [=](uint32_t lane) { return area_offset(lane & 1u, 4u * s + (lane >> 4)); },
                    [=](uint32_t lane) { return ((lane & 15u) >> 1) == p; }))
                return false;
    return true;
}
static_assert(patterns_conflict_free(), "an LDS access pattern of the split-K fp32 kernel would serialise");
}  // namespace k2

template <int K>
__global__ void __launch_bounds__(kThreads)
fused_ht_gemm_xreg_f32_ksplit_kernel(const float* __restrict__ W, const float* __restrict__ Xt,
                                     float* __restrict__ C, uint32_t M, uint32_t N, uint32_t m_per_block,
                                     uint32_t msplit, uint32_t mpx, uint32_t cgx, uint32_t nrect, float fscale,
                                     uint32_t ph)
{
    static_assert(K == 2048 || K == 4096, "two or four quarters of 1024");
    constexpr int NQ = K / 1024, PHASES = NQ / 2, KSTEPS = 64, NM = 16;
    constexpr int SPB = k2::SPB, AHEAD = k2::AHEAD;
    constexpr uint32_t kCols = 32;
    constexpr uint32_t ROW_BYTES = K * 4u;

    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t cs = wave >> 1, kp = wave & 1u;  // column set, quarter of the pair
    const uint32_t lo = lane & 15u, hi = lane >> 4;

    uint32_t cg, ms;
    if (!tile_of_workgroup(blockIdx.x, msplit, mpx, cgx, nrect, cg, ms)) return;  // uniform, before any barrier
    const uint32_t n0 = cg * kCols;
    const uint32_t m_begin = ms * m_per_block;
    if (m_begin >= M || n0 >= N) return;  // workgroup-uniform, before any barrier
    const uint32_t m_end = min(M, m_begin + m_per_block);
    const uint32_t nrb = (m_end - m_begin + kRows - 1u) / kRows;
    auto row_block = [&](uint32_t rbi) __attribute__((always_inline)) { return rbi < nrb ? rbi : 0u; };

    // ---- W streams: per stage time a wavefront moves rows 16 w .. 16 w + 15 of both streams' stages,
    // eight pieces of 4 rows x 256 B (piece i: stream i / 4, rows 4 (i % 4) .. + 3)
    const unsigned char* Wb = reinterpret_cast<const unsigned char*>(W);
    const uint32_t lds_base = (uint32_t)(uintptr_t)(lptr_t)lds;
    const uint32_t lrow = lane >> 4, lq = lane & 15u;
    uint32_t voff[8];
    auto set_voff = [&](uint32_t rbi) __attribute__((always_inline)) {
        const uint32_t r0 = m_begin + row_block(rbi) * kRows + 16u * wave + lrow;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t j = i & 3, sp = i >> 2;
            voff[i] = min(r0 + 4u * j, M - 1u) * ROW_BYTES + sp * 4096u + ((lq ^ (4u * j + lrow)) << 4);
        }
    };

    // wavefront (cs, kp) finishes row fragments mb = 2 kp, 2 kp + 1: lane (hi, lo) owns rows
    // 16 mb + 4 hi + r of column n0 + 16 cs + lo
    const uint32_t col = n0 + 16u * cs + lo;
    const uint32_t lane_off = (4u * hi * N + col) * 4u;  // inside the row block, < 2^32
    unsigned char* const Cb = reinterpret_cast<unsigned char*>(C);
    const bool cols_full = n0 + kCols <= N;
    unsigned char* const xb_mine = lds + k2::kAreaBase + wave * 2048u;
    const unsigned char* const xb_partner = lds + k2::kAreaBase + (wave ^ 1u) * 2048u;
    const unsigned char* const ring = lds + kp * 4u * k2::kStage;  // this wavefront's stream
    const uint32_t lds_wave_base = lds_base + 16u * wave * 256u;     // this wavefront's rows of a stage
    auto frag = [&](uint32_t slot, int mb, int ks) __attribute__((always_inline)) -> f32x4 {
        return *reinterpret_cast<const f32x4*>(ring + slot * k2::kStage + k2::stage_offset(16u * mb + lo, 4u * ks + hi));
    };

    {
        const unsigned char* Wph = Wb + (uint32_t)ph * 8192u;  // the pair's two quarters of every row
        auto w_issue = [&](int kq, int i) __attribute__((always_inline)) {
            const int j = i & 3, sp = i >> 2;
            global_to_lds16(voff[i], Wph + kq * 256, lds_wave_base, (sp * 4 + (kq & 3)) * k2::kStage + 4 * j * 256);
        };
        set_voff(0);

        // ---- prologue ----------------------------------------------------------------------------
        float yf[KSTEPS][4];
        {
            unsigned char* const region = lds + k2::kAreaBase + cs * 16384u;  // [quarter of the pair][8 KB]
            TileOperands<BF16> ops;
            make_tile_operands<BF16, 4>(9, ops);
            const float sigma = ph ? -1.0f : 1.0f;
            float in[2 * NQ][8];  // tiles 2 i, 2 i + 1 = quarter i of the column
            const float* Xp = Xt;
            const uint32_t lane4 = 4u * lane;
            auto load_tile = [&](int r, int i) {
                const uint32_t c = min(n0 + 16u * cs + 2u * r + kp, N - 1u);
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    const f32x4 q = *reinterpret_cast<const f32x4*>(
                        Xp + ((uint64_t)c * K + 512u * i + 256u * t + lane4));
#pragma unroll
                    for (int e = 0; e < 4; ++e) in[i][4 * t + e] = q[e];
                }
            };
#pragma unroll
            for (int i = 0; i < 2 * NQ; ++i) load_tile(0, i);
            // K = 4096: the transform is linear, so the two quarters this phase keeps are
            //   Y_{2 ph} = T(u) + T(v),  Y_{2 ph + 1} = T(u) - T(v),
            //   u = x_0 + sigma x_2,  v = x_1 + sigma x_3,  sigma = (-1)^ph,
            // x_i the quarters of the column: two 1024-point transforms per column and phase instead of
            // four (the sums are fp32 additions of the inputs: one more rounding of 2^-24).
            // K = 2048: u = x_0, v = x_1.  `half` = tile j (0 .. 3) of (u, v).
            auto split_half = [&](int j, SplitTileF32& o) __attribute__((always_inline)) {
                if constexpr (NQ == 4) {
                    float t[8];
#pragma unroll
                    for (int e = 0; e < 8; ++e) t[e] = in[j][e] + sigma * in[j + 4][e];
                    split_tile_f32(t, o);
                } else {
                    split_tile_f32(in[j], o);
                }
            };
            // Halves (pairs of tiles) software-pipelined by hand, as in the kernel above: while the
            // MFMA chains of one half run, the vector unit splits the next one.
            SplitTileF32 cur[2], nxt[2];
            split_half(0, cur[0]);
            split_half(1, cur[1]);
#pragma unroll
            for (int r = 0; r < 8; ++r) {
                // Y[h][g][t]: elements 512 g + 256 t + 4 lane + e of quarter h of this phase:
                //   Y[0] = T(u) + T(v),  Y[1] = T(u) - T(v)
                f32x4 Y[2][2][2];
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    if (r + 1 < 8) {  // tiles 2 i, 2 i + 1 (and their partners) are split already: refill them
                        load_tile(r + 1, 2 * i);
                        load_tile(r + 1, 2 * i + 1);
                        if (NQ == 4) {
                            load_tile(r + 1, 2 * i + 4);
                            load_tile(r + 1, 2 * i + 5);
                        }
                    }
                    // (the loads stay here, a round ahead of their use: left alone, the scheduler
                    // sinks them to the use and the wavefront waits out every one)
                    __builtin_amdgcn_sched_barrier(0);
                    if (!(r == 7 && i == 1)) {
                        split_half((2 * i + 2) % 4, nxt[0]);
                        split_half((2 * i + 3) % 4, nxt[1]);
                    }
                    f32x4 a[2][2];
                    tile_pair_mfma_f32(cur, ops, a);
    #pragma unroll
                    for (int t = 0; t < 2; ++t) {
                        const f32x4 u = a[0][t] + a[1][t], v = a[0][t] - a[1][t];  // the two halves of T
                        if (i == 0) {
                            Y[0][0][t] = u, Y[0][1][t] = v, Y[1][0][t] = u, Y[1][1][t] = v;
                        } else {
                            Y[0][0][t] = Y[0][0][t] + u;
                            Y[0][1][t] = Y[0][1][t] + v;
                            Y[1][0][t] = Y[1][0][t] - u;
                            Y[1][1][t] = Y[1][1][t] - v;
                        }
                    }
                    cur[0] = nxt[0];
                    cur[1] = nxt[1];
                }
                if (r >= 4) {  // the first AHEAD stage times of W, behind the last rounds of X
#pragma unroll
                    for (int u = 0; u < 2 * AHEAD; ++u) {
                        const int pc = 2 * AHEAD * (r - 4) + u;
                        w_issue(pc >> 3, pc & 7);
                    }
                }
                // the partner has read the previous round's columns
                wait_lds();
                __builtin_amdgcn_s_barrier();
#pragma unroll
                for (int h = 0; h < 2; ++h)
#pragma unroll
                    for (int t = 0; t < 2; ++t) {
                        // element 512 g + 256 t + 4 lane + e of the quarter = chunk 128 g + 64 t + lane
                        unsigned char* dst = region + h * 8192u;
                        *reinterpret_cast<f32x4*>(dst + k2::area_offset(kp, 64u * t + lane)) = Y[h][0][t] * fscale;
                        *reinterpret_cast<f32x4*>(dst + k2::area_offset(kp, 128u + 64u * t + lane)) =
                            Y[h][1][t] * fscale;
                    }
                wait_lds();
                __builtin_amdgcn_s_barrier();
                if ((int)(lo >> 1) == r) {
                    // chunk 4 s + hi of column lo % 2: one base address and constant offsets
                    const unsigned char* src = region + kp * 8192u + k2::area_read_base(lo & 1u, hi);
#pragma unroll
                    for (int s = 0; s < KSTEPS; ++s) {
                        const f32x4 q = *reinterpret_cast<const f32x4*>(src + 64u * s);
#pragma unroll
                        for (int e = 0; e < 4; ++e) yf[s][e] = q[e];
                    }
                }
            }
        }

        wait_vm(8 * (AHEAD - 1));
        wait_lds();
        __builtin_amdgcn_s_barrier();

        f32x4 fr[4][4];  // [K step % 4][mb]
#pragma unroll
        for (int mb = 0; mb < 4; ++mb) {
            fr[0][mb] = frag(0, mb, 0);
            fr[1][mb] = frag(0, mb, 1);
        }

        f32x4 acc[4][1];
#pragma unroll 1
        for (uint32_t rbi = 0; rbi < nrb; ++rbi) {
            const bool last = rbi + 1u == nrb;
            const uint32_t row_base = m_begin + rbi * kRows;
            const bool full = cols_full && row_base + kRows <= m_end;
            f32x4 before[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};  // what phase 0 stored
#pragma unroll
            for (int kq = 0; kq < SPB; ++kq) {
                // (everything below folds to constants once the loops are unrolled; SPB is a multiple
                // of 4, so stage kq of every row block lives in buffer kq % 4 of its stream)
                const int cur_slot = kq & 3, next_slot = (kq + 1) & 3;
                const int fill_kq = (kq + AHEAD) % SPB;
                const bool fill_own_block = kq + AHEAD < SPB;
                if (PHASES > 1 && kq == SPB - 2 && ph > 0 && col < N) {
#pragma unroll
                    for (int f = 0; f < 2; ++f)
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            const uint32_t row = row_base + 32u * kp + 16u * f + 4u * hi + r;
                            if (row < m_end) before[f][r] = __builtin_nontemporal_load(&C[(uint64_t)row * N + col]);
                        }
                }
#pragma unroll
                for (int ks = 0; ks < k2::kSteps; ++ks) {
                    if (kq == SPB - AHEAD && ks == 0 && !last) set_voff(rbi + 1u);
                    const int kk = kq * k2::kSteps + ks;
#pragma unroll
                    for (int m = 0; m < NM; ++m) {
                        const int s = m >> 2, mb = m & 3;  // consecutive MFMAs go to different accumulators
                        if (kk == 0 && s == 0)
                            xmfma_f32_first(acc[mb][0], fr[ks & 3][mb][s], yf[0][s]);
                        else
                            xmfma_f32_next(acc[mb][0], fr[ks & 3][mb][s], yf[kk][s]);
                        // one memory instruction in the shadow of an MFMA: fragments two K steps
                        // ahead, the eight transfer pieces of this stage time in its first two steps
                        if (m >= 12)
                            fr[(ks + 2) & 3][m - 12] =
                                ks < 2 ? frag(cur_slot, m - 12, ks + 2) : frag(next_slot, m - 12, ks - 2);
                        else if (m >= 4 && m < 8) {
                            if (ks < 2 && (fill_own_block || !last)) w_issue(fill_kq, 4 * ks + (m - 4));
                        }
                        __builtin_amdgcn_sched_barrier(0);
                    }
                    // keep the previous step's fragment registers allocated while the matrix core
                    // may still be reading them (see the 16-bit kernel)
                    asm volatile("" ::"v"(fr[(ks + 3) & 3][0]), "v"(fr[(ks + 3) & 3][1]),
                                 "v"(fr[(ks + 3) & 3][2]), "v"(fr[(ks + 3) & 3][3]));
                    if (ks == 1) {
                        const int later = SPB - kq - 2 < AHEAD - 1 ? SPB - kq - 2 : AHEAD - 1;
                        const int after_last = kq == SPB - 1 ? -1 : 8 * (later > 0 ? later : 0);
                        if (last)
                            wait_vm(after_last);
                        else
                            wait_vm(8 * (AHEAD - 1));
                        wait_lds();
                        __builtin_amdgcn_s_barrier();
                    }
                }
            }
            // ---- the pair's two quarters meet: hand over two fragments, finish the other two --------
            drain_mfma(acc);
            f32x4 keep[2], give[2];
            if (kp) {
                keep[0] = acc[2][0], keep[1] = acc[3][0], give[0] = acc[0][0], give[1] = acc[1][0];
            } else {
                keep[0] = acc[0][0], keep[1] = acc[1][0], give[0] = acc[2][0], give[1] = acc[3][0];
            }
#pragma unroll
            for (int f = 0; f < 2; ++f) *reinterpret_cast<f32x4*>(xb_mine + f * 1024u + lane * 16u) = give[f];
            wait_lds();
            __builtin_amdgcn_s_barrier();
            f32x4 sum[2];
#pragma unroll
            for (int f = 0; f < 2; ++f) {
                const f32x4 got = *reinterpret_cast<const f32x4*>(xb_partner + f * 1024u + lane * 16u);
                sum[f] = kp ? got + keep[f] : keep[f] + got;  // always (lower quarter) + (upper quarter)
                if (PHASES > 1) sum[f] = before[f] + sum[f];
            }
            if (full) {
                const uint64_t block_base = ((uint64_t)row_base + 32u * kp) * N * 4u;
#pragma unroll
                for (int f = 0; f < 2; ++f)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        unsigned char* row_ptr = Cb + (block_base + (uint64_t)((16u * f + r) * N) * 4u);  // scalar
                        const float v = sum[f][r];
                        stream_store4(lane_off, __float_as_uint(v), row_ptr);
                    }
            } else if (col < N) {
#pragma unroll
                for (int f = 0; f < 2; ++f)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const uint32_t row = row_base + 32u * kp + 16u * f + 4u * hi + r;
                        if (row < m_end) C[(uint64_t)row * N + col] = sum[f][r];
                    }
            }
        }
    }
}

}  // namespace xreg

namespace {
template <int K>
int launch_xreg_f32(const float* W, const float* Xt, float* C, uint32_t M, uint32_t N, float scale, hipStream_t s)
{
    using namespace xreg;
    constexpr uint32_t log2k = K == 512 ? 9 : 10;
    const int shift = tile_stage_shift<4>(log2k, false);
    const float fscale = (float)((double)scale * (double)(1u << shift));
    const Plan p = plan(M, N, (uint32_t)GeomF32<K>::COLS, 8u, 9u, 8u);
    auto kern = fused_ht_gemm_xreg_f32_kernel<K>;
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                            kLdsBytes) != hipSuccess)
        return MI_ERR_LAUNCH;
    hipLaunchKernelGGL(kern, dim3(p.grid), dim3(kThreads), kLdsBytes, s, W, Xt, C, M, N, p.m_per_block,
                       p.msplit, p.mpx, p.cgx, p.nrect, fscale);
    return launch_status();
}
template <int K>
int launch_ksplit_f32(const float* W, const float* Xt, float* C, uint32_t M, uint32_t N, float scale, hipStream_t s)
{
    using namespace xreg;
    const float fscale = (float)((double)scale * (double)(1u << tile_stage_shift<4>(9, false)));
    const Plan p = plan(M, N, 32u, 8u, K == 4096 ? 18u : 9u, 8u);
    auto kern = fused_ht_gemm_xreg_f32_ksplit_kernel<K>;
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                            kLdsBytes) != hipSuccess)
        return MI_ERR_LAUNCH;
    for (uint32_t ph = 0; ph < (uint32_t)K / 2048u; ++ph)
        hipLaunchKernelGGL(kern, dim3(p.grid), dim3(kThreads), kLdsBytes, s, W, Xt, C, M, N, p.m_per_block,
                           p.msplit, p.mpx, p.cgx, p.nrect, fscale, ph);
    return launch_status();
}
}  // namespace

// Called by the fp32 dispatcher of mi_fused_ht_gemm for K = 512 ... 4096 (arguments already
// validated).
int fused_gemm_f32_xreg(const float* W, const float* Xt, float* C, uint32_t M, uint32_t N, uint32_t K,
                        float scale, hipStream_t s)
{
    // W and a row block of C are addressed with 32-bit byte offsets
    if ((uint64_t)M * K * 4u > 0xffffffffull || (uint64_t)N * 4u * 64u > 0xffffffffull) return MI_ERR_SHAPE;
    switch (K) {
        case 512: return launch_xreg_f32<512>(W, Xt, C, M, N, scale, s);
        case 1024: return launch_xreg_f32<1024>(W, Xt, C, M, N, scale, s);
        case 2048: return launch_ksplit_f32<2048>(W, Xt, C, M, N, scale, s);
        case 4096: return launch_ksplit_f32<4096>(W, Xt, C, M, N, scale, s);
        default: return MI_ERR_SIZE;
    }
}

}  // namespace mi
