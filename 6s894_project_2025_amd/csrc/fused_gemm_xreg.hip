// Fused Hadamard -> GEMM with the transformed operand held in registers, gfx950, 16-bit inputs:
//     C[M,N] = W[M,K] * (scale * H_K * X[K,N]),  X given as Xt[N,K],  K = 512 or 1024
// (K = 2048, with the K range split over pairs of wavefronts: fused_gemm_xreg_k2048.hip).
//
// One workgroup = four wavefronts, one per SIMD, each with the whole 512-register budget.
//   prologue : wavefront w transforms 32768 / K columns of X (64 or 32) on the
//              matrix cores (coalesced 16-byte loads, the two-stage tile transform of
//              fwht_device.hpp; at K = 1024 the last butterfly is folded into the second stage),
//              passes them once through a wavefront-private LDS area to get from "a lane owns 8
//              consecutive k of one column" to MFMA operand order "lane (hi, lo) owns 8
//              consecutive k of column lo", and keeps all 32768 values in the 256 accumulation
//              registers for the rest of the kernel.  The workgroup therefore owns 256 or 128
//              columns, twice what fits in LDS.
//   main loop: the workgroup walks its M range in 64-row blocks.  W is the only operand that
//              moves: global -> LDS directly (no register hop), each wavefront fetching a quarter
//              of a 64-row x 256-K stage as whole 512-byte row segments into a ring of four
//              stage buffers, three stages ahead; every wavefront then reads all of it back as
//              MFMA A fragments (LDS is the broadcast medium: a W fragment serves the four
//              wavefronts' different columns).  One workgroup barrier per stage, placed after
//              the stage's last fragment read has been issued, so the first fragments of the next
//              stage are read behind the stage's last sixteen MFMAs.  With one wavefront per SIMD
//              nothing hides an instruction that waits, so every memory instruction is issued in
//              the shadow of a running MFMA.
//   epilogue : D[row 4*hi + r][column lo] of the two column fragments is packed into pairs of
//              adjacent columns and stored straight from registers, one store per K step of the
//              *next* row block (two accumulator sets take turns).
// Per compute unit the kernel reads 128 columns of X once and a 1/msplit share of W once; the
// register file, not LDS, decides how many columns a compute unit can keep.
//
// Behaviour replaced: fused_ht_gemm_pipelined, fused_ht/fusion_pipelined.cu:306-563; its
// "Load(t+1) || GEMM(t)" pipeline with asynchronous 16-byte copies (:247-268, :468-543) is the W
// stream here.
#include <type_traits>

#include "xreg_common.hpp"
#include "xreg_mfma16.hpp"

namespace mi {
namespace xreg {


// What follows from K: the transformed operand of a wavefront always fills its 256 accumulation
// registers (64 fragments of 16 columns x 32 k).
template <int K>
struct Geom {
    static_assert(K == 512 || K == 1024,
                  "register budget: 16 NBF columns x K = 32768 values per wavefront (K = 2048: "
                  "fused_gemm_xreg_k2048.hip)");
    static constexpr int NBF = 2048 / K;            // 16-column fragments per wavefront
    static constexpr int CPW = 16 * NBF;            // columns per wavefront
    static constexpr int COLS = 4 * CPW;            // columns per workgroup
    static constexpr int KSTEPS = K / 32;           // MFMA K steps per row block
    static constexpr int SPB = K / kStageK;         // W stages per row block
    static constexpr int AHEAD = SPB >= 3 ? 3 : 2;  // stages the W stream runs ahead of the MFMAs
    static constexpr int NM = 4 * NBF;              // MFMAs per K step
};


template <class T16, int K, bool OUT_F32>
__global__ void __launch_bounds__(kThreads)
fused_ht_gemm_xreg_kernel(const typename T16::E* __restrict__ W,
                          const typename T16::E* __restrict__ Xt, void* __restrict__ C, uint32_t M,
                          uint32_t N, uint32_t m_per_block, uint32_t msplit, uint32_t mpx,
                          uint32_t cgx, uint32_t nrect, int exp2, float mult)
{
    using E = typename T16::E;
    using V8 = typename T16::V8;
    typedef E V2 __attribute__((ext_vector_type(2)));
    typedef E V4 __attribute__((ext_vector_type(4)));
    using G = Geom<K>;
    constexpr int NBF = G::NBF, KSTEPS = G::KSTEPS, SPB = G::SPB, AHEAD = G::AHEAD, NM = G::NM;
    constexpr uint32_t kCols = G::COLS, CPW = G::CPW;
    static_assert(kSlots == 4 && AHEAD <= SPB && AHEAD + 1 <= kSlots, "stage g lives in buffer g % 4");
    constexpr uint32_t ROW_BYTES = K * 2u;

    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t lo = lane & 15u, hi = lane >> 4;

    // ---- which tile: consecutive workgroup ids go to different XCDs (id % 8).  The grid of
    // (column group, M slice) tiles is cut into rectangles of cgx column groups x mpx M slices, and
    // a rectangle is handled inside one XCD by workgroups that are dispatched back to back: its
    // L2 then holds mpx slices of W, each shared by cgx workgroups, and cgx blocks of X, each
    // shared by mpx.  (mpx = 1 keeps one slice of W per XCD but makes it read eight times as much
    // of X; 2 - 4 measured best.)  Rectangle r runs on XCD r % 8; ids past the last rectangle have
    // no work.
    uint32_t cg, ms;
    if (!tile_of_workgroup(blockIdx.x, msplit, mpx, cgx, nrect, cg, ms)) return;  // uniform, before any barrier
    const uint32_t n0 = cg * kCols;
    const uint32_t m_begin = ms * m_per_block;
    if (m_begin >= M || n0 >= N) return;  // workgroup-uniform, before any barrier
    const uint32_t m_end = min(M, m_begin + m_per_block);
    const uint32_t nrb = (m_end - m_begin + kRows - 1u) / kRows;
    // Workgroups that share a slice of W walk it in the same order and at the same pace: the first
    // one to ask for a line brings it into the XCD's L2, the others hit (starting them at
    // different row blocks, to spread the requests, measured 3 % slower).
    auto row_block = [&](uint32_t rbi) __attribute__((always_inline)) {  // clamped: rbi <= nrb
        return rbi < nrb ? rbi : 0u;
    };

    // ---- W stream -------------------------------------------------------------------------------
    // Stage g = (row block g / SPB, K range 256 (g % SPB) ...) lives in stage buffer g % 4.  Wavefront w moves
    // rows 16w .. 16w+15 of the block in eight pieces; piece i = rows 2i, 2i+1: lane l fetches row
    // 2i + l/32 and lands at byte 16 l of the piece's 1 KB of LDS (the transfer's fixed lane order).
    // LDS stage image: [64 rows][512 B] with 16-byte chunk q of row r stored at q ^ (r & 15), so
    // the lane asks for chunk (l % 32) ^ (r & 15): a half-wavefront still covers one contiguous
    // 512-byte row segment (four adjacent lanes one aligned 64-byte run), and a fragment read
    // (lane (hi, lo): row 16 mb + lo, chunk 4 ks + hi) hits 16 different 16-byte bank groups.
    const unsigned char* Wb = reinterpret_cast<const unsigned char*>(W);
    const uint32_t lds_base = (uint32_t)(uintptr_t)(lptr_t)lds;  // LDS byte address of the array
    const uint32_t lrow = lane >> 5, lq = lane & 31u;
    uint32_t voff[8];  // byte offset of this lane's 16 bytes of piece i, K quarter 0, in W
    auto set_voff_piece = [&](uint32_t rbi, int i) __attribute__((always_inline)) {
        const uint32_t r0 = m_begin + row_block(rbi) * kRows + 16u * wave + lrow;
        voff[i] = min(r0 + 2u * i, M - 1u) * ROW_BYTES + ((lq ^ (2u * i + lrow)) << 4);
    };
    auto set_voff = [&](uint32_t rbi) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 8; ++i) set_voff_piece(rbi, i);
    };
    const uint32_t lds_wave_base = lds_base + 16u * wave * 512u;  // this wavefront's rows of a stage
    auto w_issue = [&](int kq, int slot, int i) __attribute__((always_inline)) {
        global_to_lds16(voff[i], Wb + kq * (kStageK * 2), lds_wave_base, slot * kStageBytes + 2 * i * 512);
    };
    // the same in two halves, one on either side of an MFMA of the main loop
    auto w_target = [&](int slot, int i) __attribute__((always_inline)) {
        lds_transfer_target(lds_wave_base, slot * kStageBytes + 2 * i * 512);
    };
    auto w_go = [&](int kq, int i) __attribute__((always_inline)) {
        lds_transfer_go(voff[i], Wb + kq * (kStageK * 2));
    };
    set_voff(0);

    // ---- prologue: Y fragments of this wavefront's columns ---------------------------------------
    // Column of fragment nb, fragment column j (= MFMA B column = lane lo): n0 + CPW w + NBF j + nb,
    // so that a lane ends up with NBF adjacent output columns.  Columns are taken in the order
    // c = 16 nb + j as one software pipeline in which four things run side by side:
    //   - the fetch of X: column c + 16 is requested when column c has been consumed, so sixteen
    //     columns (32 KB per wavefront) are in flight all the time, enough to keep the path from the
    //     L2 busy across its latency;
    //   - the transform of column c on the matrix cores (its conversions in the MFMAs' shadow);
    //   - the layout change through LDS: a transformed column is written as it is produced (lane l
    //     owns 8 consecutive k), and the sixteen columns of a round are read back in operand order
    //     (lane (hi, lo): 8 consecutive k of column lo) during the first four columns of the next
    //     round, whose own results wait in registers until those reads have been issued (LDS
    //     operations of one wavefront complete in order: no barrier between its writes and reads);
    //   - stage 0 of W, requested behind the X columns of the first round.
    // Only the last round's reads are left over at the end.  The wavefront's LDS area is 32 KB (a
    // whole round at K = 1024, two rounds taking turns at K = 512), laid over its own rows of stage
    // buffers 1 .. 3 and of the 32 KB behind the ring: once its last reads have returned, the
    // wavefront requests its pieces of stages 1 .. AHEAD - 1 without waiting for anybody else.
    V8 yf[NBF][KSTEPS];
    {
        constexpr int NH = K / 512;       // 512-element halves of a column
        constexpr int TOTAL = 16 * NBF;   // columns of this wavefront
        constexpr int RPR = KSTEPS;       // reads per round: one per K step
        // half/buffer b, column j -> byte offset inside the workgroup's LDS, before the chunk term
        auto area_at = [&](int b, uint32_t j) __attribute__((always_inline)) -> uint32_t {
            return area_piece_offset(wave, (uint32_t)b + 2u * (j >> 3)) + (j & 7u) * 1024u;
        };
        constexpr int LA = K == 1024 ? 12 : 16;   // columns in flight (what the register file leaves room for)
        V8 in[LA][NH];
        // X is addressed as a uniform base (the wavefront's first column, clamped into the matrix)
        // plus a 32-bit lane offset: column (clamped to the last one) and the lane's 16 bytes
        const uint32_t col_first = min(n0 + CPW * wave, N - 1u);
        const unsigned char* const xb = reinterpret_cast<const unsigned char*>(Xt) + (uint64_t)col_first * (K * 2u);
        const uint32_t last_rel = (N - 1u - col_first) * (K * 2u), lane16 = lane << 4;
        auto column_offset = [&](int c) __attribute__((always_inline)) -> uint32_t {
            return min((uint32_t)(NBF * (c & 15) + (c >> 4)) * (K * 2u), last_rel) + lane16;
        };
        auto load_col = [&](int c) __attribute__((always_inline)) {
            const uint32_t off = column_offset(c);
#pragma unroll
            for (int t = 0; t < NH; ++t)
                in[c % LA][t] = *reinterpret_cast<const V8*>(xb + off + 1024u * t);
        };
#pragma unroll
        for (int c = 0; c < LA; ++c) load_col(c);
        PairOperands<T16> po;
        TileOperands<T16> ops;
        if constexpr (K == 1024)
            make_pair_operands<T16>(po, exp2);
        else
            make_tile_operands<T16, 2>(9, ops, exp2);
        V8 held[4][NH];
        // the reads of round nb, eight (K = 1024) or four (K = 512) at a time
        auto read_back = [&](int nb, int first, int count) __attribute__((always_inline)) {
#pragma unroll
            for (int r = first; r < first + count; ++r) {
                const int b = NH == 2 ? r / 16 : (nb & 1), s16 = r % 16;
                yf[nb][r] = *reinterpret_cast<const V8*>(lds + area_at(b, lo) + (((4u * s16 + hi) ^ lo) << 4));
            }
        };
        auto write_col = [&](int nb, int j, const V8 (&out)[NH]) __attribute__((always_inline)) {
#pragma unroll
            for (int t = 0; t < NH; ++t) {
                const int b = NH == 2 ? t : (nb & 1);
                *reinterpret_cast<V8*>(lds + area_at(b, (uint32_t)j) + ((lane ^ (uint32_t)j) << 4)) = out[t];
            }
        };
        if constexpr (K == 1024) {
            // Columns go through in pairs (A = column 2p, B = column 2p + 1), sixteen MFMA slots per
            // pair: stage 1 of A, stage 1 of B, stage 2 of A, stage 2 of B, four MFMAs each.  The
            // thirty-two conversions, four LDS writes and four loads of a pair are placed between
            // them by hand, every one at least three slots behind the MFMA whose result it reads, so
            // that no instruction waits for a result (the compiler's own order finishes one column
            // before it starts the next).  Slot k of pair p therefore also carries work of pair p - 1.
            // What bounds the loop is instruction issue: a lone wavefront issues about one
            // instruction every eight cycles (measured: an MFMA plus one vector or scalar
            // instruction per 16-cycle MFMA slot is free, every further one adds eight cycles), and a
            // column is eight MFMAs and some twenty-two other instructions.
            struct Col {
                f32x4 d0[2], d1[2];   // stage 1: tile 0 / tile 1, output half h
                u32x4 a2[2];          // the same rounded to 16 bits: operand of stage 2
                f32x4 s[2], d[2];     // stage 2: first / second half of the column
                u32x4 o[2];           // rounded: what goes to LDS
            };
            Col st[2][2];             // [pair parity][A, B]
            const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
            auto pack = [](float a, float b) __attribute__((always_inline)) -> uint32_t {
                return __builtin_bit_cast(uint32_t, V2{(E)a, (E)b});
            };
            auto S1 = [&](Col& c, int col, int i) __attribute__((always_inline)) {
                const int h = i >> 1;
                if (i & 1)
                    c.d1[h] = T16::mfma32(in[col % LA][1], po.g1[h], zero);
                else
                    c.d0[h] = T16::mfma32(in[col % LA][0], po.g1[h], zero);
            };
            auto C1 = [&](Col& c, int i) __attribute__((always_inline)) {
                const int h = i >> 2, q = i & 3;
                c.a2[h][q] = q < 2 ? pack(c.d0[h][2 * q], c.d0[h][2 * q + 1])
                                   : pack(c.d1[h][2 * q - 4], c.d1[h][2 * q - 3]);
            };
            auto S2 = [&](Col& c, int i) __attribute__((always_inline)) {
                const int h = i >> 1;
                if (i & 1)
                    c.d[h] = T16::mfma32(__builtin_bit_cast(V8, c.a2[h]), po.g2d, zero);
                else
                    c.s[h] = T16::mfma32(__builtin_bit_cast(V8, c.a2[h]), po.g2s, zero);
            };
            auto C2 = [&](Col& c, int i) __attribute__((always_inline)) {
                const int h = i >> 2, q = i & 3;
                if (q < 2)
                    c.o[0][2 * h + q] = pack(c.s[h][2 * q], c.s[h][2 * q + 1]);
                else
                    c.o[1][2 * h + q - 2] = pack(c.d[h][2 * q - 4], c.d[h][2 * q - 3]);
            };
            // column `col` is complete: to LDS, or into `held` while the previous round is read back
            auto WR = [&](Col& c, int col, int t) __attribute__((always_inline)) {
                const int nb = col >> 4, j = col & 15;
                const V8 v = __builtin_bit_cast(V8, c.o[t]);
                if (nb > 0 && j < 4)
                    held[j][t] = v;
                else
                    *reinterpret_cast<V8*>(lds + area_at(t, (uint32_t)j) + ((lane ^ (uint32_t)j) << 4)) = v;
            };
            auto LD = [&](int col, int t) __attribute__((always_inline)) {
                if (col >= TOTAL) return;
                in[col % LA][t] = *reinterpret_cast<const V8*>(xb + column_offset(col) + 1024u * t);
            };
            constexpr int PAIRS = TOTAL / 2;
#pragma unroll
            for (int p = 0; p <= PAIRS; ++p) {
                const int a = 2 * p, b = 2 * p + 1;        // this pair's columns
                Col& A = st[p & 1][0];
                Col& B = st[p & 1][1];
                Col& PA = st[(p + 1) & 1][0];              // the pair before
                Col& PB = st[(p + 1) & 1][1];
                const bool cur = p < PAIRS, prev = p > 0;
                // The previous round is read back one read per slot, from the slot after its last
                // column was written (slot 5 of the round's first pair) on: 32 slots.  The four
                // columns that get finished meanwhile wait in `held` and are written in the second
                // half of the round's third pair.
                const int nbr = a >> 4, slot0 = 16 * (p - 8 * nbr);   // round, first slot of the pair in it
#pragma unroll
                for (int k = 0; k < 16; ++k) {
                    if (cur) {
                        if (k < 4) S1(A, a, k);
                        else if (k < 8) S1(B, b, k - 4);
                        else if (k < 12) S2(A, k - 8);
                        else S2(B, k - 12);
                    }
                    // work of the pair before: the rest of its conversions and its LDS writes
                    if (prev) {
                        if (k == 0) { C2(PA, 4); C2(PA, 5); C2(PA, 6); }
                        if (k == 1) { C2(PA, 7); WR(PA, a - 2, 0); WR(PA, a - 2, 1); }
                        if (k == 2) { C2(PB, 0); C2(PB, 1); C2(PB, 2); }
                        if (k == 3) { C2(PB, 3); C2(PB, 4); C2(PB, 5); }
                        if (k == 4) { C2(PB, 6); C2(PB, 7); }
                        if (k == 5) { WR(PB, b - 2, 0); WR(PB, b - 2, 1); }
                    }
                    if (cur) {
                        if (k == 4) LD(a + LA, 0);
                        if (k == 5) LD(a + LA, 1);
                        if (k == 6) { C1(A, 0); C1(A, 1); C1(A, 2); }
                        if (k == 7) { C1(A, 3); C1(A, 4); C1(A, 5); }
                        if (k == 8) { C1(A, 6); C1(A, 7); LD(b + LA, 0); }
                        if (k == 9) { LD(b + LA, 1); C1(B, 0); C1(B, 1); }
                        if (k == 10) { C1(B, 2); C1(B, 3); C1(B, 4); }
                        if (k == 11) { C1(B, 5); C1(B, 6); C1(B, 7); }
                        if (k == 12) { C2(A, 0); C2(A, 1); C2(A, 2); }
                        if (k == 13) C2(A, 3);
                        // stage 0 of W behind the first round's columns: one piece per pair
                        if (k == 14 && p >= 4 && p < 12) w_issue(0, 0, p - 4);
                        const int at = slot0 + k;
                        if (nbr > 0 && at >= 6 && at < 6 + RPR) read_back(nbr - 1, at - 6, 1);
                        if (nbr > 0 && at >= 40 && at < 48) {
                            const int jj = (at - 40) >> 1, t = (at - 40) & 1;
                            *reinterpret_cast<V8*>(lds + area_at(t, (uint32_t)jj) + ((lane ^ (uint32_t)jj) << 4)) = held[jj][t];
                        }
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        } else {
    #pragma unroll
            for (int c = 0; c < TOTAL; ++c) {
                const int nb = c >> 4, j = c & 15;
                V8 out[NH];
                if constexpr (K == 1024) {
                    column_transform<T16>(in[j][0], in[j][1], po, out[0], out[1]);
                } else {
                    f32x4 t2[2];
                    tile_transform<T16>(in[j][0], ops, t2);
    #pragma unroll
                    for (int t = 0; t < 2; ++t)
    #pragma unroll
                        for (int r = 0; r < 4; ++r) out[0][4 * t + r] = (E)t2[t][r];
                }
                if (c + 16 < TOTAL) load_col(c + 16);
                if (c >= 8 && c < 16) w_issue(0, 0, c - 8);  // stage 0, behind the first round's columns
                if (nb > 0 && j < 4) {
                    read_back(nb - 1, j * (RPR / 4), RPR / 4);
    #pragma unroll
                    for (int t = 0; t < NH; ++t) held[j][t] = out[t];
                    if (j == 3) {
    #pragma unroll
                        for (int jj = 0; jj < 4; ++jj) write_col(nb, jj, held[jj]);
                    }
                } else {
                    write_col(nb, j, out);
                }
            }
        }
        read_back(NBF - 1, 0, RPR);
        // This wavefront's reads have returned: its rows of stage buffers 1 .. 3 are free, and it
        // requests its pieces of the stages the main loop expects to be in flight.
        wait_lds();
#pragma unroll
        for (int g = 1; g < AHEAD; ++g)
#pragma unroll
            for (int i = 0; i < 8; ++i) w_issue(g, g, i);
    }

    // Stage 0 has landed (the 8 (AHEAD - 1) pieces behind it may still be in flight) and every
    // wavefront has finished with its area.
    wait_vm(8 * (AHEAD - 1));
    __builtin_amdgcn_s_barrier();

    // Fragment of row block mb, K step ks of a stage: row 16 mb + lo, chunk 4 ks + hi.  In the
    // swizzled image that is (lane part) ^ (ks << 6) plus 8 KB per mb (frag_lane_offset), so one
    // vector instruction per K step makes the address and the four reads differ by the constant in
    // their offset field (which reaches 64 KB: buffers 2 and 3 have a lane part of their own).
    // The instruction is opaque on purpose: left to itself the compiler keeps all the addresses of
    // a stage in registers for the whole kernel, which this kernel does not have.
    // (The dynamic LDS of these kernels starts at a multiple of 512, which the XOR relies on.)
    const uint32_t frag_lane_lo = lds_base + frag_lane_offset(lo, hi);
    const uint32_t frag_lane_hi = frag_lane_lo + 2u * kStageBytes;
    auto frag_addr = [&](int slot, int ks) __attribute__((always_inline)) -> uint32_t {
        uint32_t a;
        asm volatile("v_xor_b32 %0, %2, %1" : "=v"(a) : "v"(slot >= 2 ? frag_lane_hi : frag_lane_lo), "i"(ks << 6));
        return a;
    };
    auto frag_read = [&](V8& dst, uint32_t a, int slot, int mb) __attribute__((always_inline)) {
        lds_read16(dst, a, (slot & 1) * kStageBytes + mb * 8192);
    };
    V8 fr[4][4];  // [K step % 4][mb]
    {
        const uint32_t a0 = frag_addr(0, 0), a1 = frag_addr(0, 1);
#pragma unroll
        for (int mb = 0; mb < 4; ++mb) frag_read(fr[0][mb], a0, 0, mb);
#pragma unroll
        for (int mb = 0; mb < 4; ++mb) frag_read(fr[1][mb], a1, 0, mb);
    }

    // ---- output addressing ------------------------------------------------------------------------
    // lane (hi, lo) of a row block owns rows 16 mb + 4 hi + r and the NBF adjacent columns
    // NBF lo .. NBF lo + NBF - 1 of its wavefront's columns
    constexpr uint32_t esize = OUT_F32 ? 4u : 2u;
    const uint32_t col = n0 + CPW * wave + (uint32_t)NBF * lo;
    const uint32_t lane_off = (4u * hi * N + col) * esize;  // inside the row block, < 2^32
    unsigned char* const Cb = static_cast<unsigned char*>(C);
    // `mult` is the part of the scale that is not a power of two (1 for K = 1024 and the usual
    // n^-1/2, sqrt(2)-ish for K = 512); it is applied to the fp32 result at the store.  Row blocks
    // of full column groups take the vector store path.
    const bool cols_full = n0 + kCols <= N && (N % (uint32_t)NBF) == 0;

    // one store of the interleaved epilogue: rows 16 mb + 4 hi + r of a full row block
    auto store_pair = [&](const f32x4 (&acc)[4][NBF], uint64_t block_base, int mb, int r)
        __attribute__((always_inline)) {
        // streaming stores: C is not read again, and keeping it out of the L2 leaves the cache to
        // the operands
        unsigned char* row_ptr = Cb + (block_base + (uint64_t)((16u * mb + r) * N) * esize);  // scalar
        if constexpr (NBF == 2) {
            const float v0 = acc[mb][0][r] * mult, v1 = acc[mb][1][r] * mult;
            if (OUT_F32)
                stream_store8(lane_off, u32x2{__builtin_bit_cast(uint32_t, v0), __builtin_bit_cast(uint32_t, v1)}, row_ptr);
            else
                stream_store4(lane_off, __builtin_bit_cast(uint32_t, V2{(E)v0, (E)v1}), row_ptr);
        } else {
            const float v0 = acc[mb][0][r] * mult, v1 = acc[mb][1][r] * mult, v2 = acc[mb][2][r] * mult,
                        v3 = acc[mb][3][r] * mult;
            if (OUT_F32)
                stream_store16(lane_off, u32x4{__builtin_bit_cast(uint32_t, v0), __builtin_bit_cast(uint32_t, v1),
                                               __builtin_bit_cast(uint32_t, v2), __builtin_bit_cast(uint32_t, v3)}, row_ptr);
            else
                stream_store8(lane_off, __builtin_bit_cast(u32x2, V4{(E)v0, (E)v1, (E)v2, (E)v3}), row_ptr);
        }
    };
    // the same for a row block at the edge of the matrix (masked, element by element)
    auto store_edge = [&](const f32x4 (&acc)[4][NBF], uint32_t row_base) __attribute__((always_inline)) {
#pragma unroll
        for (int mb = 0; mb < 4; ++mb)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const uint32_t row = row_base + 16u * mb + 4u * hi + r;
                if (row >= m_end) continue;
#pragma unroll
                for (int nb = 0; nb < NBF; ++nb) {
                    if (col + nb >= N) continue;
                    const float v = acc[mb][nb][r] * mult;
                    const uint64_t at = (uint64_t)row * N + col + nb;
                    if (OUT_F32)
                        static_cast<float*>(C)[at] = v;
                    else
                        static_cast<E*>(C)[at] = (E)v;
                }
            }
    };

    // ---- one row block: KSTEPS K steps into `acc`, while `prev` (the previous row block's result,
    // when the tag says there is one) is stored one piece behind each MFMA of the K steps that follow
    // the first stage's barrier.  `second_tag`: the block is the second of its pair, whose stages
    // continue the ring where the first block's stopped (buffer (SPB + kq) % 4). -------------------
    // `last_tag`: nothing follows the block, so it requests only its own remaining stages.  A tag
    // rather than a run-time condition: a branch around a transfer costs the wavefront its
    // instruction prefetch, and masking the transfer off through EXEC costs as much as the transfer
    // (measured: 13 cycles of the MFMA stream each, 192 times per workgroup at the headline shape).
    auto row_block_body = [&](auto prev_tag, auto second_tag, auto last_tag, f32x4 (&acc)[4][NBF],
                              const f32x4 (&prev)[4][NBF], uint64_t prev_base, uint32_t rbi)
        __attribute__((always_inline)) {
        constexpr bool prev_full = decltype(prev_tag)::value;
        constexpr int slot_base = decltype(second_tag)::value ? (SPB & 3) : 0;
        constexpr bool last = decltype(last_tag)::value;
#pragma unroll
        for (int kq = 0; kq < SPB; ++kq) {
            // pieces of stage g+AHEAD issued during K step ks of this stage (everything below folds to
            // constants once the loops are unrolled)
            constexpr int kPieceAt[7] = {0, 2, 4, 5, 6, 7, 8};
            const int cur_slot = (slot_base + kq) & 3;
            const int next_slot = (slot_base + kq + 1) & 3;
            const int fill_slot = (slot_base + kq + AHEAD) & 3;
            const int fill_kq = (kq + AHEAD) % SPB;
            const bool fill_own_block = kq + AHEAD < SPB;
#pragma unroll
            for (int ks = 0; ks < kStepsPerStage; ++ks) {
                const int kk = kq * kStepsPerStage + ks;
                // This step's fragments were requested two steps ago; the four of the step between
                // are the only younger reads.
                wait_lds_all_but<4>();
                // fragments two K steps ahead; the last two steps of a stage read the first two of
                // the next stage, behind the barrier
                const int read_slot = ks < 6 ? cur_slot : next_slot;
                const uint32_t fa = frag_addr(read_slot, (ks + 2) & 7);
#pragma unroll
                for (int m = 0; m < NM; ++m) {
                    const int mb = m / NBF, nb = m % NBF;
                    // up to two transfer pieces per K step, behind MFMAs 4 and 6; the LDS target
                    // goes into M0 in front of the MFMA, the transfer follows it
                    const int piece = m == 4 ? 0 : (m == 6 ? 1 : -1);
                    const int pi = piece >= 0 && piece < 2 && ks < 6 ? kPieceAt[ks] + piece : 99;
                    const bool transfer = pi < kPieceAt[ks < 6 ? ks + 1 : 6] && (fill_own_block || !last);
                    if (transfer) {
                        // from the first stage whose transfers belong to the next row block on, the
                        // lane offsets are the next block's: each is replaced right before its first
                        // such use (three vector instructions in the shadow of the MFMA before)
                        if (kq == SPB - AHEAD) set_voff_piece(rbi + 1u, pi);
                        w_target(fill_slot, pi);
                    }
                    if (kk == 0)
                        XMfma<T16>::first(acc[mb][nb], fr[ks & 3][mb], yf[nb][0]);
                    else
                        XMfma<T16>::next(acc[mb][nb], fr[ks & 3][mb], yf[nb][kk]);
                    // memory instructions in the shadow of the MFMA
                    if (m < 4) frag_read(fr[(ks + 2) & 3][m], fa, read_slot, m);
                    if (transfer) w_go(fill_kq, pi);
                    // the previous block's sixteen stores, one per K step behind its last MFMA,
                    // from the K step after the first stage's barrier on (a store costs the MFMA
                    // stream about 16 cycles; two in a row cost more than twice that)
                    if (prev_full && kk >= 6 && kk < 22 && m == NM - 1) {
                        const int e = kk - 6;
                        store_pair(prev, prev_base, e >> 2, e & 3);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
                // The matrix core reads its 128-bit A operand over several cycles after issue, and
                // the compiler, which sees an opaque statement, would hand a fragment register to a
                // temporary right behind the last MFMA that uses it (observed: a v_mov one
                // instruction later corrupted the product).  Naming the previous step's fragments
                // here keeps all four fragment sets allocated for the whole loop.
                asm volatile("" ::"v"(fr[(ks + 3) & 3][0]), "v"(fr[(ks + 3) & 3][1]),
                             "v"(fr[(ks + 3) & 3][2]), "v"(fr[(ks + 3) & 3][3]));
                if (ks == 5) {
                    // Own pieces of stage g+1 have landed.  Loads complete in order among
                    // themselves, but not relative to stores, so the count allowed to remain
                    // outstanding is the number of *loads* requested after those pieces (8 per
                    // stage g+2 .. g+AHEAD; fewer at the end of the last row block): pending
                    // stores can only make this wait longer, never shorter.
                    const int later = SPB - kq - 2 < AHEAD - 1 ? SPB - kq - 2 : AHEAD - 1;
                    const int after_last = kq == SPB - 1 ? -1 : 8 * (later > 0 ? later : 0);
                    wait_vm(last ? after_last : 8 * (AHEAD - 1));
                    wait_lds();
                    __builtin_amdgcn_s_barrier();
                }
            }
        }
        // Control leaves this variant of the block with the fragments of the next block's first
        // two K steps requested.  The variants need not agree on which registers hold the fragment
        // ring, so the compiler may copy fragment registers on the edge between two of them, and
        // a copy reads its source at once: the reads must have landed before the edge (the last
        // of them was issued NM - 4 MFMAs ago).  The build checks the generated ISA for this
        // (build.py: check_lds_reads_waited_for).
        wait_lds();
    };

    auto store_block = [&](f32x4 (&acc)[4][NBF], uint64_t base) __attribute__((always_inline)) {
        drain_mfma(acc);
#pragma unroll
        for (int mb = 0; mb < 4; ++mb)
#pragma unroll
            for (int r = 0; r < 4; ++r) store_pair(acc, base, mb, r);
    };
    auto block_place = [&](uint32_t rbi, bool& full, uint64_t& base, uint32_t& row_base)
        __attribute__((always_inline)) {
        row_base = m_begin + row_block(rbi) * kRows;
        full = cols_full && row_base + kRows <= m_end;
        base = (uint64_t)row_base * N * esize;
    };
    if constexpr (NBF <= 2) {
        // Two accumulator sets take turns: a finished full block is stored during the next one.
        static_assert(KSTEPS >= 22, "the sixteen stores take K steps 6 .. 21 of the next block");
        f32x4 accA[4][NBF], accB[4][NBF];
        bool pend = false;        // accB holds a finished full row block that is not stored yet
        uint64_t pend_base = 0;
        auto run = [&](bool prev_full, auto second_tag, f32x4 (&acc)[4][NBF], const f32x4 (&prev)[4][NBF],
                       uint64_t prev_base, uint32_t rbi) __attribute__((always_inline)) {
            const bool last = rbi + 1u == nrb;
            if (prev_full && last)
                row_block_body(std::true_type{}, second_tag, std::true_type{}, acc, prev, prev_base, rbi);
            else if (prev_full)
                row_block_body(std::true_type{}, second_tag, std::false_type{}, acc, prev, prev_base, rbi);
            else if (last)
                row_block_body(std::false_type{}, second_tag, std::true_type{}, acc, prev, prev_base, rbi);
            else
                row_block_body(std::false_type{}, second_tag, std::false_type{}, acc, prev, prev_base, rbi);
        };
        auto finish = [&](f32x4 (&acc)[4][NBF], uint32_t rbi, bool& full, uint64_t& base)
            __attribute__((always_inline)) {
            // a full block is stored during the next block; an edge block right away
            uint32_t row_base;
            block_place(rbi, full, base, row_base);
            if (!full) {
                drain_mfma(acc);
                store_edge(acc, row_base);
            }
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
    } else {
        // Four column fragments: one accumulator set is all the register file has room for (a
        // second one spilled), so a block is stored as soon as it is finished; with sixteen MFMAs
        // per K step the sixteen stores and the drain cost a few per cent of a block.
        f32x4 acc[4][NBF];
        auto one = [&](auto second_tag, uint32_t rbi) __attribute__((always_inline)) {
            if (rbi + 1u == nrb)
                row_block_body(std::false_type{}, second_tag, std::true_type{}, acc, acc, 0, rbi);
            else
                row_block_body(std::false_type{}, second_tag, std::false_type{}, acc, acc, 0, rbi);
            bool full;
            uint64_t base;
            uint32_t row_base;
            block_place(rbi, full, base, row_base);
            if (full) {
                store_block(acc, base);
            } else {
                drain_mfma(acc);
                store_edge(acc, row_base);
            }
        };
#pragma unroll 1
        for (uint32_t rbi = 0; rbi < nrb; rbi += 2u) {
            one(std::false_type{}, rbi);
            if (rbi + 1u < nrb) one(std::true_type{}, rbi + 1u);
        }
    }
    // Every transfer into LDS was waited for at the barrier of the stage before the one that read
    // it, so none is in flight when the workgroup's LDS is released.
}

template <class T16, int K, bool OUT_F32>
int launch_as(const void* W, const void* Xt, void* C, uint32_t M, uint32_t N, float scale, hipStream_t s)
{
    const OutputScale os =
        split_output_scale((double)scale, tile_stage_shift<2>(ilog2((uint32_t)K), kNarrowRange<T16>));
    const Plan p = plan16(M, N, (uint32_t)K);
    auto kern = fused_ht_gemm_xreg_kernel<T16, K, OUT_F32>;
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                            hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes) != hipSuccess)
        return MI_ERR_LAUNCH;
    hipLaunchKernelGGL(kern, dim3(p.grid), dim3(kThreads), kLdsBytes, s,
                       static_cast<const typename T16::E*>(W),
                       static_cast<const typename T16::E*>(Xt), C, M, N, p.m_per_block, p.msplit, p.mpx,
                       p.cgx, p.nrect, os.exp2, os.mult);
    return launch_status();
}

template <class T16, int K>
int launch(const void* W, const void* Xt, void* C, uint32_t M, uint32_t N, int out_f32, float scale,
           hipStream_t s)
{
    return out_f32 ? launch_as<T16, K, true>(W, Xt, C, M, N, scale, s)
                   : launch_as<T16, K, false>(W, Xt, C, M, N, scale, s);
}

}  // namespace xreg

// K = 2048 and 4096: fused_gemm_xreg_k2048.hip
int fused_gemm16_xreg_k2048(const void* W, const void* Xt, void* C, uint32_t M, uint32_t N, uint32_t K,
                            int in_dtype, int out_f32, float scale, hipStream_t s);

// Called by the dispatcher of mi_fused_ht_gemm for K = 512 ... 4096 (arguments already validated
// there).
int fused_gemm16_xreg(const void* W, const void* Xt, void* C, uint32_t M, uint32_t N, uint32_t K,
                      int in_dtype, int out_f32, float scale, hipStream_t s)
{
    // W and a row block of C are addressed with 32-bit byte offsets
    if ((uint64_t)M * K * 2u > 0xffffffffull || (uint64_t)N * 4u * 64u > 0xffffffffull)
        return MI_ERR_SHAPE;
    if (K == 1024u) {
        if (in_dtype == MI_BF16) return xreg::launch<BF16, 1024>(W, Xt, C, M, N, out_f32, scale, s);
        if (in_dtype == MI_F16) return xreg::launch<F16, 1024>(W, Xt, C, M, N, out_f32, scale, s);
    } else if (K == 512u) {
        if (in_dtype == MI_BF16) return xreg::launch<BF16, 512>(W, Xt, C, M, N, out_f32, scale, s);
        if (in_dtype == MI_F16) return xreg::launch<F16, 512>(W, Xt, C, M, N, out_f32, scale, s);
    } else if (K == 2048u || K == 4096u) {
        return fused_gemm16_xreg_k2048(W, Xt, C, M, N, K, in_dtype, out_f32, scale, s);
    } else {
        return MI_ERR_SIZE;
    }
    return MI_ERR_DTYPE;
}

}  // namespace mi

extern "C" int mi_debug_fused_gemm_tiling(uint32_t M, uint32_t N, uint32_t K, uint32_t* header,
                                          uint32_t* tiles, uint32_t capacity)
{
    using namespace mi;
    if (!header) return MI_ERR_NULL;
    if (M == 0 || N == 0) return MI_ERR_SHAPE;
    if (K != 512u && K != 1024u && K != 2048u && K != 4096u) return MI_ERR_SIZE;
    const xreg::Plan p = xreg::plan16(M, N, K);
    const uint32_t h[8] = {p.ngroups, p.msplit, p.m_per_block, p.mpx, p.cgx, p.nrect, p.grid, 0u};
    for (int i = 0; i < 8; ++i) header[i] = h[i];
    if (!tiles) return MI_OK;
    if (capacity < p.grid) return MI_ERR_SIZE;
    for (uint32_t id = 0; id < p.grid; ++id) {
        uint32_t cg = 0xffffffffu, ms = 0xffffffffu;
        if (!xreg::tile_of_workgroup(id, p.msplit, p.mpx, p.cgx, p.nrect, cg, ms)) cg = ms = 0xffffffffu;
        tiles[2u * id] = cg;
        tiles[2u * id + 1u] = ms;
    }
    return MI_OK;
}
