// Fused Hadamard -> GEMM with the transformed operand held in registers, gfx950, 16-bit inputs,
// K = 2048 (and K = 4096 as two passes over 2048 k each, the second adding to what the first
// stored), with the K range split over pairs of wavefronts:
//     C[M,N] = W[M,K] * (scale * H_K * X[K,N]),  X given as Xt[N,K].
//
// A wavefront's 256 accumulation registers hold 32768 16-bit values.  With all of K = 2048 per
// wavefront that is 16 columns: every W fragment read from LDS then feeds one MFMA, and the LDS
// (16 KB of fragment reads per K step of four MFMAs) bounds the loop at half the matrix-core rate.
// Here wavefront (cs, kp) = (wave / 2, wave % 2) holds half kp of the K range of 32 columns (the
// geometry of the K = 1024 kernel of fused_gemm_xreg.hip: two MFMAs per fragment):
//     H_2048 x = [Ya + Yb; Ya - Yb],  Ya, Yb = the 1024-point transforms of the halves of x.
// W is streamed as two streams (k < 1024 and k >= 1024), each through its own ring of four 16 KB
// stages (64 rows x 128 k; a stage is four K steps); a wavefront reads the fragments of its own
// stream only.  At the end of a row block each wavefront of a pair hands the partner the
// accumulators of two of the four 16-row fragments through LDS and finishes (adds, stores) the
// other two (a sum of two terms: the result does not depend on who adds); that meeting is hidden
// behind the MFMAs of the next row block.
// The prologue is shared inside a pair: in each of four rounds the pair transforms eight columns of
// its set, all of K (four columns per wavefront), and writes both halves into the pair's LDS area;
// after a barrier each wavefront reads its own half of the eight columns in operand order (the half
// of the lanes whose columns these are).  The area is the ring's fourth buffers plus the 32 KB behind
// the ring, so the first three stage times of W are on their way meanwhile.
//
// Main-loop statements are the hand-placed single instructions of xreg_common.hpp (see the
// K = 1024 kernel for the reasons).
//
// Behaviour replaced: fused_ht_gemm_pipelined, fused_ht/fusion_pipelined.cu:306-563.
#include <type_traits>

#include "xreg_common.hpp"
#include "xreg_mfma16.hpp"

namespace mi {
namespace xreg {
namespace k2h {

constexpr int kStage = 16 * 1024;  // 64 rows x 256 B (128 k)
constexpr int kSteps = 4;          // K steps of 32 per stage
constexpr int SPB = 8;             // stages per row block and stream
constexpr int AHEAD = 3;
constexpr int KSTEPS = 32;         // K steps per row block and wavefront
// Ring: buffer b (= stage % 4) of stream t at (4 t + b) kStage (fragment reads reach every buffer of
// a stream with a 16-bit offset).  Behind the ring 32 KB.  The prologue's area, four blocks
// [8 columns][2 KB], one per column set and K half, is the fourth buffer of either stream (set 0) and
// those 32 KB (set 1); later the 32 KB hold the hand-over buffers [wavefront][4 KB].
constexpr uint32_t kRegionBase = 8 * kStage;
static_assert(kRegionBase + 32 * 1024 == (uint32_t)kLdsBytes, "ring and the 32 KB behind it fill the 160 KB");
static_assert(8 * 2048 == kStage, "an area block is a stage buffer");
__host__ __device__ constexpr uint32_t area_block(uint32_t cs, uint32_t half)
{
    return cs ? kRegionBase + half * (uint32_t)kStage : (3u + 4u * half) * (uint32_t)kStage;
}

// LDS image of a stage: [64 rows][256 B], the 16-byte chunk q of row r stored at q ^ (r & 15)
__host__ __device__ constexpr uint32_t stage_offset(uint32_t row, uint32_t q)
{
    return row * 256u + ((q ^ (row & 15u)) << 4);
}
// lane part of a fragment address (row lo, chunk hi): the fragment of row block mb and K step ks of
// the stage is at (frag_lane ^ (ks << 6)) + 4096 mb
__host__ __device__ constexpr uint32_t frag_lane(uint32_t lo, uint32_t hi) { return lo * 256u + ((hi ^ lo) << 4); }
// a half's eight columns in the prologue area: [8 columns][128 chunks], chunk q of column c stored
// at q ^ c; for q = 4 s + hi that is area_read_base(c, hi) + 64 (s ^ (c / 4))
__host__ __device__ constexpr uint32_t area_offset(uint32_t c, uint32_t q) { return c * 2048u + ((q ^ c) << 4); }
__host__ __device__ constexpr uint32_t area_read_base(uint32_t c, uint32_t hi)
{
    return c * 2048u + ((hi ^ (c & 3u)) << 4);
}
constexpr bool patterns_ok()
{
    for (uint32_t lane = 0; lane < 64; ++lane)
        for (uint32_t mb = 0; mb < 4; ++mb)
            for (uint32_t ks = 0; ks < 4; ++ks)
                if ((frag_lane(lane & 15u, lane >> 4) ^ (ks << 6)) + 4096u * mb !=
                    stage_offset(16u * mb + (lane & 15u), 4u * ks + (lane >> 4)))
                    return false;
    for (uint32_t mb = 0; mb < 4; ++mb)
        for (uint32_t ks = 0; ks < 4; ++ks)
            if (!lds::conflict_free_b128(
                    [=](uint32_t lane) { return stage_offset(16u * mb + (lane & 15u), 4u * ks + (lane >> 4)); }))
                return false;
    for (uint32_t c = 0; c < 8; ++c)
        for (uint32_t hi = 0; hi < 4; ++hi)
            for (uint32_t s = 0; s < 32; ++s)
                if (area_read_base(c, hi) + 64u * (s ^ (c >> 2)) != area_offset(c, 4u * s + hi)) return false;
    // every lane writes chunk 64 t + lane of a column; in rounds 2 h, 2 h + 1 the lanes with
    // lo / 8 == h read chunk 4 s + hi of column lo % 8
    for (uint32_t c = 0; c < 8; ++c)
        for (uint32_t t = 0; t < 2; ++t)
            if (!lds::conflict_free_b128([=](uint32_t lane) { return area_offset(c, 64u * t + lane); })) return false;
    for (uint32_t h = 0; h < 2; ++h)
        for (uint32_t s = 0; s < 32; ++s)
            if (!lds::conflict_free_b128_masked(
                    [=](uint32_t lane) { return area_offset(lane & 7u, 4u * s + (lane >> 4)); },
                    [=](uint32_t lane) { return ((lane & 15u) >> 3) == h; }))
                return false;
    return true;
}
static_assert(patterns_ok(), "an LDS access pattern of the split-K 16-bit kernel would serialise");

}  // namespace k2h

// KTOT = 2048: the whole contraction.  KTOT = 4096: one of two passes; pass 0 (ACCUM = false)
// contracts W[:, :2048] with the first half of H_4096 x = [H_2048 a + H_2048 b; H_2048 a - H_2048 b]
// (a, b the halves of a column) and stores, pass 1 (ACCUM = true) contracts W[:, 2048:] with the
// second half and adds to what pass 0 stored.
template <class T16, bool OUT_F32, int KTOT, bool ACCUM>
__global__ void __launch_bounds__(kThreads)
fused_ht_gemm_xreg_k2048_kernel(const typename T16::E* __restrict__ W, const typename T16::E* __restrict__ Xt,
                                void* __restrict__ C, uint32_t M, uint32_t N, uint32_t m_per_block,
                                uint32_t msplit, uint32_t mpx, uint32_t cgx, uint32_t nrect, int exp2,
                                float mult)
{
    using E = typename T16::E;
    using V8 = typename T16::V8;
    typedef E V2 __attribute__((ext_vector_type(2)));
    static_assert(KTOT == 2048 || KTOT == 4096, "K = 2048, or one half of K = 4096");
    static_assert(KTOT == 4096 || !ACCUM, "a single pass stores");
    constexpr int K = KTOT, NBF = 2, NM = 8;  // K: row length of W and Xt
    constexpr int SPB = k2h::SPB, AHEAD = k2h::AHEAD, KSTEPS = k2h::KSTEPS;
    constexpr uint32_t kCols = 64;
    constexpr uint32_t ROW_BYTES = K * 2u;

    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t cs = wave >> 1, kp = wave & 1u;  // column set, K half
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
    const unsigned char* Wb = reinterpret_cast<const unsigned char*>(W) + (ACCUM ? 4096u : 0u);  // the pass's 2048 k
    const uint32_t lds_base = (uint32_t)(uintptr_t)(lptr_t)lds;
    const uint32_t lrow = lane >> 4, lq = lane & 15u;
    uint32_t voff[4];  // lane offset of rows 4 j .. 4 j + 3 (the second stream's 2048 bytes go into the scalar base)
    auto set_voff_piece = [&](uint32_t rbi, int j) __attribute__((always_inline)) {
        const uint32_t r0 = m_begin + row_block(rbi) * kRows + 16u * wave + lrow;
        voff[j] = min(r0 + 4u * j, M - 1u) * ROW_BYTES + ((lq ^ (4u * j + lrow)) << 4);
    };
    const uint32_t lds_wave_base = lds_base + 16u * wave * 256u;  // this wavefront's rows of a stage
    auto lds_piece = [](int kq, int i) constexpr { return ((i >> 2) * 4 + (kq & 3)) * k2h::kStage + 4 * (i & 3) * 256; };
    auto w_base = [&](int kq, int i) __attribute__((always_inline)) { return Wb + (kq * 256 + (i >> 2) * 2048); };
    auto w_issue = [&](int kq, int i) __attribute__((always_inline)) {
        global_to_lds16(voff[i & 3], w_base(kq, i), lds_wave_base, lds_piece(kq, i));
    };
#pragma unroll
    for (int j = 0; j < 4; ++j) set_voff_piece(0, j);

    // ---- prologue: column nb of lane (., lo) = column n0 + 32 cs + 2 lo + nb, its half kp -------------
    // Round R = 2 h + nb: the set's columns 2 (8 h + i) + nb, i = 0 .. 7; wavefront kp of the pair
    // transforms i = 4 kp .. 4 kp + 3, and the lanes with lo / 8 == h read back column i = lo % 8.
    V8 yf[NBF][KSTEPS];
    {
        PairOperands<T16> po;
        make_pair_operands<T16>(po, exp2);
        // The first three stage times of W go out before any X: vector memory operations complete in
        // order and the compiler's waits for X count only the loads it knows of, so a transfer
        // requested between two X tiles would be waited for with the older tile.
#pragma unroll
        for (int pc = 0; pc < 8 * AHEAD; ++pc) w_issue(pc >> 3, pc & 7);
        // X tiles are requested kAhead columns before their use (a round at K = 2048)
        constexpr int NT = KTOT / 512, kAhead = 16 / NT;
        V8 in[kAhead][NT];  // [column of the wavefront % kAhead][tile]
        auto load_col = [&](int c) {  // the wavefront's column c = 4 R + jj
            const uint32_t i = 4u * kp + (uint32_t)(c & 3);
            const uint32_t col = min(n0 + 32u * cs + 2u * (8u * (uint32_t)(c >> 3) + i) + (uint32_t)((c >> 2) & 1), N - 1u);
#pragma unroll
            for (int t = 0; t < NT; ++t)
                in[c % kAhead][t] = *reinterpret_cast<const V8*>(Xt + ((uint64_t)col * K + 512u * t + 8u * lane));
        };
#pragma unroll
        for (int c = 0; c < kAhead; ++c) load_col(c);
        const uint32_t cl = lo & 7u;
        const unsigned char* const src = lds + k2h::area_block(cs, kp) + k2h::area_read_base(cl, hi);
        const unsigned char* const src_even = src + 64u * (cl >> 2);  // K step s: + 64 (s ^ (cl / 4))
        const unsigned char* const src_odd = src - 64u * (cl >> 2);
#pragma unroll
        for (int R = 0; R < 4; ++R) {
            if (R > 0) {  // the partner has read the previous round's columns
                wait_lds();
                __builtin_amdgcn_s_barrier();
            }
#pragma unroll
            for (int jj = 0; jj < 4; ++jj) {
                const int c = 4 * R + jj, e = c % kAhead;
                // the lane's eight values of each k quarter of the 2048 transformed values this
                // pass keeps, [quarter][4 h .. 4 h + 3]
                f32x4 qv[4][2];
                {
                    // A, B: the 1024-point transforms of the two halves of the 2048 values this pass
                    // keeps (K = 4096: of x[0:2048] +- x[2048:4096], H_2048 being linear)
                    f32x4 sa[2], da[2], sb[2], db[2];
                    if constexpr (KTOT == 4096) {
                        column_pair_combined_f32<T16, ACCUM>(in[e][0], in[e][1], in[e][4], in[e][5], po, sa, da);
                        column_pair_combined_f32<T16, ACCUM>(in[e][2], in[e][3], in[e][6], in[e][7], po, sb, db);
                    } else {
                        column_pair_f32<T16>(in[e][0], in[e][1], po, sa, da);
                        column_pair_f32<T16>(in[e][2], in[e][3], po, sb, db);
                    }
#pragma unroll
                    for (int h = 0; h < 2; ++h) {  // A_lo + B_lo, A_hi + B_hi, A_lo - B_lo, A_hi - B_hi
                        qv[0][h] = sa[h] + sb[h];
                        qv[1][h] = da[h] + db[h];
                        qv[2][h] = sa[h] - sb[h];
                        qv[3][h] = da[h] - db[h];
                    }
                }
                if (c + kAhead < 16) load_col(c + kAhead);
                // (the loads stay here, kAhead columns ahead of their use)
                __builtin_amdgcn_sched_barrier(0);
                V8 o[4];
#pragma unroll
                for (int q = 0; q < 4; ++q)
#pragma unroll
                    for (int h = 0; h < 2; ++h)
#pragma unroll
                        for (int el = 0; el < 4; ++el) o[q][4 * h + el] = (E)qv[q][h][el];
#pragma unroll
                for (int q = 0; q < 4; ++q)  // quarter q = half q / 2, chunks 64 (q % 2) + lane of it
                    *reinterpret_cast<V8*>(lds + k2h::area_block(cs, q >> 1) +
                                           k2h::area_offset(4u * kp + (uint32_t)jj, 64u * (q & 1) + lane)) = o[q];
            }
            wait_lds();
            __builtin_amdgcn_s_barrier();
            if ((int)(lo >> 3) == (R >> 1)) {
#pragma unroll
                for (int s = 0; s < KSTEPS; ++s)
                    yf[R & 1][s] = *reinterpret_cast<const V8*>(((s & 1) ? src_odd : src_even) + 64u * s);
            }
        }
    }
    // stage 0 of W has landed (stages 1 and 2 are younger), everybody is done with the area: its
    // part inside the ring can take the first half of stage 3
    wait_vm(8 * (AHEAD - 1));
    wait_lds();
    __builtin_amdgcn_s_barrier();
#pragma unroll
    for (int i = 0; i < 4; ++i) w_issue(AHEAD, i);

    // ---- fragments of this wavefront's stream ----------------------------------------------------
    // Wavefront (cs, kp) takes the block's four row fragments in the order 2 kp, 2 kp + 1, then the
    // other two: accumulators 0 and 1 are the ones it finishes, 2 and 3 the ones it hands over.
    const uint32_t frag_lane = lds_base + kp * 4u * k2h::kStage + k2h::frag_lane(lo, hi);
    const uint32_t frag_lane_own = frag_lane + kp * 8192u, frag_lane_other = frag_lane - kp * 8192u;
    auto frag_addr = [&](uint32_t lane_part, int ks) __attribute__((always_inline)) -> uint32_t {
        uint32_t a;
        asm volatile("v_xor_b32 %0, %2, %1" : "=v"(a) : "v"(lane_part), "i"(ks << 6));
        return a;
    };
    auto frag_read = [&](V8& dst, uint32_t a, int slot, int mb) __attribute__((always_inline)) {
        lds_read16(dst, a, slot * k2h::kStage + mb * 4096);
    };
    V8 fr[4][4];  // [K step % 4][mb]
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
        const uint32_t a_own = frag_addr(frag_lane_own, ks), a_other = frag_addr(frag_lane_other, ks);
#pragma unroll
        for (int mb = 0; mb < 4; ++mb) frag_read(fr[ks][mb], mb < 2 ? a_own : a_other, 0, mb);
    }

    // ---- output: wavefront (cs, kp) finishes rows 32 kp .. 32 kp + 31 of a block; lane (hi, lo) owns
    // rows 16 f + 4 hi + r of them in the adjacent columns n0 + 32 cs + 2 lo, + 1
    constexpr uint32_t esize = OUT_F32 ? 4u : 2u;
    const uint32_t col = n0 + 32u * cs + 2u * lo;
    const uint32_t lane_off = (4u * hi * N + col) * esize;  // inside the row block, < 2^32
    unsigned char* const Cb = static_cast<unsigned char*>(C);
    const bool cols_full = n0 + kCols <= N && (N & 1u) == 0u;
    // where the two K halves meet: 4 KB per wavefront, fragment i = 2 f + nb at 1024 i + 16 lane
    const uint32_t xb_mine = lds_base + k2h::kRegionBase + wave * 4096u + lane * 16u;
    const uint32_t xb_partner = lds_base + k2h::kRegionBase + (wave ^ 1u) * 4096u + lane * 16u;

    // Transfers: two pieces per K step (behind MFMAs 4 and 6), every K step.  The stage whose reads
    // end with the barrier of K step 1 is refilled from K step 2 on: during K steps 2, 3 of stage kq
    // the first four pieces of stage kq + 4 go out (into the buffer of stage kq), during K steps 0, 1
    // of stage kq + 1 its other four.  At the barrier of stage kq the pieces of stages kq + 2 and
    // kq + 3 are the sixteen youngest, so the wait for stage kq + 1 is the same constant everywhere.
    //
    // The halves of a finished block meet while the next block is being multiplied: two accumulator
    // sets take turns, the fragments to hand over are written to LDS behind the MFMAs of K step 0,
    // become visible with the stage barrier after K step 1, are read behind the MFMAs of K step 2,
    // added and scaled in K step 4 and stored one row per K step from K step 5 on.
    f32x4 acc[2][4][NBF];
    f32x4 out[2][NBF];  // the partner's partial sums, then the finished values
    uint64_t out_base = 0;
    auto store_out = [&](int f, int r) __attribute__((always_inline)) {
        unsigned char* row_ptr = Cb + (out_base + (uint64_t)((16u * f + r) * N) * esize);  // scalar
        const float v0 = out[f][0][r], v1 = out[f][1][r];
        if (ACCUM) {
            // second pass: every element has one owner and the first pass has completed, so the
            // addition needs no ordering; done in the L2, it spares the loop a wait for loaded values
            if (OUT_F32) {
                add_f32_to_memory(lane_off, v0, row_ptr, 0);
                add_f32_to_memory(lane_off, v1, row_ptr, 4);
            } else {
                XMfma<T16>::add_pair_to_memory(lane_off, __builtin_bit_cast(uint32_t, V2{(E)v0, (E)v1}), row_ptr);
            }
        } else if (KTOT == 4096) {
            // the second pass reads these lines back: no streaming hint (M = N = 8192: 510 -> 485 us)
            if (OUT_F32)
                cached_store8(lane_off, u32x2{__float_as_uint(v0), __float_as_uint(v1)}, row_ptr);
            else
                cached_store4(lane_off, __builtin_bit_cast(uint32_t, V2{(E)v0, (E)v1}), row_ptr);
        } else if (OUT_F32) {
            stream_store8(lane_off, u32x2{__float_as_uint(v0), __float_as_uint(v1)}, row_ptr);
        } else {
            stream_store4(lane_off, __builtin_bit_cast(uint32_t, V2{(E)v0, (E)v1}), row_ptr);
        }
    };
    auto row_block_body = [&](auto last_tag, auto pending_tag, auto set_tag, uint32_t rbi) __attribute__((always_inline)) {
        constexpr bool last = decltype(last_tag)::value;
        constexpr bool pending = decltype(pending_tag)::value;  // the previous block awaits its other half
        constexpr int cur = decltype(set_tag)::value, prev = cur ^ 1;
#pragma unroll
        for (int kq = 0; kq < SPB; ++kq) {
            // (everything below folds to constants once the loops are unrolled; SPB is a multiple of
            // 4, so stage kq of every row block lives in buffer kq % 4 of its stream)
            const int cur_slot = kq & 3, next_slot = (kq + 1) & 3;
#pragma unroll
            for (int ks = 0; ks < k2h::kSteps; ++ks) {
                const int kk = kq * k2h::kSteps + ks;
                // this step's fragments were requested two steps ago; the four of the step between
                // are the only younger reads (in K step 3 of a block also the four reads of the
                // partner's sums, which K step 4 then finds complete)
                wait_lds_all_but<4>();
                if (pending && kk == 4)
                    asm volatile("" : "+v"(out[0][0]), "+v"(out[0][1]), "+v"(out[1][0]), "+v"(out[1][1]));
                const int read_slot = ks < 2 ? cur_slot : next_slot;
                const uint32_t fa_own = frag_addr(frag_lane_own, (ks + 2) & 3);
                const uint32_t fa_other = frag_addr(frag_lane_other, (ks + 2) & 3);
                const int fill_stage = ks < 2 ? kq + AHEAD : kq + AHEAD + 1;  // may lie in the next row block
                const int fill_kq = fill_stage % SPB;
#pragma unroll
                for (int m = 0; m < NM; ++m) {
                    const int mb = m >> 1, nb = m & 1;
                    const int pi = (ks < 2 ? 4 : 0) + 2 * (ks & 1) + (m == 6 ? 1 : 0);
                    const bool transfer = (m == 4 || m == 6) && (fill_stage < SPB || !last);
                    if (transfer) {
                        // the lane offsets of the next row block replace this one's right before
                        // their first use (three vector instructions in the shadow of an MFMA)
                        if (fill_stage == SPB && pi < 4) set_voff_piece(rbi + 1u, pi);
                        lds_transfer_target(lds_wave_base, lds_piece(fill_kq, pi));
                    }
                    if (kk == 0)
                        XMfma<T16>::first(acc[cur][mb][nb], fr[ks & 3][mb], yf[nb][0]);
                    else
                        XMfma<T16>::next(acc[cur][mb][nb], fr[ks & 3][mb], yf[nb][kk]);
                    if (m < 4) frag_read(fr[(ks + 2) & 3][m], m < 2 ? fa_own : fa_other, read_slot, m);
                    if (transfer) lds_transfer_go(voff[pi & 3], w_base(fill_kq, pi));
                    if (pending) {
                        if (kk == 0 && m >= 4) lds_write16(xb_mine, acc[prev][2 + ((m - 4) >> 1)][m & 1], (m - 4) * 1024);
                        if (kk == 2 && m >= 4) lds_read16(out[(m - 4) >> 1][m & 1], xb_partner, (m - 4) * 1024);
                        if (kk == 4 && m < 4) out[m >> 1][m & 1] = (acc[prev][m >> 1][m & 1] + out[m >> 1][m & 1]) * mult;
                        if (kk >= 5 && kk < 13 && m == NM - 1) store_out((kk - 5) >> 2, (kk - 5) & 3);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
                // keep the previous step's fragment registers allocated while the matrix core may
                // still be reading them (see the K = 1024 kernel)
                asm volatile("" ::"v"(fr[(ks + 3) & 3][0]), "v"(fr[(ks + 3) & 3][1]),
                             "v"(fr[(ks + 3) & 3][2]), "v"(fr[(ks + 3) & 3][3]));
                if (ks == 1) {
                    // stage kq + 1 has landed: loads complete in order, and what was requested after
                    // its pieces are the pieces of stages kq + 2 and kq + 3 (those that exist, in the
                    // last row block); pending stores can only make this wait longer
                    const int younger = (kq + 2 < SPB ? 8 : 0) + (kq + 3 < SPB ? 8 : 0);
                    wait_vm(last ? (kq + 1 < SPB ? younger : -1) : 16);
                    wait_lds();
                    __builtin_amdgcn_s_barrier();
                }
            }
        }
        // (Nothing here reads the accumulators: the next block's K step 0 hands them over behind its
        // fourth MFMA at the earliest, long after the last MFMA above has retired.  The build checks
        // the generated code for copies the register allocator might put on the loop edge.)
        // Such copies do get made of the fragment ring, whose registers the variants of this body
        // need not agree on, and a copy reads its source at once: the fragment reads requested for
        // the next block's first two K steps must have landed before control leaves this variant
        // (build.py: check_lds_reads_waited_for).
        wait_lds();
    };
    // the same meeting of the halves with nothing to hide it behind: the last block of a workgroup,
    // and blocks whose stores need bounds checks
    auto meet_now = [&](auto set_tag) __attribute__((always_inline)) {
        constexpr int cur = decltype(set_tag)::value;
        drain_mfma(acc[cur]);  // the last MFMAs retire before their accumulators are read
#pragma unroll
        for (int i = 0; i < 4; ++i) lds_write16(xb_mine, acc[cur][2 + (i >> 1)][i & 1], i * 1024);
        wait_lds();
        __builtin_amdgcn_s_barrier();
#pragma unroll
        for (int i = 0; i < 4; ++i) lds_read16(out[i >> 1][i & 1], xb_partner, i * 1024);
        wait_lds();
        asm volatile("" : "+v"(out[0][0]), "+v"(out[0][1]), "+v"(out[1][0]), "+v"(out[1][1]));
#pragma unroll
        for (int i = 0; i < 4; ++i) out[i >> 1][i & 1] = (acc[cur][i >> 1][i & 1] + out[i >> 1][i & 1]) * mult;
    };

    bool pending = false;
#pragma unroll 1
    for (uint32_t rbi = 0; rbi < nrb; ++rbi) {
        const bool last_block = rbi + 1u == nrb;
        const bool odd = rbi & 1u;
        using T = std::true_type;
        using F = std::false_type;
        using S0 = std::integral_constant<int, 0>;
        using S1 = std::integral_constant<int, 1>;
        if (!odd) {
            if (last_block && pending) row_block_body(T{}, T{}, S0{}, rbi);
            else if (last_block) row_block_body(T{}, F{}, S0{}, rbi);
            else if (pending) row_block_body(F{}, T{}, S0{}, rbi);
            else row_block_body(F{}, F{}, S0{}, rbi);
        } else {
            if (last_block && pending) row_block_body(T{}, T{}, S1{}, rbi);
            else if (last_block) row_block_body(T{}, F{}, S1{}, rbi);
            else if (pending) row_block_body(F{}, T{}, S1{}, rbi);
            else row_block_body(F{}, F{}, S1{}, rbi);
        }
        const uint32_t row_base = m_begin + rbi * kRows;
        const bool full = cols_full && row_base + kRows <= m_end;
        out_base = ((uint64_t)row_base + 32u * kp) * N * esize;
        pending = full && !last_block;  // its halves meet behind the MFMAs of the next row block
        if (pending) continue;
        if (odd)
            meet_now(S1{});
        else
            meet_now(S0{});
        if (full) {
#pragma unroll
            for (int f = 0; f < 2; ++f)
#pragma unroll
                for (int r = 0; r < 4; ++r) store_out(f, r);
        } else {
#pragma unroll
            for (int f = 0; f < 2; ++f)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const uint32_t row = row_base + 32u * kp + 16u * f + 4u * hi + r;
                    if (row >= m_end) continue;
#pragma unroll
                    for (int nb = 0; nb < NBF; ++nb) {
                        if (col + nb >= N) continue;
                        const float v = out[f][nb][r];
                        const uint64_t at = (uint64_t)row * N + col + nb;
                        if (OUT_F32)
                            static_cast<float*>(C)[at] = ACCUM ? static_cast<float*>(C)[at] + v : v;
                        else
                            static_cast<E*>(C)[at] = ACCUM ? (E)((float)static_cast<E*>(C)[at] + v) : (E)v;
                    }
                }
        }
    }
    // Every transfer into LDS was waited for at the barrier of the stage before the one that read
    // it, so none is in flight when the workgroup's LDS is released.
}

namespace {
template <class T16, bool OUT_F32, int KTOT, bool ACCUM>
int launch_pass(const void* W, const void* Xt, void* C, uint32_t M, uint32_t N, const Plan& p, OutputScale os,
                hipStream_t s)
{
    auto kern = fused_ht_gemm_xreg_k2048_kernel<T16, OUT_F32, KTOT, ACCUM>;
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                            kLdsBytes) != hipSuccess)
        return MI_ERR_LAUNCH;
    hipLaunchKernelGGL(kern, dim3(p.grid), dim3(kThreads), kLdsBytes, s, static_cast<const typename T16::E*>(W),
                       static_cast<const typename T16::E*>(Xt), C, M, N, p.m_per_block, p.msplit, p.mpx, p.cgx,
                       p.nrect, os.exp2, os.mult);
    return launch_status();
}

template <class T16, bool OUT_F32>
int launch_ksplit16(const void* W, const void* Xt, void* C, uint32_t M, uint32_t N, uint32_t K, float scale,
                    hipStream_t s)
{
    const OutputScale os = split_output_scale((double)scale, tile_stage_shift<2>(11u, kNarrowRange<T16>));
    const Plan p = plan16(M, N, K);
    if (K == 2048u) return launch_pass<T16, OUT_F32, 2048, false>(W, Xt, C, M, N, p, os, s);
    const int rc = launch_pass<T16, OUT_F32, 4096, false>(W, Xt, C, M, N, p, os, s);
    if (rc != MI_OK) return rc;
    return launch_pass<T16, OUT_F32, 4096, true>(W, Xt, C, M, N, p, os, s);
}
}  // namespace

}  // namespace xreg

// Called by fused_gemm16_xreg for K = 2048 and by the dispatcher of mi_fused_ht_gemm for K = 4096
// (arguments already validated).
int fused_gemm16_xreg_k2048(const void* W, const void* Xt, void* C, uint32_t M, uint32_t N, uint32_t K,
                            int in_dtype, int out_f32, float scale, hipStream_t s)
{
    using namespace xreg;
    if (K != 2048u && K != 4096u) return MI_ERR_SIZE;
    // W and a row block of C are addressed with 32-bit byte offsets
    if ((uint64_t)M * K * 2u > 0xffffffffull || (uint64_t)N * 4u * 64u > 0xffffffffull) return MI_ERR_SHAPE;
    if (in_dtype == MI_BF16)
        return out_f32 ? launch_ksplit16<BF16, true>(W, Xt, C, M, N, K, scale, s)
                       : launch_ksplit16<BF16, false>(W, Xt, C, M, N, K, scale, s);
    if (in_dtype == MI_F16)
        return out_f32 ? launch_ksplit16<F16, true>(W, Xt, C, M, N, K, scale, s)
                       : launch_ksplit16<F16, false>(W, Xt, C, M, N, K, scale, s);
    return MI_ERR_DTYPE;
}

}  // namespace mi
