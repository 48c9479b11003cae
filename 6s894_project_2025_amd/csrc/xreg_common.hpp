// Pieces shared by the register-resident fused GEMM kernels (fused_gemm_xreg.hip for 16-bit inputs,
// fused_gemm_xreg_f32.hip for fp32): the LDS geometry of the W stream and of the prologue's layout
// change, the opaque memory statements, the workgroup tiling and its launch plan.
#pragma once
#include "fwht_device.hpp"
#include "lds_layout.hpp"

namespace mi {
namespace xreg {

constexpr int kThreads = 256;
constexpr int kRows = 64;                         // rows of W per row block
constexpr int kStageK = 256;                      // K extent of one W stage
constexpr int kStageBytes = kRows * kStageK * 2;  // 32 KB
constexpr int kSlots = 4;                         // ring of stage buffers
constexpr int kStepsPerStage = kStageK / 32;      // 8 MFMA K steps
constexpr int kAreaBytes = 16 * 512 * 2;          // per wavefront: 16 columns x 512 k
// stage buffers 0..3 at [0, 128K); the wavefront areas of the prologue at [96K, 160K), i.e.
// on top of stage buffer 3, which is first filled after the prologue
constexpr int kAreaBase = 3 * kStageBytes;
constexpr int kLdsBytes = kAreaBase + 4 * kAreaBytes;

typedef __attribute__((address_space(3))) void* lptr_t;

// LDS image of a W stage: [64 rows][512 B], the 16-byte chunk q of row r stored at q ^ (r & 15).
__host__ __device__ constexpr uint32_t stage_offset(uint32_t row, uint32_t q)
{
    return row * 512u + ((q ^ (row & 15u)) << 4);
}
// A wavefront's area of the prologue: [16 columns][1 KB], chunk q of column j stored at q ^ j.
__host__ __device__ constexpr uint32_t area_offset(uint32_t j, uint32_t q)
{
    return j * 1024u + ((q ^ j) << 4);
}
// The lane part of a fragment address: row lo, chunk hi of a stage; the fragment of row block mb and
// K step ks is at (frag_lane_offset ^ (ks << 6)) + 8192 mb (checked below).
__host__ __device__ constexpr uint32_t frag_lane_offset(uint32_t lo, uint32_t hi)
{
    return lo * 512u + ((hi ^ lo) << 4);
}
constexpr bool lds_patterns_conflict_free()
{
    for (uint32_t lane = 0; lane < 64; ++lane)
        for (uint32_t mb = 0; mb < 4; ++mb)
            for (uint32_t ks = 0; ks < 8; ++ks)
                if ((frag_lane_offset(lane & 15u, lane >> 4) ^ (ks << 6)) + 8192u * mb !=
                    stage_offset(16u * mb + (lane & 15u), 4u * ks + (lane >> 4)))
                    return false;
    // fragment read of row block mb, K step ks: lane (hi, lo) takes row 16 mb + lo, chunk 4 ks + hi
    for (uint32_t mb = 0; mb < 4; ++mb)
        for (uint32_t ks = 0; ks < 8; ++ks)
            if (!lds::conflict_free_b128(
                    [=](uint32_t lane) { return stage_offset(16u * mb + (lane & 15u), 4u * ks + (lane >> 4)); }))
                return false;
    // prologue: every lane writes chunk `lane` of column j; lane (hi, lo) reads chunk 4 s + hi of
    // column lo
    for (uint32_t j = 0; j < 16; ++j)
        if (!lds::conflict_free_b128([=](uint32_t lane) { return area_offset(j, lane); })) return false;
    for (uint32_t s = 0; s < 16; ++s)
        if (!lds::conflict_free_b128([=](uint32_t lane) { return area_offset(lane & 15u, 4u * s + (lane >> 4)); }))
            return false;
    return true;
}
static_assert(lds_patterns_conflict_free(), "an LDS access pattern of the fused GEMM would serialise");

// The 16-bit kernels' prologue area: 32 KB per wavefront in four 8 KB pieces, piece p of wavefront w
// being the wavefront's own rows (16 w .. 16 w + 15) of stage buffer 1 + p for p < 3 and 8 KB of the
// 32 KB behind the ring for p = 3.  A piece holds eight transformed columns of 512 k, column j' at
// 1 KB j' with its 16-byte chunk q stored at q ^ j (j = the column's number in its round of 16).
// Half (K = 1024) or round parity (K = 512) b, columns 8 h .. 8 h + 7 use piece b + 2 h, so the two
// halves of a column are 32 KB apart: one address register and an immediate serve both.
__host__ __device__ constexpr uint32_t area_piece_offset(uint32_t w, uint32_t p)
{
    return (p < 3u ? (1u + p) * (uint32_t)kStageBytes : (uint32_t)(kSlots * kStageBytes)) + w * 8192u;
}
static_assert(kSlots * kStageBytes + 4 * 8192 == kLdsBytes, "the fourth pieces fill the 32 KB behind the ring");
constexpr bool area16_patterns_conflict_free()
{
    for (uint32_t b = 0; b < 2; ++b) {
        // write: every lane stores chunk `lane` of column j; read: lane (hi, lo) takes chunk 4 s + hi of column lo
        for (uint32_t j = 0; j < 16; ++j)
            if (!lds::conflict_free_b128([=](uint32_t lane) {
                    return area_piece_offset(0, b + 2u * (j >> 3)) + (j & 7u) * 1024u + ((lane ^ j) << 4);
                }))
                return false;
        for (uint32_t s = 0; s < 16; ++s)
            if (!lds::conflict_free_b128([=](uint32_t lane) {
                    const uint32_t lo = lane & 15u, hi = lane >> 4;
                    return area_piece_offset(0, b + 2u * (lo >> 3)) + (lo & 7u) * 1024u + (((4u * s + hi) ^ lo) << 4);
                }))
                return false;
    }
    return true;
}
static_assert(area16_patterns_conflict_free(), "an LDS access pattern of the 16-bit prologue would serialise");

// Waits out the matrix-core pipeline before `acc` is read by anything but an MFMA.  Two statements:
// the delay itself, which names no register (naming them lets the compiler set the operands up
// with register copies *in front of* the statement, i.e. reads of the accumulators right behind
// the last MFMA: observed with sixteen accumulators), and an empty statement that the
// accumulators pass through, so that no read of them (a register copy, say) can move above the
// delay.
__device__ __forceinline__ void mfma_delay()
{
    asm volatile("s_nop 15\n\ts_nop 7" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
}
__device__ __forceinline__ void drain_mfma(f32x4 (&acc)[4][1])
{
    mfma_delay();
    asm volatile("" : "+v"(acc[0][0]), "+v"(acc[1][0]), "+v"(acc[2][0]), "+v"(acc[3][0]));
}
__device__ __forceinline__ void drain_mfma(f32x4 (&acc)[4][2])
{
    mfma_delay();
    asm volatile(""
                 : "+v"(acc[0][0]), "+v"(acc[0][1]), "+v"(acc[1][0]), "+v"(acc[1][1]),
                   "+v"(acc[2][0]), "+v"(acc[2][1]), "+v"(acc[3][0]), "+v"(acc[3][1]));
}
__device__ __forceinline__ void drain_mfma(f32x4 (&acc)[4][4])
{
    mfma_delay();
    asm volatile(""
                 : "+v"(acc[0][0]), "+v"(acc[0][1]), "+v"(acc[0][2]), "+v"(acc[0][3]),
                   "+v"(acc[1][0]), "+v"(acc[1][1]), "+v"(acc[1][2]), "+v"(acc[1][3]),
                   "+v"(acc[2][0]), "+v"(acc[2][1]), "+v"(acc[2][2]), "+v"(acc[2][3]),
                   "+v"(acc[3][0]), "+v"(acc[3][1]), "+v"(acc[3][2]), "+v"(acc[3][3]));
}

__device__ __forceinline__ void wait_lds() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }
// at most n vector memory loads of this wavefront still outstanding (they complete in order); a
// negative n means there is nothing to wait for.  `n` must fold to a constant once the loops around
// the call are unrolled: it is an immediate of the instruction, so a count that does not fold, or
// one the counter's six bits cannot hold, fails to build instead of silently dropping the wait.
__device__ __forceinline__ void wait_vm(int n)
{
    if (n >= 0) asm volatile("s_waitcnt vmcnt(%0)" ::"i"(n) : "memory");
}

// A wavefront that has its SIMD to itself issues roughly one instruction every eight cycles
// (measured on loops of one v_mfma_f32_16x16x32 plus n independent instructions: 19 cycles for n = 0,
// 20 for n = 1, 24 / 32 / 39 for n = 2 / 3 / 4, the same for vector and scalar arithmetic; one
// ds_read_b128 per MFMA: 27 cycles; s_nop and satisfied waits cost next to nothing).  Between two
// 16-cycle MFMAs one other instruction is free and every further one costs the MFMA stream eight
// cycles, so the statements below are as few instructions as they can be, and are placed by hand.
//
// 16 bytes per lane from global memory straight into LDS, in two statements so that an MFMA can
// stand between them (M0 must be written one instruction before the transfer that uses it):
// lane l's bytes come from base + lane_off and land at lds_wave_base + lds_imm + 16 l.  Scalar
// base + 32-bit lane offset form, so that no vector arithmetic is spent on addresses; `lds_imm`
// must fold to a constant (an immediate of the scalar add: a transfer then needs no scalar
// register of its own).  The instruction's own offset field is left at zero: the hardware adds
// it to the LDS address as well as to the global one.
// (M0 carries the LDS base of the transfer.  It is a reserved register that cannot be named as a
// clobber, so the build reads the generated ISA instead and fails if anything but these statements
// touches M0 in a kernel that uses them: build.py, check_m0_is_the_transfers_alone.)
__device__ __forceinline__ void lds_transfer_target(uint32_t lds_wave_base, int lds_imm)
{
    asm volatile("s_add_i32 m0, %0, %1" :: "s"(lds_wave_base), "i"(lds_imm) : "memory", "scc");
}
__device__ __forceinline__ void lds_transfer_go(uint32_t lane_off, const void* base)
{
    asm volatile("global_load_lds_dwordx4 %0, %1" :: "v"(lane_off), "s"(base) : "memory");
}
// both statements at once, where nothing useful can stand between them
__device__ __forceinline__ void global_to_lds16(uint32_t lane_off, const void* base, uint32_t lds_wave_base,
                                                int lds_imm)
{
    asm volatile("s_add_i32 m0, %2, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 :: "v"(lane_off), "s"(base), "s"(lds_wave_base), "i"(lds_imm) : "memory", "scc");
}
// A 16-byte LDS read as an opaque statement: address register + constant offset (below 64 KB), no
// wait inserted by the compiler at the use: the caller waits with wait_lds_all_but.
template <class V>
__device__ __forceinline__ void lds_read16(V& dst, uint32_t addr, int offset)
{
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "i"(offset) : "memory");
}
// One 16-byte LDS write per lane, equally opaque; the data registers must stay as they are until
// the write has been waited for.
template <class V>
__device__ __forceinline__ void lds_write16(uint32_t addr, V v, int offset)
{
    asm volatile("ds_write_b128 %0, %1 offset:%2" ::"v"(addr), "v"(v), "i"(offset) : "memory");
}
// at most N LDS reads of this wavefront still outstanding (they complete in order)
template <int N>
__device__ __forceinline__ void wait_lds_all_but()
{
    static_assert(N >= 0 && N <= 15, "the counter has four bits");
    asm volatile("s_waitcnt lgkmcnt(%0)" :: "n"(N) : "memory");
}
// streaming (non-temporal) stores, scalar base + 32-bit lane offset
__device__ __forceinline__ void stream_store4(uint32_t lane_off, uint32_t v, void* base)
{
    asm volatile("global_store_dword %0, %1, %2 nt" :: "v"(lane_off), "v"(v), "s"(base) : "memory");
}
__device__ __forceinline__ void stream_store8(uint32_t lane_off, u32x2 v, void* base)
{
    asm volatile("global_store_dwordx2 %0, %1, %2 nt" :: "v"(lane_off), "v"(v), "s"(base) : "memory");
}
// the same without the streaming hint, for results that are read again soon
__device__ __forceinline__ void cached_store4(uint32_t lane_off, uint32_t v, void* base)
{
    asm volatile("global_store_dword %0, %1, %2" :: "v"(lane_off), "v"(v), "s"(base) : "memory");
}
__device__ __forceinline__ void cached_store8(uint32_t lane_off, u32x2 v, void* base)
{
    asm volatile("global_store_dwordx2 %0, %1, %2" :: "v"(lane_off), "v"(v), "s"(base) : "memory");
}
// (A store of more than 8 bytes still reads its data registers during the next cycles; the compiler
// keeps ordinary code away from them for that long, but does not know what this statement is.)
__device__ __forceinline__ void stream_store16(uint32_t lane_off, u32x4 v, void* base, int offset = 0)
{
    asm volatile("global_store_dwordx4 %0, %1, %2 offset:%3 nt\n\ts_nop 1" :: "v"(lane_off), "v"(v), "s"(base), "i"(offset) : "memory");
}

// Workgroup id -> (column group, M slice); false for an id past the last rectangle.
__host__ __device__ inline bool tile_of_workgroup(uint32_t id, uint32_t msplit, uint32_t mpx, uint32_t cgx,
                                                  uint32_t nrect, uint32_t& cg, uint32_t& ms)
{
    const uint32_t x = id & 7u, j = id >> 3;  // XCD, index inside the XCD
    const uint32_t rsz = mpx * cgx;
    const uint32_t rect = (j / rsz) * 8u + x, in = j % rsz;
    if (rect >= nrect) return false;
    const uint32_t rects_m = msplit / mpx;
    ms = (rect % rects_m) * mpx + in % mpx;
    cg = (rect / rects_m) * cgx + in / mpx;
    return true;
}

// How the (column group, M slice) grid is cut.  One workgroup fills a compute unit (all of its
// registers and LDS), so the launch runs in rounds of 256 workgroups; a workgroup costs one prologue
// plus a fixed time per 64-row block (16-bit kernel: measured ~6.5 us and ~2.9 us, the same for
// every K: a row block is 64 rows x 131072 / K columns x K; fp32 kernels: ~15 us, twice that at
// K = 4096, and 13.7 us).  The number of M slices is the one that minimises
// rounds x (prologue + row blocks per slice) in those units (`pro_cost` : `block_cost`, 9 : 4 for
// the 16-bit kernel): enough slices to fill the chip, no more than that (every slice repeats the
// transform of its columns), and no nearly empty last round.
struct Plan {
    uint32_t ngroups, msplit, m_per_block;
    uint32_t mpx, cgx, nrect, grid;  // XCD rectangles
};
inline Plan plan(uint32_t M, uint32_t N, uint32_t cols, uint32_t mpx_max, uint32_t pro_cost = 9u,
                 uint32_t block_cost = 4u)
{
    Plan p{};
    p.ngroups = (N + cols - 1u) / cols;
    const uint32_t row_blocks = (M + kRows - 1u) / kRows;
    uint64_t best = ~0ull;
    uint32_t best_s = 1;
    for (uint32_t sp = 1; sp <= row_blocks && sp <= 256u; ++sp) {
        const uint32_t rb = (row_blocks + sp - 1u) / sp;
        const uint32_t slices = (row_blocks + rb - 1u) / rb;  // what sp really yields
        const uint64_t rounds = ((uint64_t)p.ngroups * slices + 255u) / 256u;
        const uint64_t cost = rounds * (pro_cost + block_cost * (uint64_t)rb);
        if (cost < best) {
            best = cost;
            best_s = slices;
        }
    }
    const uint32_t rb = (row_blocks + best_s - 1u) / best_s;
    p.m_per_block = rb * kRows;
    p.msplit = (M + p.m_per_block - 1u) / p.m_per_block;
    // Rectangles: mpx | msplit, cgx | ngroups, at most 32 workgroups (one round of an XCD).
    // Rectangle r runs on XCD r % 8, so the busiest XCD gets ceil(nrect / 8) rectangles.  Wanted,
    // in this order: as few rounds on the busiest XCD as possible, a load within 15 % of an even
    // spread over the eight XCDs, the largest rectangle, M extent 4 before 2, 8, 1.  (1 x 1 is
    // the plain order, so there is always a candidate.)
    const uint32_t total = p.ngroups * p.msplit;
    const uint32_t even = (total + 7u) / 8u;
    const uint32_t pref[4] = {4u, 2u, 8u, 1u};
    uint64_t best_key = ~0ull;
    for (uint32_t k = 0; k < 4; ++k) {
        const uint32_t m = pref[k];
        if (m > mpx_max || p.msplit % m != 0u) continue;
        for (uint32_t c = 1; c * m <= 32u; ++c) {
            if (p.ngroups % c != 0u) continue;
            const uint32_t nrect = (p.msplit / m) * (p.ngroups / c);
            const uint32_t busiest = ((nrect + 7u) / 8u) * m * c;
            const uint64_t rounds = (busiest + 31u) / 32u;
            const uint64_t uneven = (uint64_t)busiest * 100u > (uint64_t)even * 115u ? 1u : 0u;
            const uint64_t key = (rounds << 40) | (uneven << 36) | ((uint64_t)(32u - m * c) << 24) |
                                 ((uint64_t)k << 20) | busiest;
            if (key < best_key) {
                best_key = key;
                p.mpx = m;
                p.cgx = c;
                p.nrect = nrect;
            }
        }
    }
    p.grid = ((p.nrect + 7u) / 8u) * 8u * p.mpx * p.cgx;
    return p;
}

// The plan of the 16-bit kernels by K: 131072 / K columns per workgroup (64 at K = 4096, whose two
// passes each transform twice as much per column as the K = 2048 kernel does for the same main loop).
inline Plan plan16(uint32_t M, uint32_t N, uint32_t K)
{
    if (K == 4096u) return plan(M, N, 64u, 8u, 18u, 4u);
    return plan(M, N, 131072u / K, 8u);
}

}  // namespace xreg
}  // namespace mi
