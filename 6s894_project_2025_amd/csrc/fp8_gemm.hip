// FP8 (OCP E4M3FN) GEMM with per-row scales (mi_fp8_gemm_rowscale), gfx950:
//     out[t][n] = bf16( (sum_k qa[t][k] * qb[n][k]) * sa[t] * sb[n] ),  fp32 accumulate.
// The reference has no FP8 path.  MFMA-bound shape (T = 8192, N = 14336, K = 4096 in the
// benchmark configuration).
//
// Workgroup tile 256 x 256, four wavefronts of 128 x 128, K walked in steps of 128 bytes with
// v_mfma_f32_16x16x128_f8f6f4 (unscaled form).  Both operand tiles go global -> LDS directly (eight
// lanes per 128-byte row segment, so the L1 coalesces), double buffered: the loads of step s+1
// are in flight while step s is multiplied, and the first fragments of step s+1 are read from
// LDS behind the last MFMAs of step s.  LDS tiles are [256 rows][8 chunks of 16 B]
// with chunk c of LDS row r stored at c ^ (r & 7); a lane of K-group hi reads chunks hi and hi + 4
// of its row (any K assignment works as long as both operands use the same one).  Both the staging
// writes and these fragment reads measured bank-conflict free; chunks 2*hi, 2*hi + 1 did not.
// qb rows are the MFMA A operand and are stored in LDS in the order that lets a lane own 32
// consecutive output columns; the result is staged through LDS once more so that C rows are
// written as whole 512-byte runs.
#include <type_traits>

#include "common.hpp"
#include "lds_layout.hpp"

namespace mi {
namespace {

typedef int i32x8 __attribute__((ext_vector_type(8)));

constexpr int kTile = 256;           // rows of qa and of qb per workgroup
constexpr int kStepBytes = 128;      // K bytes per step
constexpr int kTileBytes = kTile * kStepBytes;  // 32 KB
constexpr int kThreads = 256;

// acc += A(16 x 128, E4M3FN) * B(128 x 16, E4M3FN) with the accumulator tied in place in the AGPR
// file.  Written as inline assembly because, with all 256 AGPRs holding accumulators, the
// compiler's own MFMA selection kept shuffling accumulators between register files inside the K
// loop.  Hazards the compiler can no longer see: the operands come from LDS reads (ordinary
// register dependencies, which it still tracks), the two idle cycles cover a VALU-written operand,
// and the accumulators are first read after the drain at the end of the K loop.
__device__ __forceinline__ void mfma_fp8(f32x4& c, const i32x8& a, const i32x8& b)
{
    asm volatile("s_nop 1\n\tv_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
}

__host__ __device__ constexpr uint32_t tile_off(uint32_t row, uint32_t chunk)
{
    return (row * 8u + (chunk ^ (row & 7u))) << 4;
}
// Epilogue image of the 256 x 256 bf16 result: [256 rows][512 B], chunk c of row r stored at
// c ^ (r & 31).
__host__ __device__ constexpr uint32_t out_tile_off(uint32_t row, uint32_t chunk)
{
    return row * 512u + ((chunk ^ (row & 31u)) << 4);
}
constexpr bool lds_patterns_conflict_free()
{
    // operand fragments: lane (hi, lo) reads row r0 + lo, chunks hi and hi + 4
    for (uint32_t half = 0; half < 2; ++half)
        if (!lds::conflict_free_b128(
                [=](uint32_t lane) { return tile_off(lane & 15u, (lane >> 4) + 4u * half); }))
            return false;
    // epilogue: lane (hi, lo) writes row 16 ti + lo, chunk 4 hi + r (+ 16 per wavefront column); the
    // copy-out reads row 8 i + tid / 32, chunk tid % 32
    for (uint32_t r = 0; r < 4; ++r)
        if (!lds::conflict_free_b128(
                [=](uint32_t lane) { return out_tile_off(lane & 15u, 4u * (lane >> 4) + r); }))
            return false;
    for (uint32_t w = 0; w < 4; ++w)
        if (!lds::conflict_free_b128(
                [=](uint32_t lane) { return out_tile_off((64u * w + lane) >> 5, (64u * w + lane) & 31u); }))
            return false;
    return true;
}
static_assert(lds_patterns_conflict_free(), "an LDS access pattern of the FP8 GEMM would serialise");

// LDS row r of the qb tile holds tile row 128*(r>>7) + 8*(r&15) + ((r>>4)&7): fragment block nb of
// a wavefront (LDS rows 16*nb .. 16*nb+15) then carries columns 8*lo + nb.
__device__ __forceinline__ uint32_t qb_tile_row(uint32_t r)
{
    return (r & 128u) + 8u * (r & 15u) + ((r >> 4) & 7u);
}

__global__ void __launch_bounds__(kThreads)
fp8_gemm_rowscale_kernel(const uint8_t* __restrict__ qa, const float* __restrict__ sa,
                         const uint8_t* __restrict__ qb, const float* __restrict__ sb,
                         __bf16* __restrict__ out, uint32_t T, uint32_t N, uint32_t K,
                         uint32_t tiles_t, uint32_t tiles_n)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];  // 2 x (A tile + B tile)
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    // wavefront index as a scalar, so LDS bases of the direct transfers (M0) are scalar arithmetic
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t lo = lane & 15u, hi = lane >> 4;
    const uint32_t wt = wave >> 1, wn = wave & 1u;

    // tile order: consecutive workgroup ids land on different XCDs; an XCD works on 4 row tiles x
    // a run of column tiles at a time, so its L2 serves most operand re-reads
    uint32_t tm, tn;
    {
        const uint32_t id = blockIdx.x;
        const uint32_t groups_t = (tiles_t + 3u) / 4u;  // groups of 4 row tiles
        const uint32_t per_group = 4u * tiles_n;
        // spread groups over XCDs round-robin
        const uint32_t xcd = id & 7u, j = id >> 3;
        const uint32_t slots = (groups_t + 7u) / 8u;           // groups per XCD
        const uint32_t g = xcd * slots + j / per_group;         // group of this workgroup
        const uint32_t w = j % per_group;
        tm = g * 4u + (w & 3u);
        tn = w >> 2;
        if (g >= groups_t || tm >= tiles_t) return;  // padding ids of an uneven split
    }
    const uint32_t t0 = tm * kTile, n0 = tn * kTile;

    // Operand staging, global -> LDS directly (no register hop): wavefront w, instruction i fills
    // the 1 KB of LDS rows 32*i + 8*w .. +7 of a tile, lane l landing at byte 16*l of that run.
    // Under the swizzle, slot l of the run is row r = 32*i + 8*w + l/8, position l%8, which holds
    // global chunk (l%8) ^ (r & 7) = (l%8) ^ (l/8 % 8): eight adjacent lanes still cover one whole
    // 128-byte row segment, so the loads coalesce.
    const uint32_t cg = (lane & 7u) ^ ((lane >> 3) & 7u);
    uint32_t oa[8], ob[8];  // 32-bit byte offsets (operands are checked to be below 4 GiB)
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const uint32_t r = 32u * i + 8u * wave + (lane >> 3);
        const uint32_t ra = min(t0 + r, T - 1u);               // qa tile: LDS row = tile row
        const uint32_t rb = min(n0 + qb_tile_row(r), N - 1u);  // qb tile: permuted
        oa[i] = ra * K + 16u * cg;
        ob[i] = rb * K + 16u * cg;
    }
    typedef __attribute__((address_space(1))) const void* gptr_t;
    typedef __attribute__((address_space(3))) void* lptr_t;
    // instruction pair i (of 8) of the transfer of K step k0 / 128 into LDS buffer `buf`
    auto stage_part = [&](uint32_t buf, uint32_t k0, int i) {
        unsigned char* A = lds + buf * (2u * kTileBytes);
        unsigned char* B = A + kTileBytes;
        const uint32_t run = (32u * i + 8u * wave) * 128u;  // wavefront-uniform
        __builtin_amdgcn_global_load_lds((gptr_t)(qb + (ob[i] + k0)), (lptr_t)(B + run), 16, 0, 0);
        __builtin_amdgcn_global_load_lds((gptr_t)(qa + (oa[i] + k0)), (lptr_t)(A + run), 16, 0, 0);
    };
    auto stage = [&](uint32_t buf, uint32_t k0) {
#pragma unroll
        for (int i = 0; i < 8; ++i) stage_part(buf, k0, i);
    };

    f32x4 acc[8][8];  // [nb][ti]
#pragma unroll
    for (int nb = 0; nb < 8; ++nb)
#pragma unroll
        for (int ti = 0; ti < 8; ++ti) acc[nb][ti] = f32x4{0.f, 0.f, 0.f, 0.f};

    const uint32_t ksteps = K / kStepBytes;
    auto frag = [&](const unsigned char* tile, uint32_t r) {
        const u32x4 x0 = *reinterpret_cast<const u32x4*>(tile + tile_off(r, hi));
        const u32x4 x1 = *reinterpret_cast<const u32x4*>(tile + tile_off(r, hi + 4u));
        return i32x8{(int)x0[0], (int)x0[1], (int)x0[2], (int)x0[3],
                     (int)x1[0], (int)x1[1], (int)x1[2], (int)x1[3]};
    };
    const uint32_t ra0 = 128u * wn + lo;  // first LDS row of this lane's qb fragments (MFMA A)
    const uint32_t rb0 = 128u * wt + lo;  // first LDS row of its qa fragments (MFMA B)

    // Two LDS buffers, transfers running two steps ahead of the multiplication.  The barrier of
    // step ks sits after the sixth of its eight fragment columns: by then every LDS read of the
    // current buffer has been issued and waited for, and the transfer of step ks+1 (started two
    // steps earlier) has landed.  Behind the barrier the current buffer is refilled with step ks+2
    // (half of the transfer instructions in the shadow of the last sixteen MFMAs, the other half
    // behind the first sixteen of the next step), and the fragments step ks+1 starts with are
    // read, each qb fragment right after its last use.
    stage(0, 0);
    {
        const uint32_t k1 = ksteps > 1 ? 1u : 0u;
#pragma unroll
        for (int i = 0; i < 4; ++i) stage_part(1, k1 * kStepBytes, i);
    }
    asm volatile("s_waitcnt vmcnt(8)" ::: "memory");  // the 16 transfers of step 0 are the oldest
    __syncthreads();
    i32x8 af[8], b0, b1;
#pragma unroll
    for (int nb = 0; nb < 8; ++nb) af[nb] = frag(lds + kTileBytes, ra0 + 16u * nb);
    b0 = frag(lds, rb0);
    b1 = frag(lds, rb0 + 16u);
    // The body is branch-free: the last two steps of a tile repeat transfers of earlier K steps
    // (valid addresses, results never read) and read fragments nobody uses, which is cheaper than
    // conditional code on the matrix-core critical path.  Those stray transfers are drained before
    // the epilogue reuses LDS.
#pragma unroll 1
    for (uint32_t ks = 0; ks < ksteps; ++ks) {
        const uint32_t buf = ks & 1u;
        const uint32_t k1 = ks + 1 < ksteps ? ks + 1 : 0u;                          // step after this one
        const uint32_t k2 = ks + 2 < ksteps ? ks + 2 : 0u;  // and the next
        const unsigned char* A = lds + buf * (2u * kTileBytes);  // qa tile
        const unsigned char* An = lds + (buf ^ 1u) * (2u * kTileBytes);
        i32x8 bfr[8];
        bfr[0] = b0;
        bfr[1] = b1;
#pragma unroll
        for (int ti = 0; ti < 6; ++ti) {
#pragma unroll
            for (int nb = 0; nb < 8; ++nb) {
                mfma_fp8(acc[nb][ti], af[nb], bfr[ti]);
                if (nb == 0) bfr[ti + 2] = frag(A, rb0 + 16u * (ti + 2));
                if (ti < 2 && (nb & 3) == 1)
                    stage_part(buf ^ 1u, k1 * kStepBytes, 4 + 2 * ti + (nb >> 2));
            }
            // keep the scheduler from hoisting later fragment reads up here: with all 512
            // registers in use, longer live ranges turn into accumulator shuffling
            __builtin_amdgcn_sched_barrier(0);
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
#pragma unroll
        for (int nb = 0; nb < 8; ++nb) {
            if (nb == 0) b0 = frag(An, rb0);
            if (nb == 1) b1 = frag(An, rb0 + 16u);
            mfma_fp8(acc[nb][6], af[nb], bfr[6]);
            if ((nb & 3) == 2) stage_part(buf, k2 * kStepBytes, nb >> 2);
            if ((nb & 3) == 3) __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int nb = 0; nb < 8; ++nb) {
            mfma_fp8(acc[nb][7], af[nb], bfr[7]);
            af[nb] = frag(An + kTileBytes, ra0 + 16u * nb);
            if ((nb & 3) == 2) stage_part(buf, k2 * kStepBytes, 2 + (nb >> 2));
            if (nb & 1) __builtin_amdgcn_sched_barrier(0);
        }
    }
    // drain: stray transfers, and the matrix-core pipeline before the accumulators are read
    asm volatile("s_nop 15\n\ts_nop 15\n\ts_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();

    // ---- epilogue: scale, narrow, stage through LDS, store whole rows ---------------------------
    // D[m'][n']: n' = lo -> qa row t0 + 128*wt + 16*ti + lo; m' = 4*hi + r -> column
    // 128*wn + 8*m' + nb = 128*wn + 32*hi + 8*r + nb.  LDS image: [256 rows][512 B], 16-byte chunk
    // ch of row r stored at ch ^ (r & 31).
    typedef __bf16 bf16x8v __attribute__((ext_vector_type(8)));
    // this lane's 32 column scales (columns 128*wn + 32*hi + 0..31), loaded once
    float sbv[32];
    {
        const uint32_t cbase = n0 + 128u * wn + 32u * hi;
        if (cbase + 32u <= N) {
#pragma unroll
            for (int v = 0; v < 8; ++v) {
                const f32x4 x = *reinterpret_cast<const f32x4*>(sb + cbase + 4u * v);
#pragma unroll
                for (int j = 0; j < 4; ++j) sbv[4 * v + j] = x[j];
            }
        } else {
#pragma unroll
            for (int v = 0; v < 32; ++v) sbv[v] = sb[min(cbase + v, N - 1u)];
        }
    }
#pragma unroll
    for (int ti = 0; ti < 8; ++ti) {
        const uint32_t rl = 128u * wt + 16u * ti + lo;
        const float st = sa[min(t0 + rl, T - 1u)];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const uint32_t col = 128u * wn + 32u * hi + 8u * r;  // 8 consecutive columns: nb = 0..7
            bf16x8v o;
#pragma unroll
            for (int nb = 0; nb < 8; ++nb) o[nb] = (__bf16)(acc[nb][ti][r] * st * sbv[8 * r + nb]);
            const uint32_t ch = col >> 3;
            *reinterpret_cast<bf16x8v*>(lds + out_tile_off(rl, ch)) = o;
        }
    }
    __syncthreads();
    const bool vec_ok = (N & 7u) == 0;
#pragma unroll 4
    for (uint32_t i = 0; i < 32; ++i) {
        const uint32_t rl = 8u * i + (tid >> 5), ch = tid & 31u;
        const bf16x8v o = *reinterpret_cast<const bf16x8v*>(lds + out_tile_off(rl, ch));
        const uint32_t t = t0 + rl, col = n0 + 8u * ch;
        if (t < T && col < N) {
            __bf16* dst = out + (uint64_t)t * N + col;
            if (vec_ok && col + 8u <= N) {
                // streaming store: the result is not read again here, and keeping it out of the
                // caches leaves them to the operand panels that the following tiles re-read
                __builtin_nontemporal_store(o, reinterpret_cast<bf16x8v*>(dst));
            } else {
#pragma unroll
                for (int j = 0; j < 8; ++j)
                    if (col + j < N) dst[j] = o[j];
            }
        }
    }
}

}  // namespace
}  // namespace mi

extern "C" int mi_fp8_gemm_rowscale(const void* qa, const float* sa, const void* qb,
                                    const float* sb, void* out, uint32_t T, uint32_t N, uint32_t K,
                                    void* stream)
{
    using namespace mi;
    if (K == 0 || (K & 127u)) return MI_ERR_SHAPE;
    if (T == 0 || N == 0) return MI_OK;
    if (!qa || !sa || !qb || !sb || !out) return MI_ERR_NULL;
    if (!aligned16(qa) || !aligned16(qb) || !aligned16(out)) return MI_ERR_ALIGN;
    if ((uint64_t)T * K > 0xffffffffull || (uint64_t)N * K > 0xffffffffull) return MI_ERR_SHAPE;
    const uint32_t tiles_t = (T + kTile - 1) / kTile, tiles_n = (N + kTile - 1) / kTile;
    // ids: 8 XCDs x (groups of 4 row tiles per XCD) x (4 * tiles_n); uneven splits are padded
    const uint32_t groups_t = (tiles_t + 3u) / 4u;
    const uint32_t slots = (groups_t + 7u) / 8u;
    const uint64_t grid = (uint64_t)8u * slots * 4u * tiles_n;
    if (grid > 0x7fffffffull) return MI_ERR_SHAPE;
    const size_t lds = 4u * kTileBytes;  // 128 KB (also holds the 256 x 512 B result image)
    auto kern = fp8_gemm_rowscale_kernel;
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
        return MI_ERR_LAUNCH;
    hipLaunchKernelGGL(kern, dim3((uint32_t)grid), dim3(kThreads), lds, static_cast<hipStream_t>(stream),
                       static_cast<const uint8_t*>(qa), sa, static_cast<const uint8_t*>(qb), sb,
                       static_cast<__bf16*>(out), T, N, K, tiles_t, tiles_n);
    return launch_status();
}
