// fp32 variant of the fused Hadamard -> GEMM for short transforms, K = 32, 64, 128 (see
// fused_gemm.hip for the structure; K = 256 runs the GEMV kernels, K >= 512 those or the
// register-resident kernels of fused_gemm_xreg_f32.hip: see fused_gemm_f32 below).
//
// The transformed tile Y[BN][K] is kept in LDS as fp32; the prologue runs the fp32 transform on
// the bf16 matrix cores with exact three-piece operands (tile_transform_f32), and the
// contraction uses the fp32 matrix-core instruction v_mfma_f32_16x16x4_f32, so every product
// and sum is fp32 (there is no reduced-precision shortcut on this hardware).
// One 16-byte fragment per lane supplies four consecutive K for four MFMAs: lane (lo, hi) of K-step
// kk holds k = 16*kk + 4*hi + s, s = 0..3, for both operands.  W reaches that order through a
// wavefront-private LDS staging area (coalescable loads in, operand-order reads out).
#include "fwht_device.hpp"

namespace mi {

// K = 512 ... 4096 with the transformed operand in registers: fused_gemm_xreg_f32.hip
int fused_gemm_f32_xreg(const float* W, const float* Xt, float* C, uint32_t M, uint32_t N, uint32_t K,
                        float scale, hipStream_t s);

// The GEMV kernels (fused_gemv.hip and the files it names) on X given column by column: the same
// product with 16 columns per workgroup.
namespace gemv {
int launch_any(const float* W, const float* X, float* Y, uint32_t M, uint32_t N, uint32_t B, float scale,
               bool columns_contiguous, hipStream_t s);
}  // namespace gemv

namespace {

constexpr int kThreads = 512;
constexpr int kWaves = kThreads / 64;
constexpr int kStageBytes = 64 * 64;  // per wavefront: 64 rows x 16 K x 4 B

template <int LOG_NB>
__device__ __forceinline__ uint32_t y_off(uint32_t n, uint32_t q, uint32_t col_bytes,
                                          uint32_t swz_mask)
{
    return (n * (col_bytes >> 4) + (q ^ ((n >> LOG_NB) & swz_mask))) << 4;
}

template <int BN>
__global__ void __launch_bounds__(kThreads)
fused_ht_gemm_f32_kernel(const float* __restrict__ W, const float* __restrict__ Xt,
                         float* __restrict__ C, uint32_t M, uint32_t N, uint32_t K, uint32_t logK,
                         uint32_t m_per_block, float fscale)
{
    constexpr int NB = BN / 16;
    constexpr int LOG_NB = NB == 4 ? 2 : (NB == 2 ? 1 : 0);
    extern __shared__ __attribute__((aligned(16))) unsigned char ylds[];

    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint32_t lo = lane & 15u, hi = lane >> 4;
    const uint32_t n0 = blockIdx.x * BN;
    const uint32_t chunks_per_col = K >> 2;
    const uint32_t swz_mask = (chunks_per_col >= 16u ? 16u : chunks_per_col) - 1u;
    const uint32_t col_bytes = K * 4u;

    // staging layout: row r (64 bytes), 16-byte chunk c stored at position c ^ ((r >> 1) & 3)
    // (conflict-free for both the writer's and the reader's lane order)
    unsigned char* stage = ylds + (size_t)BN * K * 4u + wave * kStageBytes;
    const uint32_t wr_off = (lane >> 2) * 64u + (((lane & 3u) ^ ((lane >> 3) & 3u)) << 4);
    const uint32_t rd_off = lo * 64u + ((hi ^ ((lo >> 1) & 3u)) << 4);

    const uint32_t m_begin = blockIdx.y * m_per_block;
    const uint32_t m_end = min(M, m_begin + m_per_block);
    const uint32_t ksteps = K >> 4;
    f32x4 acc[NB][4];

    {
        // a 512-element tile holds 512 / K whole columns (the operands leave the tile's upper index
        // bits alone)
        TileOperands<BF16> ops;
        make_tile_operands<BF16, 4>(logK, ops);
        const uint32_t block_tiles = (BN * K) >> 9;
        const uint64_t total = (uint64_t)N * K;
        for (uint32_t t0 = wave; t0 < block_tiles; t0 += kWaves) {
            float in[8];
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                // element e of the block's transformed tile: column e >> logK, k = e % K
                const uint32_t e = t0 * 512u + 256u * t + 4u * lane;
                const uint64_t off = (uint64_t)(n0 + (e >> logK)) * K + (e & (K - 1u));
                f32x4 q = {0.f, 0.f, 0.f, 0.f};
                if (off + 4u <= total) q = *reinterpret_cast<const f32x4*>(Xt + off);
#pragma unroll
                for (int r = 0; r < 4; ++r) in[4 * t + r] = q[r];
            }
            f32x4 y[2];
            tile_transform_f32(in, ops, y);
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                const uint32_t e = t0 * 512u + 256u * t + 4u * lane;
                const uint32_t n = e >> logK, q = (e & (K - 1u)) >> 2;
                *reinterpret_cast<f32x4*>(ylds + y_off<LOG_NB>(n, q, col_bytes, swz_mask)) = y[t] * fscale;
            }
        }
    }
    __syncthreads();

    for (uint32_t mb = m_begin + wave * 64u; mb < m_end; mb += kWaves * 64u) {
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
            for (int mi = 0; mi < 4; ++mi) acc[nb][mi] = f32x4{0.f, 0.f, 0.f, 0.f};
        // W goes global -> registers with four adjacent lanes on the 64 contiguous bytes a row
        // contributes to a K step (the pattern the L1 coalesces; one lane per row, which is what
        // the MFMA operand wants, runs at a third of the rate), then through a wavefront-private
        // 4 KB LDS area into operand order.  Piece mi of the wavefront holds rows 16 mi + lane/4,
        // 16-byte chunk lane%4; reader lane (hi, lo) takes row 16 mi + lo, chunk hi.  LDS
        // operations of one wavefront complete in order, so no barrier is needed.
        const float* wsrc[4];
#pragma unroll
        for (int mi = 0; mi < 4; ++mi) {
            const uint32_t m = min(mb + 16u * mi + (lane >> 2), M - 1u);
            wsrc[mi] = W + (uint64_t)m * K + 4u * (lane & 3u);
        }
        // Software pipeline: while step kk is multiplied, the fragments of step kk+1 are already
        // on their way out of LDS and the W pieces of step kk+2 are in flight from memory.
        f32x4 wreg[4];   // W pieces of the step after the one whose fragments are being fetched
        f32x4 a_nx[NB], b_nx[4];
        auto fetch = [&](uint32_t kk) {  // wreg (step kk) -> staging -> fragments of step kk
#pragma unroll
            for (int mi = 0; mi < 4; ++mi)
                *reinterpret_cast<f32x4*>(stage + mi * 1024u + wr_off) = wreg[mi];
#pragma unroll
            for (int nb = 0; nb < NB; ++nb)
                a_nx[nb] = *reinterpret_cast<const f32x4*>(
                    ylds + y_off<LOG_NB>(NB * lo + nb, 4u * kk + hi, col_bytes, swz_mask));
#pragma unroll
            for (int mi = 0; mi < 4; ++mi)
                b_nx[mi] = *reinterpret_cast<const f32x4*>(stage + mi * 1024u + rd_off);
        };
        auto gload = [&](uint32_t kk) {
#pragma unroll
            for (int mi = 0; mi < 4; ++mi)
                wreg[mi] = *reinterpret_cast<const f32x4*>(wsrc[mi] + 16u * kk);
        };
        gload(0);
        fetch(0);
        gload(1);  // K >= 32: at least two steps
        for (uint32_t kk = 0; kk < ksteps; ++kk) {
            f32x4 a[NB], b[4];
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) a[nb] = a_nx[nb];
#pragma unroll
            for (int mi = 0; mi < 4; ++mi) b[mi] = b_nx[mi];
            if (kk + 1 < ksteps) {
                fetch(kk + 1);
                if (kk + 2 < ksteps) gload(kk + 2);
            }
#pragma unroll
            for (int s = 0; s < 4; ++s)
#pragma unroll
                for (int nb = 0; nb < NB; ++nb)
#pragma unroll
                    for (int mi = 0; mi < 4; ++mi)
                        acc[nb][mi] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[nb][s], b[mi][s],
                                                                           acc[nb][mi], 0, 0, 0);
        }

#pragma unroll
        for (int mi = 0; mi < 4; ++mi) {
            const uint32_t m = mb + 16u * mi + lo;
            if (m >= m_end) continue;
            const uint32_t col0 = n0 + (4u * NB) * hi;
            if (col0 >= N) continue;
            const uint32_t ncols = min((uint32_t)(4 * NB), N - col0);
            float* p = C + (uint64_t)m * N + col0;
#pragma unroll
            for (int r = 0; r < 4; ++r)
#pragma unroll
                for (int nb = 0; nb < NB; ++nb)
                    if ((uint32_t)(NB * r + nb) < ncols) p[NB * r + nb] = acc[nb][mi][r];
        }
    }
}

template <int BN>
int launch(const float* W, const float* Xt, float* C, uint32_t M, uint32_t N, uint32_t K,
           float scale, hipStream_t s)
{
    const uint32_t logK = ilog2(K);
    const int shift = tile_stage_shift<4>(logK, false);
    const float fscale = (float)((double)scale * (double)(1u << shift));
    const uint32_t n_tiles = (N + BN - 1) / BN;
    const uint32_t row_blocks = (M + 511u) / 512u;
    // one workgroup per compute unit fits (LDS): aim at one round of 256 workgroups
    uint32_t msplit = (256u + n_tiles - 1u) / n_tiles;
    if (msplit < 1u) msplit = 1u;
    if (msplit > row_blocks) msplit = row_blocks;
    uint32_t m_per_block = ((row_blocks + msplit - 1u) / msplit) * 512u;
    msplit = (M + m_per_block - 1u) / m_per_block;
    const size_t lds = (size_t)BN * K * 4u + (size_t)kWaves * kStageBytes;
    auto kern = fused_ht_gemm_f32_kernel<BN>;
    if (lds > 64u * 1024u) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
            return MI_ERR_LAUNCH;
    }
    hipLaunchKernelGGL(kern, dim3(n_tiles, msplit), dim3(kThreads), lds, s, W, Xt, C, M, N, K, logK,
                       m_per_block, fscale);
    return launch_status();
}

}  // namespace

int fused_gemm_f32(const float* W, const float* Xt, float* C, uint32_t M, uint32_t N, uint32_t K,
                   float scale, hipStream_t s)
{
    // Small and medium outputs: the GEMV kernels, 16 columns per workgroup.  The GEMM kernels give a
    // workgroup 64 columns or more (256 at K = 256), which pays once every workgroup walks many row
    // blocks; below that their prologue and their few, long workgroups cost more than they save.
    // Measured, GEMV route against GEMM kernel, us:
    //   K = 64: 512^2 11.3 / 15.1, 2048^2 17.8 / 20.0;  K = 128: 1024^2 11.4 / 19.5, 2048^2 26.3 / 23.6;
    //   K = 256 (64 columns per workgroup from 128 pairs of 64 columns x 64 rows on): 512^2 11.7 / 29.9,
    //   1024^2 11.3 / 30.5, 2048^2 24.7 / 31.9, 4096^2 72.0 / 79.7, 8192^2 255.8 / 258.0: every shape;
    //   K = 512: 512^2 9.4 / 30.0, 1024^2 14.2 / 30.5, 2048^2 39.6 / 45.1, 3072^2 87.2 / 88.8, 4096^2 134.9 /
    //   133.8, 8192 x 1024 71.9 / 74.8, 1024 x 8192 77.2 / 74.4;  K = 1024: 512^2 12.1 / 30.5, 1024^2 23.6 /
    //   30.6, 2048^2 71.2 / 76.0, 3072^2 157.9 / 162.6, 4096^2 255.5 / 246.9;
    //   K = 2048: 512^2 19.2 / 32.5, 1024^2 43.9 / 47.6, 2048^2 136.5 / 136.5, 4096^2 509 / 492.
    {
        const uint64_t groups = (uint64_t)((N + 15u) / 16u) * ((M + 63u) / 64u);  // >= 256: the large-shape GEMV kernels
        const uint64_t outputs = (uint64_t)M * N;
        bool by_gemv = false;
        if (K == 256u)
            by_gemv = true;
        else if (K < 256u)
            by_gemv = outputs <= 1536ull * 1024ull;
        else if (K <= 1024u)
            by_gemv = groups >= 256u && N <= 4096u && outputs <= 3072ull * 3072ull;
        else if (K == 2048u)
            by_gemv = groups >= 256u && N <= 4096u && outputs < 2048ull * 2048ull;
        if (by_gemv) return gemv::launch_any(W, Xt, C, M, K, N, scale, true, s);
    }
    switch (K) {
        case 32:
        case 64:
        case 128: return launch<32>(W, Xt, C, M, N, K, scale, s);
        case 512:
        case 1024:
        case 2048:
        case 4096: return fused_gemm_f32_xreg(W, Xt, C, M, N, K, scale, s);
        default: return MI_ERR_SIZE;
    }
}

}  // namespace mi
