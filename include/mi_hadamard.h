/*
 * mi_hadamard.h -- C ABI of the MI355X (gfx950) fast Hadamard transform library.
 *
 * Plain pointers and sizes only; no torch or HIP types appear in the signatures (`stream` is a
 * hipStream_t passed as void*, NULL = the null stream).  Every entry point
 *   - enqueues its kernels on `stream` and returns without synchronising,
 *   - allocates no device memory and keeps no mutable global state (safe from any host thread),
 *   - returns MI_OK (0) or a negative mi_status; mi_status_string() turns it into text.
 * All matrices are dense row-major with no padding between rows.
 */
#ifndef MI_HADAMARD_H
#define MI_HADAMARD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum mi_dtype {
    MI_F32 = 0,
    MI_BF16 = 1,
    MI_F16 = 2,
} mi_dtype;

typedef enum mi_status {
    MI_OK = 0,
    MI_ERR_DTYPE = -1,     /* dtype code not supported by this entry point            */
    MI_ERR_SIZE = -2,      /* transform length not a power of two in the valid range  */
    MI_ERR_ALIGN = -3,     /* a pointer is not 16-byte aligned                        */
    MI_ERR_NULL = -4,      /* a required pointer is NULL                              */
    MI_ERR_SHAPE = -5,     /* a dimension violates the entry point's tiling contract  */
    MI_ERR_LAUNCH = -6,    /* hipGetLastError() reported a launch failure             */
    MI_ERR_ALIAS = -7,     /* input/output overlap that the entry point cannot honour */
} mi_status;

/* Library version (major*10000 + minor*100 + patch). */
int mi_version(void);

/* Text for a status code; never NULL. */
const char* mi_status_string(int status);

/*
 * Walsh-Hadamard transform over the last dimension:  out[r, :] = scale * H_n * in[r, :]
 * for r in [0, rows), H_n the Sylvester matrix H[i][j] = (-1)^popcount(i & j).
 *
 * Replaces the reference's internal seam
 *     template<DType> void run_fht(void* a, void* out, uint32_t numel, uint32_t had_size,
 *                                  cudaStream_t)                 csrc/main.cuh:5-6,
 *                                                                HadaCore/hadamard_transform.cpp:8-9
 * which its pybind op hadamard_transform(x, inplace) calls (csrc/hadamard_transform.cpp:49-59).
 * Differences: `rows` is 64-bit (the reference's numel is u32); any row count is accepted (the
 * reference pads numel to a multiple of 256 first, csrc/hadamard_transform.cpp:31-39); fp32 is
 * accepted; `scale` is explicit (the reference hard-wires n^-1/2 in its kernel constants,
 * HadaCore/hadamard_transform_cuda.cu:139-142).
 *
 *   in, out : device pointers, 16-byte aligned, rows*n elements; in == out is allowed
 *             (in place); partial overlap is not.
 *   n       : power of two, 1 <= n <= 32768.
 *   dtype   : mi_dtype.  bf16/fp16 accumulate in fp32 on the matrix cores and round to the
 *             storage type between MFMA stages and at the store; fp32 stays fp32 throughout.
 */
int mi_fwht(const void* in, void* out, uint64_t rows, uint32_t n, int dtype, float scale,
            void* stream);

/*
 * Fused Hadamard + GEMV-batch:  Y[M,B] = W[M,N] * (scale * H_N * X[N,B]),
 * the transform running down each column of X (dimension 0).
 *
 * Replaces  fused_hadamard_gemv_kernel(const float* W, const float* X, float* Y, int M, int N,
 * int B)  and its _vec variant, fused_ht/fwht_gemv_fusion.cu:98-105,176-183, launched from
 * benchmark_fused (:371-420).  Layouts are the ones that file indexes: X[i*B + b] (:50-51),
 * W[row*N + k] (:146), Y[row*B + b] (:156).  scale = 1 reproduces the reference (raw +-1
 * butterfly, :118-133).
 *
 *   dtype : MI_F32 only.   N : power of two, 2 <= N <= 2048 (the 16-column tile of the
 *   transformed operand must fit in LDS).   M, B >= 1.
 *   Y must not overlap W or X.
 */
int mi_fused_ht_gemv(const void* W, const void* X, void* Y, uint32_t M, uint32_t N, uint32_t B,
                     int dtype, float scale, void* stream);

/*
 * Fused Hadamard -> GEMM:  C[M,N] = W[M,K] * (scale * H_K * X[K,N]),  X given as Xt[N,K]
 * (each logical column of X contiguous).  The transformed operand never goes to HBM.
 *
 * Replaces  fused_ht_gemm_pipelined(const float* X, const float* W, float* C)  with compile-time
 * KDIM/NDIM/MDIM, fused_ht/fusion_pipelined.cu:306-310, launched at :662-683.  Layouts:
 * X[col*KDIM + k] (:164,612), W[row*KDIM + k] (:211,498), C[row*NDIM + col] (:220,558).
 * scale = 1 reproduces the reference.
 *
 *   in_dtype  : MI_F32 (fp32 MFMA) or MI_BF16 / MI_F16 (16-bit MFMA, fp32 accumulate).
 *   out_dtype : MI_F32, or the same 16-bit type as in_dtype.
 *   K : power of two, 32 <= K <= 4096.   M, N >= 1 (edge tiles are masked).
 *   The register-resident kernels (16-bit inputs with K >= 512, MI_F32 with K >= 256) address W
 *   with 32-bit byte offsets: W larger than 4 GiB, or N >= 2^24, is MI_ERR_SHAPE.
 * K = 4096 enqueues two kernels on `stream` for every dtype (the second adds to what the first
 * stored in C, so nothing else may touch C between them); every other case is one kernel.
 * Precision at K = 4096: each kernel accumulates its half of the K range in fp32.  With MI_F32
 * output the halves meet in fp32 (one more fp32 rounding than a single pass).  With 16-bit output
 * the first kernel stores its half-K sum P0 rounded to the 16-bit type and the second adds its own
 * half P1, rounded to 16 bits, in 16-bit arithmetic (a packed add performed by the L2; masked edge
 * blocks add in fp32 and round once), so the result carries up to three 16-bit roundings instead of
 * the single one of K <= 2048:
 *     |C - exact| <= ulp16(P0) + ulp16(P1) + ulp16(C),   ulp16(v) = the 16-bit type's spacing at |v|,
 * which is a larger *relative* error than usual when P0 and P1 nearly cancel, and for MI_F16 a half-K
 * sum beyond 65504 becomes infinite even if the total is representable.  Callers that need the
 * single rounding ask for MI_F32 output.
 */
int mi_fused_ht_gemm(const void* W, const void* Xt, void* C, uint32_t M, uint32_t N, uint32_t K,
                     int in_dtype, int out_dtype, float scale, void* stream);

/*
 * Randomized Hadamard + FP8 quantize:  y[t,:] = scale * H_n * (sign .* x[t,:]) rounded to bf16,
 * then per row   amax = max|y|,  a = max(amax, 1e-30f),  row_scale[t] = a / 448,
 * q[t,j] = e4m3fn_rne(clamp(y[t,j] * (448 / a), -448, 448))   (OCP E4M3FN; IEEE fp32 ops; for
 * finite y the clamp never changes a value because |y| <= amax).
 *
 * No counterpart in the reference (it has no FP8 path); part of the build contract's hot path.
 *
 *   x         : bf16 [T,n];  n power of two, 16 <= n <= 4096.
 *   sign      : int8 [n], entries +1 / -1.
 *   q         : uint8 [T,n] E4M3FN codes.      row_scale : fp32 [T] (dequantisation factors).
 *   y_out     : optional bf16 [T,n] dump of the pre-quant values (NULL to skip).
 */
int mi_rht_quant_fp8(const void* x, const int8_t* sign, void* q, float* row_scale, void* y_out,
                     uint64_t T, uint32_t n, float scale, void* stream);

/*
 * FP8 GEMM with per-row scales:  out[T,N] = bf16( (qa[T,K] . qb[N,K]^T) * sa[t] * sb[n] ),
 * E4M3FN operands, fp32 accumulate.  No counterpart in the reference.
 *   K multiple of 128;  T, N >= 1.
 */
int mi_fp8_gemm_rowscale(const void* qa, const float* sa, const void* qb, const float* sb,
                         void* out, uint32_t T, uint32_t N, uint32_t K, void* stream);

/*
 * One-wavefront MFMA layout check:  D[16,16] = A[16,Kk] * B[Kk,16]  with exactly one matrix-core
 * instruction, operands gathered under the register layout the kernels assume.
 * Mirrors the reference's test hook  test_mma_m16_n8_k16(x, y)  (csrc/test_frag.cu:8-62,
 * exported at csrc/hadamard_transform.cpp:83-89).
 *   kind 0: v_mfma_f32_16x16x32_bf16 (Kk = 32)    kind 1: v_mfma_f32_16x16x16_bf16 (Kk = 16)
 *   kind 2: v_mfma_f32_16x16x32_f16  (Kk = 32)    kind 3: v_mfma_f32_16x16x16_f16  (Kk = 16)
 *   kind 4: v_mfma_f32_16x16x4_f32   (Kk = 4, A and B fp32)
 *   A, B: row-major, element type per kind;  D: fp32 row-major.
 */
int mi_debug_mfma_16x16(int kind, const void* A, const void* B, float* D, void* stream);

/*
 * Element-wise narrowing conversions as the kernels perform them (hardware RNE), for unit tests
 * (the reference's  test_bit_convert, csrc/test_bit.cu:8-42).
 *   kind 0: fp32 -> bf16 bits (uint16)    kind 1: fp32 -> fp16 bits (uint16)
 *   kind 2: fp32 -> E4M3FN code (uint8), input clamped to +-448 first
 */
int mi_debug_convert(int kind, const float* in, void* out, uint64_t count, void* stream);

/*
 * Same contract as mi_fwht, but computed by a minimal kernel written against the device-side
 * embedding API (csrc/hadamard_device.hpp: HadamardTransformDevice<IO, LOG_N>), one call of
 * hadamard_transform_device per workgroup.  Exists so the embedding API -- the counterpart of the
 * reference's  HadamardTransform<dtype,N>::hadamard_transform_device  (csrc/hada_handler.cuh:
 * 227-264, thin caller csrc/main.cu:42-53) -- is tested for every length and element type.
 *   rows must be a multiple of the API's N_ROWS (512 / n for n <= 512, else 1): MI_ERR_SHAPE.
 */
int mi_debug_device_fwht(const void* in, void* out, uint64_t rows, uint32_t n, int dtype,
                         float scale, void* stream);

/*
 * Host-only: how mi_fused_ht_gemm cuts a 16-bit problem with K = 512 ... 4096 into workgroups (no
 * GPU call; MI_ERR_SIZE for any other K).
 * The (column group, M slice) grid, the XCD rectangles and the map from workgroup id to tile are
 * what decides L2 reuse and the number of launch rounds; this hook lets a test check on the CPU
 * that every tile is handled by exactly one workgroup.  No counterpart in the reference.
 *   header[8] : ngroups (groups of 131072 / K columns, 64 at K = 4096), msplit (M slices), m_per_block (rows per slice),
 *               mpx, cgx (rectangle extents in M slices and column groups), nrect, grid
 *               (workgroups launched), 0
 *   tiles     : NULL, or 2 * capacity uint32: for workgroup id i, tiles[2i] = column group and
 *               tiles[2i+1] = M slice, or 0xffffffff twice for an id without work
 * Returns MI_ERR_SIZE when capacity < grid (header is filled in either way).
 */
int mi_debug_fused_gemm_tiling(uint32_t M, uint32_t N, uint32_t K, uint32_t* header, uint32_t* tiles,
                               uint32_t capacity);

#ifdef __cplusplus
}
#endif
#endif /* MI_HADAMARD_H */
