/*
 * CPU oracle for the Hadamard hot path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain C, the arithmetic the reference defines for
 *   - the normalised Walsh-Hadamard transform over the last dimension,
 *   - the fused  Y = W * H(X)  (HT+GEMV)  and  C = W * H(X)  (HT->GEMM) products,
 *   - IEEE round-to-nearest-even fp32 -> bf16 / fp16 conversion,
 * and defines (the reference has no counterpart) the randomized-Hadamard FP8 e4m3fn
 * quantizer with per-row amax scales.
 *
 * Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may build, load or
 * call it, and only as the checker.  The shipped library never links or calls it.
 *
 * Pinning status (each function is checked by tests/test_oracle.py against something other
 * than its own formula):
 *   oracle_sylvester           scipy.linalg.hadamard, H*H = n*I, Kronecker recursion
 *   oracle_fwht_*              brute-force matrix product with oracle_sylvester / scipy,
 *                              involution, Parseval, unit vectors, constant vector
 *   oracle_fused_ht_gemv_f64   numpy  W @ (s*H @ X);  W = I reduces to the transform
 *   oracle_fused_ht_gemm_f64   numpy  W @ (s*H @ Xt.T);  W = I reduces to the transform
 *   oracle_f32_to_bf16/f16     torch CPU  .to(bfloat16) / .to(float16)  on dense bit sweeps
 *   oracle_e4m3fn_encode       torch CPU  .to(float8_e4m3fn)  on every finite |x| <= 448 bf16
 *                              value and a dense fp32 sweep; format definition (OCP FP8)
 *   oracle_rht_quant_fp8       PARITY UNPINNED BY THE REFERENCE (it has no FP8 path); pinned
 *                              only by the two functions above plus numpy amax / division
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ---- Sylvester matrix ------------------------------------------------------------------ */
/* H[i][j] = (-1)^popcount(i & j): the sign rule of csrc/hada.cuh:62-83 (entry sign is the
 * parity of sum k_i & m_i over rotated axes) and the matrix scipy.linalg.hadamard builds,
 * which HadaCore/test.py:27 and bench/bench.py:51 take as the definition of correct. */
void oracle_sylvester(uint32_t n, int8_t* H)
{
    for (uint32_t i = 0; i < n; ++i)
        for (uint32_t j = 0; j < n; ++j)
            H[(size_t)i * n + j] = (__builtin_popcount(i & j) & 1) ? -1 : 1;
}

/* ---- transform over the last dimension ---------------------------------------------------- */
/* In-place butterfly, stride h = 1, 2, ..., n/2, pairs (j, j+h):
 * the serial loop of fused_ht/fusion_pipelined.cu:117-129, then one multiply by `scale`
 * (the reference's torch op always uses n^-1/2, HadaCore/test.py:24-27,40). */
void oracle_fwht_f64(double* x, uint64_t rows, uint32_t n, double scale)
{
    for (uint64_t r = 0; r < rows; ++r) {
        double* v = x + r * (uint64_t)n;
        for (uint32_t h = 1; h < n; h <<= 1)
            for (uint32_t i = 0; i < n; i += (h << 1))
                for (uint32_t j = i; j < i + h; ++j) {
                    double a = v[j], b = v[j + h];
                    v[j] = a + b;
                    v[j + h] = a - b;
                }
        for (uint32_t j = 0; j < n; ++j) v[j] *= scale;
    }
}

/* Same loop in fp32 arithmetic: the scalar CPU port that bench.py can time. */
void oracle_fwht_f32(float* x, uint64_t rows, uint32_t n, float scale)
{
    for (uint64_t r = 0; r < rows; ++r) {
        float* v = x + r * (uint64_t)n;
        for (uint32_t h = 1; h < n; h <<= 1)
            for (uint32_t i = 0; i < n; i += (h << 1))
                for (uint32_t j = i; j < i + h; ++j) {
                    float a = v[j], b = v[j + h];
                    v[j] = a + b;
                    v[j + h] = a - b;
                }
        for (uint32_t j = 0; j < n; ++j) v[j] *= scale;
    }
}

/* y = x @ (H_n * scale) by brute force: the truth path of HadaCore/test.py:40 and
 * bench/bench.py:55-59, in fp64.  O(rows * n^2): small cases only. */
void oracle_fwht_matrix_f64(const double* x, double* y, uint64_t rows, uint32_t n, double scale)
{
    for (uint64_t r = 0; r < rows; ++r)
        for (uint32_t j = 0; j < n; ++j) {
            double acc = 0.0;
            for (uint32_t i = 0; i < n; ++i) {
                double v = x[r * (uint64_t)n + i];
                acc += (__builtin_popcount(i & j) & 1) ? -v : v;
            }
            y[r * (uint64_t)n + j] = acc * scale;
        }
}

/* ---- fused HT + GEMV --------------------------------------------------------------------- */
/* Y[M,B] = W[M,N] * (scale * H_N * X[N,B]), all row-major as INDEXED by the reference:
 * X[i*B + b] (fused_ht/fwht_gemv_fusion.cu:50-51), W[row*N + k] (:146), Y[row*B + b] (:156).
 * The transform runs down each column of X (dim 0).  The reference applies the raw +-1
 * butterfly (:118-133), i.e. scale = 1. */
void oracle_fused_ht_gemv_f64(const double* W, const double* X, double* Y, uint32_t M,
                              uint32_t N, uint32_t B, double scale)
{
    double* col = (double*)malloc(sizeof(double) * N);
    for (uint32_t b = 0; b < B; ++b) {
        for (uint32_t i = 0; i < N; ++i) col[i] = X[(size_t)i * B + b];
        oracle_fwht_f64(col, 1, N, scale);
        for (uint32_t m = 0; m < M; ++m) {
            double acc = 0.0;
            for (uint32_t k = 0; k < N; ++k) acc += W[(size_t)m * N + k] * col[k];
            Y[(size_t)m * B + b] = acc;
        }
    }
    free(col);
}

/* ---- fused HT -> GEMM -------------------------------------------------------------------- */
/* C[M,N] = W[M,K] * (scale * H_K * X[K,N]) with X stored as Xt[N,K] row-major, i.e. each
 * logical column of X is contiguous: X[col*KDIM + k] (fused_ht/fusion_pipelined.cu:164,612),
 * W[row*KDIM + k] (:211,498), C[row*NDIM + col] (:220,558).  Reference scale = 1 (:85-106). */
void oracle_fused_ht_gemm_f64(const double* W, const double* Xt, double* C, uint32_t M,
                              uint32_t N, uint32_t K, double scale)
{
    double* col = (double*)malloc(sizeof(double) * K);
    for (uint32_t c = 0; c < N; ++c) {
        memcpy(col, Xt + (size_t)c * K, sizeof(double) * K);
        oracle_fwht_f64(col, 1, K, scale);
        for (uint32_t m = 0; m < M; ++m) {
            double acc = 0.0;
            for (uint32_t k = 0; k < K; ++k) acc += W[(size_t)m * K + k] * col[k];
            C[(size_t)m * N + c] = acc;
        }
    }
    free(col);
}

/* ---- IEEE RNE narrowing conversions ------------------------------------------------------- */
/* Semantics of the reference's constexpr converter (csrc/utils.cuh:181-261): round to nearest,
 * ties to even, subnormals, overflow to inf, NaN stays NaN (quiet). */
static inline uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

uint16_t oracle_f32_to_bf16(float f)
{
    uint32_t u = f32_bits(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb;
    return (uint16_t)(u >> 16);
}

float oracle_bf16_to_f32(uint16_t h) { return bits_f32((uint32_t)h << 16); }

uint16_t oracle_f32_to_f16(float f)
{
    uint32_t u = f32_bits(f);
    uint32_t sign = (u >> 16) & 0x8000u;
    uint32_t a = u & 0x7fffffffu;
    if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((a >> 13) & 0x3ffu));
    if (a >= 0x47800000u) return (uint16_t)(sign | 0x7c00u); /* >= 65536 -> inf (incl. inf) */
    if (a < 0x33000000u) return (uint16_t)sign;               /* < 2^-25 -> 0 */
    int32_t e = (int32_t)(a >> 23) - 127;
    uint32_t m = (a & 0x7fffffu) | 0x800000u;
    uint32_t shift, out;
    if (e < -14) {
        shift = (uint32_t)(13 + (-14 - e)); /* subnormal target */
        out = 0;
    } else {
        shift = 13;
        out = (uint32_t)(e + 15) << 10;
        m &= 0x7fffffu;
    }
    uint32_t q = m >> shift;
    uint32_t rem = m & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) q += 1; /* carry may bump the exponent: fine */
    out += q;
    return (uint16_t)(sign | out);
}

float oracle_f16_to_f32(uint16_t h)
{
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1fu, m = h & 0x3ffu;
    if (e == 0x1f) return bits_f32(sign | 0x7f800000u | (m << 13));
    if (e == 0) {
        float v = ldexpf((float)m, -24);
        return sign ? -v : v;
    }
    return bits_f32(sign | ((e + 112u) << 23) | (m << 13));
}

/* ---- FP8 E4M3FN (OCP): 1-4-3, bias 7, max 448, no inf, NaN = S.1111.111 --------------------- */
/* Round to nearest even; |x| above 448 saturates to 448 here (callers clamp first, so the
 * choice only matters for direct calls); NaN -> 0x7f | sign. */
uint8_t oracle_e4m3fn_encode(float f)
{
    uint32_t u = f32_bits(f);
    uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
    uint32_t a = u & 0x7fffffffu;
    if (a > 0x7f800000u) return (uint8_t)(sign | 0x7fu);
    float x = bits_f32(a);
    if (x >= 448.0f) return (uint8_t)(sign | 0x7eu);
    /* spacing: subnormals (below 2^-6) step 2^-9; normals step 2^(e-3) */
    int e;
    (void)frexpf(x, &e); /* x = m * 2^e, m in [0.5,1) -> floor(log2 x) = e-1 */
    int ex = e - 1;
    if (x == 0.0f) return sign;
    if (ex < -6) ex = -6;
    float step = ldexpf(1.0f, ex - 3);
    float q = x / step;          /* exact: power-of-two division */
    float r = nearbyintf(q);     /* default rounding mode: nearest even */
    float y = r * step;          /* representable e4m3 magnitude (maybe next binade) */
    if (y >= 448.0f) y = 448.0f;
    if (y == 0.0f) return sign;
    int e2;
    float m2 = frexpf(y, &e2); /* y = m2 * 2^e2, m2 in [0.5,1) */
    int ey = e2 - 1;
    if (ey < -6) {
        uint32_t mant = (uint32_t)(y / ldexpf(1.0f, -9));
        return (uint8_t)(sign | mant);
    }
    uint32_t mant = (uint32_t)((m2 * 2.0f - 1.0f) * 8.0f);
    return (uint8_t)(sign | ((uint32_t)(ey + 7) << 3) | mant);
}

float oracle_e4m3fn_decode(uint8_t c)
{
    uint32_t e = (c >> 3) & 0xfu, m = c & 7u;
    float v;
    if (e == 0xf && m == 7) return NAN;
    if (e == 0) v = ldexpf((float)m, -9);
    else v = ldexpf(1.0f + (float)m / 8.0f, (int)e - 7);
    return (c & 0x80u) ? -v : v;
}

/* Per-row amax quantizer applied to already-computed pre-quant values y[T,n] (fp32 holding the
 * values the device rounds to, e.g. bf16-representable numbers).  Convention (fixed by this
 * build; the reference has no FP8 path):
 *   amax_r  = max_j |y_rj|
 *   a_r     = max(amax_r, 1e-30f)
 *   scale_r = a_r / 448.0f          (IEEE fp32 division)  -> dequant factor, stored
 *   inv_r   = 448.0f / a_r          (IEEE fp32 division)
 *   q_rj    = e4m3fn_rne( clamp(y_rj * inv_r, -448, 448) )   (fp32 multiply) */
void oracle_quant_fp8_rows(const float* y, uint8_t* q, float* row_scale, uint64_t T, uint32_t n)
{
    for (uint64_t r = 0; r < T; ++r) {
        const float* v = y + r * (uint64_t)n;
        float amax = 0.0f;
        for (uint32_t j = 0; j < n; ++j) {
            float a = fabsf(v[j]);
            if (a > amax) amax = a;
        }
        float a = amax > 1e-30f ? amax : 1e-30f;
        volatile float sc = a / 448.0f;
        volatile float inv = 448.0f / a;
        row_scale[r] = sc;
        for (uint32_t j = 0; j < n; ++j) {
            volatile float t = v[j] * inv;
            float c = t;
            if (c > 448.0f) c = 448.0f;
            if (c < -448.0f) c = -448.0f;
            q[r * (uint64_t)n + j] = oracle_e4m3fn_encode(c);
        }
    }
}

/* Randomized Hadamard: y = scale * H_n * (sign .* x) per row, in fp64, from fp32 input values
 * (the caller passes bf16-representable x).  sign[j] in {+1,-1}. */
void oracle_rht_f64(const float* x, const int8_t* sign, double* y, uint64_t T, uint32_t n,
                    double scale)
{
    for (uint64_t r = 0; r < T; ++r) {
        double* v = y + r * (uint64_t)n;
        for (uint32_t j = 0; j < n; ++j) v[j] = (double)x[r * (uint64_t)n + j] * (double)sign[j];
    }
    oracle_fwht_f64(y, T, n, scale);
}

/* ---- array forms of the scalar converters (ctypes convenience) ---------------------------- */
void oracle_f32_to_bf16_array(const float* x, uint16_t* y, uint64_t n)
{
    for (uint64_t i = 0; i < n; ++i) y[i] = oracle_f32_to_bf16(x[i]);
}
void oracle_f32_to_f16_array(const float* x, uint16_t* y, uint64_t n)
{
    for (uint64_t i = 0; i < n; ++i) y[i] = oracle_f32_to_f16(x[i]);
}
void oracle_f16_to_f32_array(const uint16_t* x, float* y, uint64_t n)
{
    for (uint64_t i = 0; i < n; ++i) y[i] = oracle_f16_to_f32(x[i]);
}
void oracle_e4m3fn_encode_array(const float* x, uint8_t* y, uint64_t n)
{
    for (uint64_t i = 0; i < n; ++i) y[i] = oracle_e4m3fn_encode(x[i]);
}
void oracle_e4m3fn_decode_array(const uint8_t* x, float* y, uint64_t n)
{
    for (uint64_t i = 0; i < n; ++i) y[i] = oracle_e4m3fn_decode(x[i]);
}
