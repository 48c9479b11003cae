// Version / status text and the one-wavefront debug hooks of the C ABI.
#include "common.hpp"

namespace mi {
namespace {

// One MFMA under the operand layout the kernels assume:
//   A (16 x Kk): lane l holds row l%16, columns (Kk/4)*(l/16) + j
//   B (Kk x 16): lane l holds column l%16, rows (Kk/4)*(l/16) + j
//   D (16 x 16): lane l holds column l%16, rows 4*(l/16) + r
template <class T16, int KK>
__global__ void __launch_bounds__(64) debug_mfma16_kernel(const typename T16::E* A,
                                                         const typename T16::E* B, float* D)
{
    const uint32_t lane = threadIdx.x, lo = lane & 15u, hi = lane >> 4;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    if constexpr (KK == 32) {
        typename T16::V8 a, b;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            a[j] = A[lo * 32u + 8u * hi + j];
            b[j] = B[(8u * hi + j) * 16u + lo];
        }
        acc = T16::mfma32(a, b, acc);
    } else {
        typename T16::V4 a, b;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            a[j] = A[lo * 16u + 4u * hi + j];
            b[j] = B[(4u * hi + j) * 16u + lo];
        }
        acc = T16::mfma16(a, b, acc);
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) D[(4u * hi + r) * 16u + lo] = acc[r];
}

__global__ void __launch_bounds__(64) debug_mfma_f32_kernel(const float* A, const float* B,
                                                           float* D)
{
    const uint32_t lane = threadIdx.x, lo = lane & 15u, hi = lane >> 4;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(A[lo * 4u + hi], B[hi * 16u + lo], acc, 0, 0, 0);
#pragma unroll
    for (int r = 0; r < 4; ++r) D[(4u * hi + r) * 16u + lo] = acc[r];
}

__global__ void debug_convert_kernel(int kind, const float* in, void* out, uint64_t count)
{
    const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= count) return;
    const float x = in[i];
    if (kind == 0) {
        static_cast<__bf16*>(out)[i] = (__bf16)x;
    } else if (kind == 1) {
        static_cast<_Float16*>(out)[i] = (_Float16)x;
    } else {
        const float c = __builtin_amdgcn_fmed3f(x, -448.0f, 448.0f);
        const int w = __builtin_amdgcn_cvt_pk_fp8_f32(c, c, 0, false);
        static_cast<uint8_t*>(out)[i] = (uint8_t)(w & 0xff);
    }
}

}  // namespace
}  // namespace mi

extern "C" int mi_version(void) { return 100; }

extern "C" const char* mi_status_string(int status)
{
    switch (status) {
        case MI_OK: return "ok";
        case MI_ERR_DTYPE: return "unsupported dtype for this entry point";
        case MI_ERR_SIZE: return "transform length must be a power of two in the supported range";
        case MI_ERR_ALIGN: return "pointer is not 16-byte aligned";
        case MI_ERR_NULL: return "null pointer";
        case MI_ERR_SHAPE: return "dimension violates the entry point's contract";
        case MI_ERR_LAUNCH: return "kernel launch failed";
        case MI_ERR_ALIAS: return "input and output overlap";
        default: return "unknown status";
    }
}

extern "C" int mi_debug_mfma_16x16(int kind, const void* A, const void* B, float* D, void* stream)
{
    using namespace mi;
    if (!A || !B || !D) return MI_ERR_NULL;
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (kind) {
        case 0:
            hipLaunchKernelGGL((debug_mfma16_kernel<BF16, 32>), dim3(1), dim3(64), 0, s,
                               static_cast<const __bf16*>(A), static_cast<const __bf16*>(B), D);
            break;
        case 1:
            hipLaunchKernelGGL((debug_mfma16_kernel<BF16, 16>), dim3(1), dim3(64), 0, s,
                               static_cast<const __bf16*>(A), static_cast<const __bf16*>(B), D);
            break;
        case 2:
            hipLaunchKernelGGL((debug_mfma16_kernel<F16, 32>), dim3(1), dim3(64), 0, s,
                               static_cast<const _Float16*>(A), static_cast<const _Float16*>(B), D);
            break;
        case 3:
            hipLaunchKernelGGL((debug_mfma16_kernel<F16, 16>), dim3(1), dim3(64), 0, s,
                               static_cast<const _Float16*>(A), static_cast<const _Float16*>(B), D);
            break;
        case 4:
            hipLaunchKernelGGL(debug_mfma_f32_kernel, dim3(1), dim3(64), 0, s,
                               static_cast<const float*>(A), static_cast<const float*>(B), D);
            break;
        default: return MI_ERR_DTYPE;
    }
    return launch_status();
}

extern "C" int mi_debug_convert(int kind, const float* in, void* out, uint64_t count, void* stream)
{
    using namespace mi;
    if (kind < 0 || kind > 2) return MI_ERR_DTYPE;
    if (count == 0) return MI_OK;
    if (!in || !out) return MI_ERR_NULL;
    const uint64_t blocks = (count + 255u) / 256u;
    if (blocks > 0x7fffffffull) return MI_ERR_SHAPE;
    hipLaunchKernelGGL(debug_convert_kernel, dim3((uint32_t)blocks), dim3(256), 0,
                       static_cast<hipStream_t>(stream), kind, in, out, count);
    return launch_status();
}
