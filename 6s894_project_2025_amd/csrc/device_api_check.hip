// A minimal kernel written against the device-side embedding API (hadamard_device.hpp), exported
// as mi_debug_device_fwht so the API itself is tested for every length and element type, not only
// through the tuned stand-alone kernels.  Same role as the reference's thin caller
// hadamard_transform_ker (csrc/main.cu:42-53) around hadamard_transform_device.
#include "hadamard_device.hpp"

namespace mi {
namespace {

template <class HT>
__global__ void __launch_bounds__(HT::THREADS)
device_api_kernel(const typename HT::T* in, typename HT::T* out, OutputScale os)
{
    extern __shared__ f32x4 lds[];
    const typename HT::Operands ops = HT::prepare(os);
    const uint64_t off = (uint64_t)blockIdx.x * HT::N_ROWS * HT::N;
    HT::hadamard_transform_device(in + off, out + off, lds, ops, os);
}

template <class IO, int LOG_N>
int launch_one(const void* in, void* out, uint64_t rows, float scale, hipStream_t s)
{
    using HT = HadamardTransformDevice<IO, LOG_N>;
    if (rows % HT::N_ROWS != 0) return MI_ERR_SHAPE;
    const uint64_t calls = rows / HT::N_ROWS;
    if (calls > 0x7fffffffull) return MI_ERR_SHAPE;
    auto kern = device_api_kernel<HT>;
    if (HT::LDS_BYTES > 64 * 1024) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                hipFuncAttributeMaxDynamicSharedMemorySize,
                                HT::LDS_BYTES) != hipSuccess)
            return MI_ERR_LAUNCH;
    }
    hipLaunchKernelGGL(kern, dim3((uint32_t)calls), dim3(HT::THREADS), HT::LDS_BYTES, s,
                       static_cast<const typename HT::T*>(in), static_cast<typename HT::T*>(out),
                       output_scale<IO, LOG_N>(scale));
    return launch_status();
}

template <class IO, int LOG_N = 0>
int launch_any(uint32_t p, const void* in, void* out, uint64_t rows, float scale, hipStream_t s)
{
    if constexpr (LOG_N > 15) {
        return MI_ERR_SIZE;
    } else {
        if (p == (uint32_t)LOG_N) return launch_one<IO, LOG_N>(in, out, rows, scale, s);
        return launch_any<IO, LOG_N + 1>(p, in, out, rows, scale, s);
    }
}

}  // namespace
}  // namespace mi

extern "C" int mi_debug_device_fwht(const void* in, void* out, uint64_t rows, uint32_t n, int dtype,
                                    float scale, void* stream)
{
    using namespace mi;
    if (!is_pow2(n) || n > 32768u) return MI_ERR_SIZE;
    if (rows == 0) return MI_OK;
    if (!in || !out) return MI_ERR_NULL;
    if (!aligned16(in) || !aligned16(out)) return MI_ERR_ALIGN;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const uint32_t p = ilog2(n);
    switch (dtype) {
        case MI_F32: return launch_any<Io32>(p, in, out, rows, scale, s);
        case MI_BF16: return launch_any<Io16<BF16>>(p, in, out, rows, scale, s);
        case MI_F16: return launch_any<Io16<F16>>(p, in, out, rows, scale, s);
        default: return MI_ERR_DTYPE;
    }
}
