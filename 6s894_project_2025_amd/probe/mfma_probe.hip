// Matrix-core throughput probe (mi_probe_mfma_rate), gfx950.  Built into libmi_probe.so, a
// measurement aid beside the product library: nothing in libmi_hadamard.so depends on it.
//
// What a kernel can get out of the matrix cores depends on more than the instruction's issue
// rate: the clock the chip sustains under the load (which depends on the operand data: random
// bit patterns draw more power than constant ones), how many wavefronts per SIMD issue MFMAs, and
// what else (LDS fragment reads) runs beside them.  This probe measures exactly that, so that the
// roofline fraction of the GEMM kernels can be read against a ceiling observed on the same box
// instead of the paper peak: every workgroup runs `steps` K steps of eight independent
// v_mfma_f32_16x16x32_bf16 (or four v_mfma_f32_32x32x16_bf16, the same flops) on operands taken
// from caller-supplied memory, optionally with four 16-byte-per-lane LDS fragment reads per step
// issued in the shadow of the MFMAs, and reports its elapsed shader clock cycles.
//
// No counterpart in the reference (it has no matrix-core kernels in its fused path).
#include "common.hpp"
#include "mi_probe.h"

namespace mi {
namespace {

template <int SHAPE, int READS>
__global__ void __launch_bounds__(1024)
mfma_probe_kernel(const unsigned char* __restrict__ operands, uint64_t* __restrict__ cycles,
                  uint32_t steps)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    // 32 KB of operand data into LDS (fragment source), two B operands per lane from memory
    for (uint32_t i = threadIdx.x; i < 32768u / 16u; i += blockDim.x)
        reinterpret_cast<u32x4*>(lds)[i] = reinterpret_cast<const u32x4*>(operands)[i];
    bf16x8 b[2];
    for (int i = 0; i < 2; ++i)
        b[i] = reinterpret_cast<const bf16x8*>(operands + 32768u)[(threadIdx.x * 2u + i) & 2047u];
    __syncthreads();
    const unsigned char* base = lds + (wave & 3u) * 4096u + lane * 16u;
    bf16x8 fr[4][4];
#pragma unroll
    for (int s = 0; s < 4; ++s)
#pragma unroll
        for (int m = 0; m < 4; ++m) fr[s][m] = *reinterpret_cast<const bf16x8*>(base + 1024u * m);
    f32x4 acc[8];
    f32x16 wide[2];
#pragma unroll
    for (int n = 0; n < 8; ++n) acc[n] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int n = 0; n < 2; ++n)
#pragma unroll
        for (int j = 0; j < 16; ++j) wide[n][j] = 0.f;

    const uint64_t t0 = __builtin_readcyclecounter();
    for (uint32_t it = 0; it < steps; it += 4u) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            if constexpr (SHAPE == 16) {
#pragma unroll
                for (int n = 0; n < 8; ++n) {
                    acc[n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fr[u][n >> 1], b[n & 1], acc[n], 0, 0, 0);
                    if (n < READS)
                        fr[(u + 2) & 3][n] = *reinterpret_cast<const bf16x8*>(
                            base + 1024u * n + ((it + u) & 1u) * 16384u);
                }
            } else {
#pragma unroll
                for (int n = 0; n < 4; ++n) {
                    wide[n & 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fr[u][n], b[n >> 1], wide[n & 1], 0, 0, 0);
                    if (n < READS)
                        fr[(u + 2) & 3][n] = *reinterpret_cast<const bf16x8*>(
                            base + 1024u * n + ((it + u) & 1u) * 16384u);
                }
            }
        }
    }
    float sum = 0.f;
#pragma unroll
    for (int n = 0; n < 8; ++n) sum += acc[n][0] + acc[n][3];
#pragma unroll
    for (int n = 0; n < 2; ++n) sum += wide[n][0] + wide[n][15];
    const uint64_t t1 = __builtin_readcyclecounter();
    // The oldest wavefront of a SIMD gets the matrix core first, so with several per SIMD they
    // finish one after the other: the workgroup's time is that of its slowest wavefront.
    __syncthreads();  // everyone is done with the fragment source
    uint64_t* slot = reinterpret_cast<uint64_t*>(lds);
    if (lane == 0) slot[wave] = t1 - t0;
    __syncthreads();
    // the sum keeps the MFMA chain alive; it is stored where the caller can ignore it
    if (threadIdx.x == 0) {
        uint64_t worst = 0;
        for (uint32_t w = 0; w < blockDim.x / 64u; ++w) worst = slot[w] > worst ? slot[w] : worst;
        cycles[blockIdx.x] = worst;
        cycles[gridDim.x + blockIdx.x] = (uint64_t)__builtin_bit_cast(uint32_t, sum);
    }
}

template <int SHAPE, int READS>
int launch_probe(const void* operands, uint64_t* cycles, uint32_t waves_per_simd, uint32_t steps,
                 hipStream_t s)
{
    auto kern = mfma_probe_kernel<SHAPE, READS>;
    // 150 KB of LDS: one workgroup per compute unit, so `waves_per_simd` is what it says
    constexpr int lds = 150 * 1024;
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                            hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess)
        return MI_ERR_LAUNCH;
    hipLaunchKernelGGL(kern, dim3(256), dim3(256u * waves_per_simd), lds, s,
                       static_cast<const unsigned char*>(operands), cycles, steps);
    return launch_status();
}

}  // namespace
}  // namespace mi

extern "C" int mi_probe_mfma_rate(int shape, int lds_reads, uint32_t waves_per_simd, uint32_t steps,
                                  const void* operands, uint64_t* cycles, void* stream)
{
    using namespace mi;
    if (!operands || !cycles) return MI_ERR_NULL;
    if (!aligned16(operands)) return MI_ERR_ALIGN;
    if (waves_per_simd != 1u && waves_per_simd != 2u && waves_per_simd != 4u) return MI_ERR_SHAPE;
    if (steps == 0 || (steps & 3u)) return MI_ERR_SHAPE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (shape == 16 && lds_reads == 0) return launch_probe<16, 0>(operands, cycles, waves_per_simd, steps, s);
    if (shape == 16 && lds_reads == 4) return launch_probe<16, 4>(operands, cycles, waves_per_simd, steps, s);
    if (shape == 32 && lds_reads == 0) return launch_probe<32, 0>(operands, cycles, waves_per_simd, steps, s);
    if (shape == 32 && lds_reads == 4) return launch_probe<32, 4>(operands, cycles, waves_per_simd, steps, s);
    return MI_ERR_SHAPE;
}
