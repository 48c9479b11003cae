// Instruction-issue probe (mi_probe_issue_rate), gfx950.  Built into libmi_probe.so.
//
// The register-resident GEMM kernels run one wavefront per SIMD, and how many instructions such a
// wavefront can issue beside its MFMAs decides what their main loops cost; the streaming kernels run
// two to four wavefronts per SIMD and are bound by how fast a SIMD issues vector instructions of each
// kind.  Both are properties of the chip that no document states; this probe measures them:
//   mode 0: every wavefront runs `reps` x 8 groups of [one v_mfma_f32_16x16x32_bf16 + n other
//           instructions of one kind] and reports shader clock cycles per group;
//   mode 1: no MFMA, `reps` x 64 independent instructions of one kind per wavefront, waves_per_simd
//           wavefronts on every SIMD of one compute unit: cycles per instruction and SIMD.
// No counterpart in the reference.
#include "common.hpp"
#include "mi_probe.h"

namespace mi {
namespace {

enum Kind { kVAdd = 0, kCvtPkBf16 = 1, kSAdd = 2, kDsRead = 3, kCvtPkFp8 = 4, kMax3 = 5, kLshl = 6, kKinds = 7 };

template <int KIND>
__device__ __forceinline__ void one(uint32_t& d, float a, float b, f32x4& sink, uint32_t lds_addr)
{
    if (KIND == kVAdd) asm volatile("v_add_f32 %0, %1, %2" : "=v"(d) : "v"(a), "v"(b));
    if (KIND == kCvtPkBf16) asm volatile("v_cvt_pk_bf16_f32 %0, %1, %2" : "=v"(d) : "v"(a), "v"(b));
    if (KIND == kSAdd) asm volatile("s_add_u32 s20, s21, 5" ::: "s20", "scc");
    if (KIND == kDsRead) asm volatile("ds_read_b128 %0, %1" : "=v"(sink) : "v"(lds_addr));
    if (KIND == kCvtPkFp8) asm volatile("v_cvt_pk_fp8_f32 %0, %1, %2" : "=v"(d) : "v"(a), "v"(b));
    if (KIND == kMax3) asm volatile("v_max3_f32 %0, |%1|, |%2|, %1" : "=v"(d) : "v"(a), "v"(b));
    if (KIND == kLshl) asm volatile("v_lshlrev_b32 %0, 16, %1" : "=v"(d) : "v"(a));
}

template <int KIND, int N, bool WITH_MFMA>
__global__ void __launch_bounds__(1024)
issue_probe_kernel(const float* __restrict__ in, float* __restrict__ out, uint64_t* __restrict__ cycles, uint32_t reps)
{
    __shared__ float sm[4096];
    float a[8];
    for (int i = 0; i < 8; ++i) a[i] = in[(threadIdx.x & 255u) * 8u + i];
    sm[threadIdx.x] = a[0];
    bf16x8 A, B;
    for (int i = 0; i < 8; ++i) {
        A[i] = (__bf16)a[i];
        B[i] = (__bf16)a[7 - i];
    }
    f32x4 acc[8], sink = {0.f, 0.f, 0.f, 0.f};
    for (int i = 0; i < 8; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
    uint32_t d[4] = {0u, 0u, 0u, 0u};
    const uint32_t lds_addr = (threadIdx.x & 255u) * 16u;
    __syncthreads();
    const uint64_t t0 = __builtin_readcyclecounter();
#pragma unroll 1
    for (uint32_t r = 0; r < reps; ++r) {
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            if (WITH_MFMA) asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+v"(acc[u]) : "v"(A), "v"(B));
#pragma unroll
            for (int i = 0; i < (WITH_MFMA ? N : 8); ++i) one<KIND>(d[i & 3], a[2 * (i & 3)], a[2 * (i & 3) + 1], sink, lds_addr);
        }
        if (KIND == kDsRead) asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    }
    const uint64_t t1 = __builtin_readcyclecounter();
    float s = sink[0] + sink[3];
    for (int i = 0; i < 8; ++i) s += acc[i][0] + acc[i][3];
    out[threadIdx.x] = s + (float)(d[0] ^ d[1] ^ d[2] ^ d[3]);
    if ((threadIdx.x & 63u) == 0) cycles[threadIdx.x >> 6] = t1 - t0;
}

template <int KIND, int N, bool WITH_MFMA>
int launch(const float* in, float* out, uint64_t* cycles, uint32_t waves_per_simd, uint32_t reps, hipStream_t s)
{
    hipLaunchKernelGGL((issue_probe_kernel<KIND, N, WITH_MFMA>), dim3(1), dim3(256u * waves_per_simd), 0, s, in,
                       out, cycles, reps);
    return launch_status();
}

template <int KIND>
int launch_with_mfma(int n, const float* in, float* out, uint64_t* cycles, uint32_t reps, hipStream_t s)
{
    switch (n) {
        case 0: return launch<KIND, 0, true>(in, out, cycles, 1u, reps, s);
        case 1: return launch<KIND, 1, true>(in, out, cycles, 1u, reps, s);
        case 2: return launch<KIND, 2, true>(in, out, cycles, 1u, reps, s);
        case 3: return launch<KIND, 3, true>(in, out, cycles, 1u, reps, s);
        case 4: return launch<KIND, 4, true>(in, out, cycles, 1u, reps, s);
        default: return MI_ERR_SHAPE;
    }
}

}  // namespace
}  // namespace mi

extern "C" int mi_probe_issue_rate(int mode, int kind, int n, uint32_t waves_per_simd, uint32_t reps,
                                   const float* in, float* out, uint64_t* cycles, void* stream)
{
    using namespace mi;
    if (!in || !out || !cycles) return MI_ERR_NULL;
    if (reps == 0 || kind < 0 || kind >= kKinds) return MI_ERR_SHAPE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (mode == 0) {
        if (waves_per_simd != 1u) return MI_ERR_SHAPE;
        switch (kind) {
            case kVAdd: return launch_with_mfma<kVAdd>(n, in, out, cycles, reps, s);
            case kSAdd: return launch_with_mfma<kSAdd>(n, in, out, cycles, reps, s);
            case kDsRead: return launch_with_mfma<kDsRead>(n, in, out, cycles, reps, s);
            case kCvtPkBf16: return launch_with_mfma<kCvtPkBf16>(n, in, out, cycles, reps, s);
            default: return MI_ERR_SHAPE;
        }
    }
    if (mode == 1) {
        if (waves_per_simd < 1u || waves_per_simd > 4u) return MI_ERR_SHAPE;
        switch (kind) {
            case kVAdd: return launch<kVAdd, 8, false>(in, out, cycles, waves_per_simd, reps, s);
            case kCvtPkBf16: return launch<kCvtPkBf16, 8, false>(in, out, cycles, waves_per_simd, reps, s);
            case kCvtPkFp8: return launch<kCvtPkFp8, 8, false>(in, out, cycles, waves_per_simd, reps, s);
            case kMax3: return launch<kMax3, 8, false>(in, out, cycles, waves_per_simd, reps, s);
            case kLshl: return launch<kLshl, 8, false>(in, out, cycles, waves_per_simd, reps, s);
            default: return MI_ERR_SHAPE;
        }
    }
    return MI_ERR_SHAPE;
}
