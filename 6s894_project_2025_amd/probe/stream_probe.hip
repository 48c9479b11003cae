// Streaming-rate probe (mi_probe_stream_rate), gfx950.  Built into libmi_probe.so.
//
// The GEMM kernels stream one operand through every compute unit (W of the fused kernels: 1 MB per
// compute unit and launch at the headline shape), and how fast a compute unit can take data in
// from the L2 and from beyond it bounds their main loops as much as the matrix cores do.  This
// probe measures it: 256 workgroups of four wavefronts (one per compute unit), each wavefront
// reading `bytes_per_wave` contiguous bytes in pieces of 1 KB per instruction, `depth` pieces
// requested before the oldest half of them is waited for,
//   mode 0: global_load_lds_dwordx4 (global -> LDS directly, what the GEMM kernels use),
//   mode 1: global_load_dwordx4 into registers.
// `share` consecutive workgroup ids read the same 4 x bytes_per_wave region: consecutive ids run
// on different XCDs, so share = 1 and share = 8 read every byte from beyond the L2 (once per
// XCD), while share = 32 puts four readers of a region on each XCD (three of four requests can hit
// its L2).  The time of the launch is taken by the caller (events around a series of launches).
// No counterpart in the reference.
#include "common.hpp"
#include "mi_probe.h"

namespace mi {
namespace {

template <int MODE, int DEPTH>
__global__ void __launch_bounds__(256)
stream_probe_kernel(const unsigned char* __restrict__ src, uint32_t* __restrict__ out, uint64_t region_bytes,
                    uint32_t rounds, uint32_t share)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const uint32_t lane = threadIdx.x & 63u, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const unsigned char* base = src + (uint64_t)(blockIdx.x / share) * region_bytes +
                                (uint64_t)wave * rounds * (uint64_t)(DEPTH * 1024);
    u32x4 acc = {0u, 0u, 0u, 0u};
    if (MODE == 0) {
        const uint32_t slot = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)lds) + wave * (uint32_t)(DEPTH * 1024);
        for (uint32_t it = 0; it < rounds; ++it) {
            const unsigned char* p = base + (uint64_t)it * (uint64_t)(DEPTH * 1024);
#pragma unroll
            for (int j = 0; j < DEPTH; ++j)
                asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                             :: "v"(lane * 16u + 1024u * j), "s"(p), "s"(slot + 1024u * j) : "memory");
            asm volatile("s_waitcnt vmcnt(%0)" :: "n"(DEPTH / 2) : "memory");
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        acc = *reinterpret_cast<const u32x4*>(lds + wave * (uint32_t)(DEPTH * 1024) + lane * 16u);
    } else {
        for (uint32_t it = 0; it < rounds; ++it) {
            const unsigned char* p = base + (uint64_t)it * (uint64_t)(DEPTH * 1024);
            u32x4 v[DEPTH];
#pragma unroll
            for (int j = 0; j < DEPTH; ++j) v[j] = *reinterpret_cast<const u32x4*>(p + lane * 16u + 1024u * j);
#pragma unroll
            for (int j = 0; j < DEPTH; ++j) acc ^= v[j];
        }
    }
    out[blockIdx.x * 256u + threadIdx.x] = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
}

template <int MODE, int DEPTH>
int launch(const unsigned char* src, uint32_t* out, uint64_t bytes_per_wave, uint32_t share, hipStream_t s)
{
    const uint32_t rounds = (uint32_t)(bytes_per_wave / (uint64_t)(DEPTH * 1024));
    hipLaunchKernelGGL((stream_probe_kernel<MODE, DEPTH>), dim3(256), dim3(256), MODE == 0 ? 4 * DEPTH * 1024 : 0,
                       s, src, out, 4u * bytes_per_wave, rounds, share);
    return launch_status();
}

template <int MODE>
int launch_depth(uint32_t depth, const unsigned char* src, uint32_t* out, uint64_t bytes_per_wave, uint32_t share,
                 hipStream_t s)
{
    switch (depth) {
        case 4: return launch<MODE, 4>(src, out, bytes_per_wave, share, s);
        case 8: return launch<MODE, 8>(src, out, bytes_per_wave, share, s);
        case 16: return launch<MODE, 16>(src, out, bytes_per_wave, share, s);
        default: return MI_ERR_SIZE;
    }
}

}  // namespace
}  // namespace mi

extern "C" int mi_probe_stream_rate(int mode, uint32_t depth, uint32_t share, uint64_t bytes_per_wave,
                                    const void* src, uint32_t* out, void* stream)
{
    using namespace mi;
    if (mode != 0 && mode != 1) return MI_ERR_SIZE;
    if (share == 0 || 256u % share != 0) return MI_ERR_SIZE;
    if (bytes_per_wave == 0 || bytes_per_wave % (16u * 1024u) != 0 || bytes_per_wave > (1ull << 30)) return MI_ERR_SIZE;
    if (!src || !out) return MI_ERR_NULL;
    if (!aligned16(src)) return MI_ERR_ALIGN;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const unsigned char* p = static_cast<const unsigned char*>(src);
    return mode == 0 ? launch_depth<0>(depth, p, out, bytes_per_wave, share, s)
                     : launch_depth<1>(depth, p, out, bytes_per_wave, share, s);
}
