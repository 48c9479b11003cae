// Shared device/host helpers for the gfx950 Hadamard kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "mi_hadamard.h"

namespace mi {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;

// 16-bit storage types the matrix cores take directly.  `E` is the element type, `V8`/`V4` the
// 8- and 4-wide MFMA operand vectors.
struct BF16 {
    static constexpr int kCode = MI_BF16;
    using E = __bf16;
    using V8 = bf16x8;
    using V4 = bf16x4;
    static __device__ __forceinline__ f32x4 mfma32(V8 a, V8 b, f32x4 c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ f32x4 mfma16(V4 a, V4 b, f32x4 c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4, a),
                                                         __builtin_bit_cast(s16x4, b), c, 0, 0, 0);
    }
};

struct F16 {
    static constexpr int kCode = MI_F16;
    using E = _Float16;
    using V8 = f16x8;
    using V4 = f16x4;
    static __device__ __forceinline__ f32x4 mfma32(V8 a, V8 b, f32x4 c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ f32x4 mfma16(V4 a, V4 b, f32x4 c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x16f16(a, b, c, 0, 0, 0);
    }
};

// Entry of a Hadamard matrix that acts only on the index bits in `mask` and is the identity on
// the others:  0 if a and b differ outside the mask, else c * (-1)^popcount(a & b & mask).
// Sign rule = Sylvester ordering, H[i][j] = (-1)^popcount(i & j).
__device__ __forceinline__ float masked_hadamard_entry(uint32_t a, uint32_t b, uint32_t mask,
                                                       float c)
{
    if ((a ^ b) & ~mask) return 0.0f;
    return (__popc(a & b & mask) & 1) ? -c : c;
}

inline bool is_pow2(uint32_t x) { return x && !(x & (x - 1)); }
inline uint32_t ilog2(uint32_t x) { return 31u - (uint32_t)__builtin_clz(x); }
inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

inline int launch_status()
{
    return hipGetLastError() == hipSuccess ? MI_OK : MI_ERR_LAUNCH;
}

}  // namespace mi
