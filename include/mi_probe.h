/*
 * mi_probe.h -- C ABI of libmi_probe.so, the measurement aid that ships beside libmi_hadamard.so
 * (benchmark harness only; the product library neither links nor loads it).
 * Status codes are mi_status values (mi_hadamard.h).
 */
#ifndef MI_PROBE_H
#define MI_PROBE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/*
 * Matrix-core throughput probe: 256 workgroups (one per compute unit) of 256 * waves_per_simd
 * threads each run `steps` K steps of eight independent v_mfma_f32_16x16x32_bf16 (shape 16) or
 * four v_mfma_f32_32x32x16_bf16 (shape 32; the same 131072 flops per wavefront and step), with
 * lds_reads (0 or 4) 16-byte-per-lane LDS fragment reads per step beside them, on operands copied
 * from `operands`; cycles[w] receives the shader clock cycles workgroup w spent in the loop.  Used
 * to measure the clock and the matrix-core rate the chip sustains for a given operand pattern.
 * No counterpart in the reference.
 *   operands : device, 16-byte aligned, at least 64 KiB (any bit pattern; bf16 operands)
 *   cycles   : device, 512 x uint64: [0, 256) cycles per workgroup, [256, 512) a checksum of each
 *              workgroup's accumulators (an output whose only purpose is to keep the arithmetic alive)
 *   waves_per_simd in {1, 2, 4};  steps a positive multiple of 4.
 */
int mi_probe_mfma_rate(int shape, int lds_reads, uint32_t waves_per_simd, uint32_t steps,
                       const void* operands, uint64_t* cycles, void* stream);

/*
 * Instruction-issue probe, one compute unit (a single workgroup).  No counterpart in the reference.
 *   mode 0: one wavefront per SIMD runs reps x 8 groups of [one v_mfma_f32_16x16x32_bf16 + n (0..4)
 *           independent instructions of `kind`]; cycles[w] = shader clock cycles of wavefront w, so
 *           cycles / (8 reps) is the cost of a group.  kind: 0 v_add_f32, 1 v_cvt_pk_bf16_f32,
 *           2 s_add_u32, 3 ds_read_b128.  waves_per_simd must be 1.
 *   mode 1: no MFMA: waves_per_simd (1..4) wavefronts per SIMD each run reps x 64 independent
 *           instructions of `kind` (0 v_add_f32, 1 v_cvt_pk_bf16_f32, 4 v_cvt_pk_fp8_f32, 5 v_max3_f32,
 *           6 v_lshlrev_b32); max(cycles) / (64 reps waves_per_simd) = cycles per instruction and SIMD.
 *   in     : device, 256 x 8 fp32 (any finite values)      out : device, 1024 fp32 (keeps the work alive)
 *   cycles : device, 16 x uint64
 */
int mi_probe_issue_rate(int mode, int kind, int n, uint32_t waves_per_simd, uint32_t reps,
                        const float* in, float* out, uint64_t* cycles, void* stream);

/*
 * Streaming-rate probe: 256 workgroups of four wavefronts (one per compute unit); every wavefront
 * reads bytes_per_wave contiguous bytes, 1 KB per instruction, `depth` (4, 8 or 16) instructions
 * requested before the older half is waited for; mode 0: global_load_lds_dwordx4 (global -> LDS
 * directly), mode 1: global_load_dwordx4 into registers.  `share` (a divisor of 256) consecutive
 * workgroup ids read the same region of 4 x bytes_per_wave bytes at src + (id / share) x that;
 * consecutive ids run on different XCDs.  The caller times a series of launches; rate per compute
 * unit = 4 x bytes_per_wave / time.  No counterpart in the reference.
 *   src : device, 16-byte aligned, (256 / share) x 4 x bytes_per_wave bytes (any contents)
 *   out : device, 65536 x uint32 (keeps the loads alive)
 *   bytes_per_wave : a positive multiple of 16 KiB
 */
int mi_probe_stream_rate(int mode, uint32_t depth, uint32_t share, uint64_t bytes_per_wave,
                         const void* src, uint32_t* out, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MI_PROBE_H */
