/*
 * flashlight_amd_probe.h -- C ABI of libflashlight_amd_probe.so, a bench-only library.
 *
 * Micro-benchmarks that put the forward's measured rate in context (what the matrix pipe alone sustains on given
 * data; what the forward's key-tile step costs as an instruction mix).  Not part of the drop-in boundary: the
 * product library libflashlight_amd.so exports none of this, and only bench.py loads it.  Nothing here has a
 * counterpart in the reference.
 */
#ifndef FLASHLIGHT_AMD_PROBE_H
#define FLASHLIGHT_AMD_PROBE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* error codes (negative), the same values as in flashlight_amd.h */
#define FLP_ERR_UNSUPPORTED (-4)
#define FLP_ERR_ARG (-5)
#define FLP_ERR_ALIGN (-7)

/* Measurement aid with no counterpart in the reference: launches a kernel that does nothing but issue
 * v_mfma_f32_32x32x16_bf16 (the instruction both products of the forward are built from) on operand fragments read
 * once from `operands`, so that the matrix-pipe rate this part sustains on given data can be put next to the
 * forward's.  One workgroup of 512 threads per compute unit, two waves per SIMD; every lane reads 12 16-byte
 * fragments (8 A, 4 B) at 16-byte index (thread * 12 + j) % n_fragments and issues iters * 32 MFMAs; one float per
 * thread is written to `sink` (n_workgroups * 512 floats).  Work = n_workgroups * 8 * iters * 32 * 32768 FLOP.
 * Returns 0, or a negative code for bad arguments. */
int fl_probe_mfma_rate(const void* operands, int64_t n_fragments, int iters, int n_workgroups, float* sink, void* stream);

/* Measurement aid with no counterpart in the reference: the forward's key-tile step reduced to its instruction mix and
 * data dependences, on zero operands held in registers (head_dim 64 or 128; 2 * iters blocks of 32 keys x 32 queries
 * per wave, workgroups of 4 waves).  level 0: the block's MFMAs alone; 1: MFMAs and the softmax's vector work with no
 * dependence between them; 2: the step as the forward has it (scores chained on one accumulator, weights from the
 * scores, P.V from the weights); 3: the same with the K and V fragments read from LDS; 4: level 2 in a three-stage
 * order (P.V on the previous block's weights, so that both groups of MFMAs run under this block's vector work).  The time per block against the
 * MFMAs' own time says what the instruction mix, its dependences and the operand reads cost before any global memory,
 * transfer or barrier enters.  One float per thread goes to `sink` (n_workgroups * 256 floats). */
int fl_probe_step(int head_dim, int level, int iters, int n_workgroups, float* sink, void* stream);

/* Measurement aid: how much vector work fits under matrix instructions.  Every wave runs `iters` times a loop of 8 units of
 * matrix work on independent accumulators (mfma_rows = 32: one v_mfma_f32_32x32x16_bf16 per unit; 16: two
 * v_mfma_f32_16x16x32_bf16), each unit followed by `valu_per_mfma` (0, 1, 2, 3, 4, 6 or 8) vector instructions of one kind
 * on other registers (valu_kind 0: v_fma_f32, 1: v_exp_f32, 2: v_cvt_pk_bf16_f32, 3: v_dot2c_f32_bf16, 4: v_add_f32), in
 * fixed registers and fixed order, zero operands.  Workgroups of 256 * waves_per_simd threads (1 or 2 waves per SIMD
 * when n_workgroups is the number of compute units).  `wave_cycles` (n_workgroups * 4 * waves_per_simd int64) receives
 * every wave's shader-clock cycles for the whole loop; `sink` one float per thread.  Cycles per unit of matrix work per
 * SIMD = slowest wave's cycles / (8 * iters) / waves_per_simd (the waves of a SIMD share its matrix pipe). */
int fl_probe_coissue(int mfma_rows, int valu_kind, int valu_per_mfma, int waves_per_simd, int iters, int n_workgroups,
                     float* sink, long long* wave_cycles, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FLASHLIGHT_AMD_PROBE_H */
