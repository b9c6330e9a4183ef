/*
 * hw_rates.h -- C ABI of libsage_hwrates.so: hardware-rate micro-benchmarks of the MI355X units the attention
 * kernel is priced against.  A measurement aid of the benchmark tools, not part of the drop-in library
 * (libsage_mi355x.so exports none of this); no counterpart in the reference.
 *
 * kind: 0 v_mfma_i32_32x32x32_i8 from registers, 1 v_mfma_f32_32x32x64_f8f6f4 (fp8) from registers, 2 LDS reads
 * (ds_read_b128), 3 / 4 the two MFMAs with every operand fragment read from LDS as the attention kernel does,
 * 5 v_fma_f32, 6 v_exp_f32, 7 v_cvt_pk_fp8_f32, 8 the softmax mix (per score one fma, one exp2, half a packed fp8
 * conversion).  sage_microbench launches `grid` workgroups (one per compute unit is the intended use) of
 * 4 * waves_per_simd wavefronts (1, 2 or 4 per SIMD), `iters` iterations each, on `stream` (a hipStream_t); the
 * caller times the launch.  sage_microbench_units gives the work of one wavefront per iteration: operations (a
 * multiply-add counts 2), bytes, or instructions.  `sink` (device memory) takes grid * 1024 ints.
 *
 * sage_coexec: how much the matrix pipe and the vector ALU of a SIMD slow each other down.  Workgroups of eight
 * wavefronts (two per SIMD): wavefronts 0-3 issue MFMAs (mfma_kind 0 INT8 32x32x32, 1 FP8 32x32x64; 16 per iteration),
 * wavefronts 4-7 vector instructions (valu_kind 0 v_fma_f32, 1 v_cvt_pk_u8_f32, 2 v_max3_i32, 3 a mix of the FP8
 * softmax with one conversion per code: 64 + 64 + 32 per iteration, 4 the mix the kernels run: 64 v_fma_f32 +
 * 32 v_cvt_pknorm_u16_f32 + 16 v_perm_b32 + 32 v_max3_i32).  mode 1 runs the MFMA half alone, 2 the vector half alone, 3 both.
 *
 * sage_period: the steady-state 128-key tile period of the FP8 P.V attention kernel at head_dim 128 as an instruction
 * mix without the attention around it: eight wavefronts in two groups half a period apart, per wavefront and period 16
 * INT8 MFMAs + 8 FP8 MFMAs + 2 row-sum MFMAs fed by 32 ds_read_b128, the 160-odd vector instructions of a tile's row
 * maximum and probability codes, and four 1 KB global->LDS requests; one LDS-only barrier per period.  `parts` switches
 * the pieces on (1 MFMAs, 2 fragments from LDS, 4 vector half, 8 requests); `random_operands` chooses the operand bits
 * (0 a regular low-entropy pattern, 1 hashed bytes: the same instructions, but the multipliers, the register file and
 * LDS see bits that toggle, and the clock the part sustains differs).  What the schedule costs on the hardware before
 * masks, rescales, prologue, epilogue and imbalance.
 *
 * sage_period64: the same work per compute unit and period (256 query rows x 128 keys, head_dim 128) as an instruction mix
 * for a design the attention kernel does NOT have: one wavefront per SIMD, 64 query rows per wavefront, so that every K / V
 * fragment read from LDS feeds two MFMAs (half the fragment reads), matrix and vector work of neighbouring 64-key steps
 * interleaved inside one instruction stream, output accumulators in the accumulation registers.  Whether that design
 * would pay, measured before anyone writes the kernel.
 */
#ifndef SAGE_HW_RATES_H
#define SAGE_HW_RATES_H
#include <stddef.h>
#ifdef __cplusplus
extern "C" {
#endif
#define HWR_OK 0
#define HWR_EINVAL (-1)
#define HWR_ELAUNCH (-4)
#define HWR_ESIZE (-5)
double sage_microbench_units(int kind);
int sage_microbench(int kind, int grid, int waves_per_simd, int iters, void* sink, size_t sink_bytes, void* stream);
int sage_coexec(int mfma_kind, int valu_kind, int mode, int grid, int iters, void* sink, size_t sink_bytes, void* stream);
int sage_period64(int random_operands, int grid, int periods, void* sink, size_t sink_bytes, const void* src, size_t src_bytes, void* stream);
int sage_period(int parts, int random_operands, int grid, int periods, void* sink, size_t sink_bytes, const void* src, size_t src_bytes, void* stream);
#ifdef __cplusplus
}
#endif
#endif
