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
#ifdef __cplusplus
}
#endif
#endif
