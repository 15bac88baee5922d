/* Ceiling probes of libtkx_microbench.so: kernels that bench.py times on the box it runs on, next to the operator's
 * own figures. They have no counterpart in the reference (which reports no roofline); they exist so that the ceilings
 * a measured TFLOP/s is compared with are measured by the same run, on the same device, with committed code.
 * Status codes: 0 ok, 1 bad argument, 3 HIP runtime failure. All pointers are device pointers; `stream` is a
 * hipStream_t. The caller times the launches (HIP events on `stream`). */
#ifndef TKX_MICROBENCH_H_
#define TKX_MICROBENCH_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* One workgroup of 8 waves per CU, each wave issuing 8 independent v_mfma_f32_32x32x16_bf16 per iteration on
 * operands taken from `operands` (64 KB of bf16 values: their bits decide the clock the matrix cores settle at),
 * nothing else in the loop. `sink`: at least 4 bytes, never written in practice. */
int32_t tkxmb_mfma_bf16(const void* operands, int32_t iters, void* sink, void* stream);
/* FLOP of one such launch on the current device. */
int64_t tkxmb_mfma_bf16_flops(int32_t iters);

/* The same loop on v_mfma_scale_f32_32x32x64_f8f6f4 with e4m3fn operands and no block scales (`operands`: 64 KB
 * of fp8 bytes), and its FLOP per launch. */
int32_t tkxmb_mfma_fp8(const void* operands, int32_t iters, void* sink, void* stream);
int64_t tkxmb_mfma_fp8_flops(int32_t iters);

/* 2048 workgroups of 8 waves; each streams one region of `region_bytes` (a multiple of 8192) out of `regions`
 * (a multiple of 8) consecutive ones at `src` into LDS with direct-to-LDS loads, 8 KB outstanding per wave; `share`
 * (1..32) workgroups that run on one XCD at the same time read the same region. */
int32_t tkxmb_operand_stream(const void* src, int64_t region_bytes, int32_t regions, int32_t share, void* stream);
/* Bytes one such launch moves into LDS (share times the distinct bytes it reads). */
int64_t tkxmb_operand_stream_bytes(int64_t region_bytes);

#ifdef __cplusplus
}
#endif
#endif /* TKX_MICROBENCH_H_ */
