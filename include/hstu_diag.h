/*
 * Diagnostics of libhstu_hip.so: issue rates of the pieces of one 32 x 32 score block of the attention kernels on the
 * GPU the call runs on.  No counterpart in the reference; it exists so that the roofline argument for the attention
 * kernels (what the matrix cores and the vector unit sustain, alone and together, on real operand values) can be
 * re-measured with the library itself: `python bench.py --workload rates`.
 */
#ifndef HSTU_DIAG_H
#define HSTU_DIAG_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* what one iteration of a wave does */
enum {
    HSTU_RATE_SILU = 0,       /* SiLU of 16 values per lane (mul, exp, add, rcp, mul) and their packing to bf16 */
    HSTU_RATE_MFMA = 1,       /* 16 v_mfma_f32_32x32x16_bf16: a chain of 8 (S) and 8 on four accumulators (P V) */
    HSTU_RATE_BLOCK = 2,      /* the S chain, the SiLU of its result, P V with the packed result: one block without LDS */
    HSTU_RATE_PIPELINED = 3,  /* S of the next block and P V of the previous one interleaved with the SiLU of this one */
    HSTU_RATE_MFMA_FP8 = 4    /* 4 v_mfma_f32_32x32x64_f8f6f4 on four accumulators (the FLOPs of 16 of the 16-bit ones) */
};

/*
 * Launches 256 * waves_per_simd workgroups of 256 threads (waves_per_simd in 1..4 waves on every SIMD of a 256-CU GPU),
 * each wave running `iters` iterations of `mode` on operands it reads once from `operands` (1 MiB of bf16 / e4m3 values
 * chosen by the caller: zeros and random values give different rates).  `sink` takes one float per thread
 * (256 * 256 * waves_per_simd floats); `ticks` two uint64 per workgroup: its duration in core clocks (s_memtime) and in
 * ticks of the 100 MHz constant clock (s_memrealtime).  Asynchronous on `stream`; the caller times it with events.
 * Returns 0, or -1 for arguments out of range; MFMA and BLOCK fit their registers up to 3 waves per SIMD, PIPELINED up to 2,
 * and are rejected beyond.
 */
int hstu_hip_measure_block_rates(int mode, int waves_per_simd, int iters, const void* operands, float* sink, uint64_t* ticks, void* stream);

#ifdef __cplusplus
}
#endif
#endif
