/*
 * llmmm_probe.h -- measurement probes of libllmmm.so: what this very GPU sustains, and where a launch of the tile
 * kernels spends its time.  Instrumentation only: nothing here replaces an interface of the reference, and no
 * product path calls it.  The drop-in surface is llmmm.h.
 */
#ifndef LLMMM_PROBE_H
#define LLMMM_PROBE_H

#include "llmmm.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ---- peak-rate probes ---------------------------------------------------------------------
 * What this very GPU sustains, next to the nominal peaks: the counterpart of the reference's register-only MMA
 * loop test_fp8_peak_work(stream) (examples/005.fp8.test.cu:19-71).
 * llmmm_probe_mfma enqueues `workgroups` x 8 wavefronts that issue v_mfma back to back from registers for `iters`
 * iterations; kind: LLMMM_DTYPE_F16 / LLMMM_DTYPE_BF16 (16x16x32) or LLMMM_PROBE_FP8 (e4m3, 16x16x128).  `operands`
 * = 32 KB of device memory whose bits become the operand fragments (the sustained rate depends on them: zeros run at
 * full clock, random data draws more power); `sink` = one float of device memory, never written in practice.
 * llmmm_probe_mfma_flops gives the FLOP of such a launch, so rate = flops / measured time.
 * llmmm_probe_hbm_read reads `bytes` (a multiple of 16) once with `workgroups` x 512 threads and writes nothing. */
#define LLMMM_PROBE_FP8 2
LLMMM_API int    llmmm_probe_mfma(int kind, const void* operands, float* sink, int workgroups, int iters, void* stream);
LLMMM_API double llmmm_probe_mfma_flops(int kind, int workgroups, int iters);
LLMMM_API int    llmmm_probe_hbm_read(const void* src, size_t bytes, float* sink, int workgroups, void* stream);

/* Where a launch of the 256 x 256 tile kernels spends its time.  These run the product kernels of llmmm_fp8_gemm(LLMMM_OUT_FP8Q)
 * / llmmm_fp16_gemm at M, N multiples of 256 (row-major operands), built with clock readings at five points of every wave:
 * 0 kernel entry, 1 first operands in LDS (end of the prologue), 2 end of the K loop, 3 last store issued, 4 stores acknowledged.
 * stamps: device memory of llmmm_probe_phases_bytes(M, N) bytes; afterwards, as 64-bit words, record (t * 8 + w) * 12 of
 * workgroup t and wave w (8 per workgroup) holds at [2 p] the constant 100 MHz clock at point p, at [2 p + 1] the shader's
 * cycle counter, at [10] the shader cycles the wave spent waiting in the K loop (loads landed + barrier of every stage) and at [11] the part
 * of those spent waiting for its own loads.
 * The reference measures its kernels from outside only (ncu.sh); no counterpart. */
LLMMM_API size_t llmmm_probe_phases_bytes(int M, int N);
LLMMM_API int    llmmm_probe_fp8_gemm_phases(const void* A, const float* As, const void* Bt, const float* Bs, void* C, float* Cs, int M, int N, int K,
                                             void* stamps, size_t stamps_bytes, void* stream);
LLMMM_API int    llmmm_probe_fp16_gemm_phases(int dtype, const void* A, const void* B, void* C, int M, int N, int K, void* stamps, size_t stamps_bytes,
                                              void* stream);

/* The decode-sized fused-quantisation GEMM in column strips (M <= 16 on the few-column-group projections) lets the eight
 * workgroups of a 128-column group exchange their row maxima through device memory and wait for each other, with a bound
 * on the wait (20 ms).  *count = waves that ever hit that bound since the library was loaded: 0 on a healthy device; a
 * non-zero value means results of such calls are not to be trusted.  Synchronises the device.  No counterpart in the
 * reference (its kernels never split K, README.md:22). */
LLMMM_API int llmmm_probe_strip_exchange_timeouts(unsigned* count);

#ifdef __cplusplus
}
#endif
#endif /* LLMMM_PROBE_H */
