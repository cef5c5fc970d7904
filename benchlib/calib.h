/*
 * calib.h - C ABI of libagh_calib.so, the measurement-only companion of bench.py.  Not part of the product library
 * (libautograph_hip.so) and not declared in include/: these launches have no counterpart in the reference.
 * Every entry point takes the hipStream_t to launch on as `stream` (bench.py passes agh_stream(), so the HIP events
 * that time the product's kernels time these too), returns 0, a negative argument error (-1 invalid, -3 null,
 * -4 range) or a positive hipError_t, and leaves a message for calib_last_error_string().
 */
#ifndef AGH_CALIB_H
#define AGH_CALIB_H
#include <stddef.h>
#ifdef __cplusplus
extern "C" {
#endif

/* Calibration launches, for measurement only: what the part sustains at best on the two resources the kernels here are bound by.
 * calib_mfma_bf16: `blocks` workgroups of 4 waves, each wave `iters` times 16 independent
 * v_mfma_f32_32x32x16_bf16 (shape 0) or 64 independent v_mfma_f32_16x16x32_bf16 (shape 1, the form the bf16
 * GEMM uses) on register operands (zero_operands != 0: all zero; else bf16 patterns shaped like N(0, 0.02^2)
 * samples), 2 * 32*32*16 * 16 * (1 + shape) * iters * 4 * blocks flop, no memory traffic; `sink` is
 * 1 KiB of device memory that is practically never written.  calib_copy / calib_read: a plain
 * 16-byte nontemporal copy / read of `bytes` bytes with a grid of `blocks` workgroups of 256 threads
 * (grid-stride); also the pass of known size that profiler byte counters are scaled by.  calib_mix:
 * every 16 bytes of `dst` (`write_bytes` in all) receive the xor of the 16 bytes at the same offset of
 * `reads_per_write` consecutive source streams of `write_bytes` each (so `src` holds reads_per_write *
 * write_bytes bytes): the read:write mix of a gather kernel such as col2im in its simplest, fully coalesced form.
 * calib_mfma_dma: the MFMA-only loop on zero operands (`blocks` workgroups of 4 waves that each take a whole CU,
 * `iters` times 16 MFMAs per wave) with `loads_per_16_mfma` (0, 2, 4, 8 or 16) direct-to-LDS loads of 1 KiB spread
 * between the MFMAs of every wave; every workgroup cycles through a window of `window_bytes` of its own inside `src`
 * (`src_bytes` >= blocks * (window_bytes + 896)), so small windows are served by L2 and large ones from beyond it:
 * what the matrix pipes sustain while a CU pulls bytes through its L1 at the rate a GEMM tile needs. */
int calib_mfma_bf16(void *stream, void *sink, int zero_operands, int iters, int blocks, int shape);
int calib_copy(void *stream, const void *src, void *dst, size_t bytes, int blocks);
int calib_read(void *stream, const void *src, void *sink, size_t bytes, int blocks);
int calib_mix(void *stream, const void *src, void *dst, size_t write_bytes, int reads_per_write, int blocks);
int calib_mfma_dma(void *stream, const void *src, size_t src_bytes, void *sink, int loads_per_16_mfma, size_t window_bytes,
                   int iters, int blocks);
const char *calib_last_error_string(void);

#ifdef __cplusplus
}
#endif
#endif
