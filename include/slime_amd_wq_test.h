/*
 * slime_amd_wq_test.h - C ABI of libslime_amd_wq_test.so: instruments of the test-suite and the benchmark for the
 * kernels of libslime_amd_wq.so (slime_amd_wq.h).  Nothing here is part of the product interface and no caller of the
 * weight-conversion path needs this library: exhaustive on-device self-checks of the element functions the production
 * kernels use (compiled from the same header-only definitions), and compute-free kernels with known traffic that
 * hardware counters and achieved bandwidths are scaled against.
 *
 * Conventions (pointers, streams, return codes) are those of slime_amd_wq.h.
 */
#ifndef SLIME_AMD_WQ_TEST_H
#define SLIME_AMD_WQ_TEST_H

#include <stdint.h>

#include "slime_amd_wq.h"

#ifdef __cplusplus
extern "C" {
#endif

/* WQ_ABI_VERSION of the product header this library was compiled against. */
int wq_test_abi_version(void);

/* wq_selftest_fp8_elem: for every bf16 amax a in [amax_lo, amax_hi) (bit patterns, finite) and every
 * bf16 x with |x| <= max(a, floor), compares the production element function (reciprocal + two FMA
 * refinement + hardware e4m3 conversion) with plain IEEE division + software RNE conversion.
 * Writes {mismatch count, first mismatching (a<<16|x)} to out[0..1] (DEVICE uint64[2], zeroed here).
 * wq_selftest_int4_elem: same for the INT4 element function q = rintf(x/scale).
 * wq_selftest_cvt_fp8: compares the hardware fp32->e4m3 conversion with the software one for the
 * fp32 bit patterns [lo, hi) whose magnitude is <= 464 or NaN. */
int wq_selftest_fp8_elem(uint32_t amax_lo, uint32_t amax_hi, int mode, uint64_t *out, void *stream);
int wq_selftest_int4_elem(uint32_t amax_lo, uint32_t amax_hi, uint64_t *out, void *stream);
int wq_selftest_cvt_fp8(uint64_t lo, uint64_t hi, uint64_t *out, void *stream);
/* wq_selftest_cvt_bf16: hardware fp32->bf16 conversion vs software RNE for the non-NaN fp32 bit
 * patterns in [lo, hi).  wq_selftest_decode_fp8: hardware e4m3fn->fp32 vs the format definition for all
 * 256 codes.  Same out[] convention. */
int wq_selftest_cvt_bf16(uint64_t lo, uint64_t hi, uint64_t *out, void *stream);
int wq_selftest_decode_fp8(uint64_t *out, void *stream);

/* Plain 16-byte-per-lane copy of n_bytes (multiple of 16, 16-byte aligned): the known-traffic kernel
 * that hardware counters are scaled against. */
int wq_copy_bytes(const void *src, void *dst, int64_t n_bytes, void *stream);

/* A compute-free stream with `reads_per_write` (2 or 4) bytes read per byte written - the block-FP8 quantiser's and the
 * INT4 packer's read:write mix: dst[16 KiB piece i] = xor of src[pieces reads_per_write * i ...].  n_out_bytes a multiple
 * of 16384; src holds reads_per_write * n_out_bytes.  The benchmark runs it next to the quantisers to show what the
 * memory system gives that mix on the box at hand. */
int wq_stream_fold_bytes(const void *src, void *dst, int64_t n_out_bytes, int reads_per_write, void *stream);

/* The mirror image for the dequantisers' mixes: `writes_per_read` (2 or 4) bytes written per byte read - FP8 -> bf16 and
 * INT4 -> bf16.  Output piece w (of writes_per_read) of every 4 KiB input piece is the input with w added to each dword.
 * n_in_bytes a multiple of 16384; dst holds writes_per_read * n_in_bytes. */
int wq_stream_expand_bytes(const void *src, void *dst, int64_t n_in_bytes, int writes_per_read, void *stream);

/* An empty kernel over `workgroups` workgroups of `threads` lanes: what a launch costs on the box at hand before any
 * byte moves (dispatch, wave start-up, completion), the floor under every small launch. */
int wq_empty_launch(int64_t workgroups, int threads, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* SLIME_AMD_WQ_TEST_H */
