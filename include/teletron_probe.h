/* teletron_probe.h -- C ABI of libteletron_probe.so: MEASUREMENT ONLY.
 *
 * Plain streaming kernels with the access shapes of the normalization kernels and no arithmetic,
 * used by the benchmark and the profile summaries to show what the memory system gives each
 * read/write mix.  Nothing here has a counterpart in the reference (it has no instrumentation), and
 * nothing in libteletron_norm.so or the extension modules links or loads this library: a caller
 * that binds the operators never sees it.
 *
 * All pointers are device pointers, 16-byte aligned.  Calls are asynchronous on `stream`
 * (a hipStream_t passed as void*).  Status codes are those of teletron_norm.h (0 = ok,
 * 1 = invalid argument, 2 = unsupported combination, 3 = misaligned pointer, 5 = HIP error).
 */
#ifndef TELETRON_PROBE_H_
#define TELETRON_PROBE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TT_PROBE_ABI_VERSION 1

int tt_probe_abi_version(void);

/* Thread-local detail of the last non-zero status returned on this thread. */
const char *tt_probe_last_error(void);

/* Plain copy of `bytes` (a multiple of 16) from src to dst: one-shot grid, every wavefront copies one
 * contiguous 6 KiB run (six 16-byte accesses per lane, the shape of a 3072-column two-byte row) and
 * exits.  The achievable-bandwidth yardstick the benchmark prints next to each result, and the kernel
 * of known traffic the FETCH_SIZE / WRITE_SIZE counters are calibrated on. */
int tt_probe_stream_copy(void *dst, const void *src, size_t bytes, void *stream);

/* A plain stream of `reads` tensors read (0..4) and `writes` tensors written (0..2), `bytes` each, where
 * every wavefront moves one contiguous run of accesses_per_lane KiB per tensor (1, 2 or 6 accesses of
 * 16 bytes per lane) and writes, to written tensor j, the dword-wise sum of the tensors read plus j
 * (with no tensor read: the run index in dword 0 of every 16 bytes, then 1, 2, 3; plus j).
 * Tensors read: a, b, a + bytes, b + bytes in this order; written: dst, dst + bytes.  a_bytes, b_bytes and
 * dst_bytes are the lengths of the three allocations; a call that would step outside one of them
 * returns 1 (invalid argument) before anything is launched.
 * Built mixes: up to 2 reads with up to 1 write in every shape; 3+1, 2+2 and 4+2 (the mixes of the
 * residual and gated kernels) with 1 and 6 accesses per lane; any other combination returns 2.
 * persistent_blocks = 0 launches one wavefront per run (one-shot grid), otherwise that many workgroups of
 * four wavefronts stride over the runs.  write_through != 0 uses the write-through store of the
 * backward kernels instead of the plain streaming store. */
int tt_probe_stream(void *dst, size_t dst_bytes, const void *a, size_t a_bytes, const void *b, size_t b_bytes,
                    size_t bytes, int reads, int writes, int accesses_per_lane, int persistent_blocks,
                    int write_through, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* TELETRON_PROBE_H_ */
