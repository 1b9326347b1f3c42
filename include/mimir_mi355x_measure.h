/* Measurement aids of libmimir_mi355x.so: entry points that bench.py and the profiles use to time and
 * take apart the library's own launches. They are no part of the drop-in boundary (include/mimir_mi355x.h):
 * nothing in the reference corresponds to them and a host that only runs the product never calls them. */
#ifndef MIMIR_MI355X_MEASURE_H
#define MIMIR_MI355X_MEASURE_H

#include "mimir_mi355x.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Between timed_begin and timed_end, each launch of the fixed-point Q4_0 GEMV
 * kernel made by the calling thread (at most max_launches of them; not under
 * stream capture) is bracketed by its own pair of HIP events. timed_end waits
 * for the device and writes the milliseconds of each launch, in order. */
MI355X_API mi355x_status mi355x_timed_begin(int max_launches);
MI355X_API mi355x_status mi355x_timed_end(float* ms_each, int* n_launches);
/* While stamps is not NULL, every launch of the whole-chip Q4_0 decode kernel (one to four rows of x by a Q4_0
 * matrix; a build of it apart from the one that otherwise runs, so that the product's kernel carries no trace of
 * this) writes five int64 readings of the device's 100 MHz clock per workgroup to stamps[5 * workgroup ..]: at
 * entry, once x is staged in LDS, after its first row of W, after its last, and at exit. The caller provides
 * 40 bytes per workgroup of the largest launch (at most two workgroups per compute unit) and reads them back
 * after the launch; NULL stops it. Process-wide. */
MI355X_API mi355x_status mi355x_gemv_stamps(void* stamps);
/* Reads `bytes` bytes at p with 128-bit loads from `grid` workgroups of
 * `threads` threads and folds them into scratch (at least grid*threads/64
 * floats): the practical ceiling of a streaming read on this device. */
MI355X_API mi355x_status mi355x_stream_read(const void* p, size_t bytes, float* scratch, int grid, int threads, void* stream);

/* The kernel, with its template arguments, that the calling thread's latest Q4_0 product launched: of one row of x,
 * or the prompt-sized one of mi355x_qgemm_bf16 (for its panel route, the cut of Y into tiles); or, if it came later,
 * the kernel of its latest mi355x_attention call with keys (attn_prompt_kernel, attn_partial_kernel,
 * attn_decode_kernel). Which of the library's launch shapes the dispatch chose, as a NUL-terminated string of at most
 * n bytes. */
MI355X_API mi355x_status mi355x_last_kernel(char* buf, size_t n);

#ifdef __cplusplus
}
#endif
#endif /* MIMIR_MI355X_MEASURE_H */
