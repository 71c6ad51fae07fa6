/*
 * libdfa3d_measure - yardsticks for the machine the DFA3D kernels run on.  NOT part of the operator library:
 * bench.py loads it to put the kernels' timings next to what the hardware does for the bare access patterns
 * they are made of (a streaming copy, random row gathers, random scalar gathers, LDS atomics) and to see
 * which XCD each workgroup of a launch lands on.
 *
 * Same conventions as libdfa3d_hip: device pointers into caller-owned memory, launch on `stream`, no
 * synchronisation, 0 on success / negative for a rejected argument / positive hipError_t.
 */
#ifndef DFA3D_MEASURE_H
#define DFA3D_MEASURE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* dst[i] = src[i], 16 bytes per lane: `bytes` read and `bytes` written.  bytes % 16 == 0, 16-byte aligned. */
int dfa3d_measure_stream_copy(void *dst, const void *src, size_t bytes, void *stream);

/* out[block] = id of the XCD (accelerator die) the workgroup `block` ran on, for a launch of `blocks`
 * workgroups of `threads` threads that each spin for about `spin_clocks` shader clocks (so that the whole
 * grid is resident at once, as a real kernel's is). */
int dfa3d_measure_xcd_map(int32_t *out, int blocks, int threads, int spin_clocks, void *stream);

/* Random row gathers: every group of row_bytes/16 lanes reads whole rows of `row_bytes` (64, 128 or 256) at
 * pseudo-random row indices below `rows` (a power of two), `in_flight` (1, 2, 4 or 8) independent loads at a
 * time, `iters` rounds.  blocks x 256 threads.  Rows read in total: blocks * 256 / (row_bytes/16) * iters *
 * in_flight.  `sink` (at least 16 bytes) is only written if a sum of zeros is non-zero. */
int dfa3d_measure_row_gather(const void *src, size_t rows, int row_bytes, int in_flight, int blocks, int iters,
                             void *sink, void *stream);

/* Random 8-byte gathers, one per lane (64 different cache lines per wavefront instruction), from the first
 * `bytes` (a power of two) of src; `in_flight` (1, 2, 4 or 8) independent loads at a time.  Loads in total:
 * blocks * 256 * iters * in_flight. */
int dfa3d_measure_pair_gather(const void *src, size_t bytes, int in_flight, int blocks, int iters, void *sink,
                              void *stream);

/* LDS atomics: blocks x 256 threads, `iters` atomics each on an 8192-word array.
 * mode 0 float add, one bank per lane; 1 float add, random addresses; 2 float add, one address;
 * 3 integer add returning, random; 4 integer add, random; 5 integer exchange, random. */
int dfa3d_measure_lds_atomics(int mode, int blocks, int iters, void *sink, void *stream);

#ifdef __cplusplus
}
#endif
#endif
