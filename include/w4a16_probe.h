/*
 * Measurement aids of libw4a16.so.  Nothing here belongs to the GEMM path or has a counterpart in
 * the reference: these entry points exist so that a benchmark can time what the machine gives a
 * kernel that does nothing but read, or nothing but synchronise, launched the way the GEMM
 * kernels are.  Conventions (pointers, streams, return codes) are those of w4a16.h.
 */
#ifndef W4A16_PROBE_H_
#define W4A16_PROBE_H_

#include "w4a16.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Measurement aid (no counterpart in the reference): a plain streaming read of `bytes` at `src`,
 * launched like the decode kernels.  Its time on a buffer of a matrix's size is the ceiling that a
 * launch, the first trip to HBM and the streaming itself set for a GEMM that reads the matrix once. */
int w4a16_probe_read(w4a16_handle* h, const void* src, size_t bytes, void* stream);

/* The same read with the load pipeline of the GEMM kernels: every lane keeps `in_flight` (2, 4, 8 or 16)
 * 16-byte loads in flight, issued in place and waited for by count, `wg_per_cu` (1, 2 or 4) workgroups of
 * eight waves per CU; hint 0 = plain loads, 1 = non-temporal, 2 = system scope.  `bytes` is rounded down
 * to a multiple of 1024.  For sweeping what the memory system gives a kernel that only reads. */
int w4a16_probe_stream(w4a16_handle* h, const void* src, size_t bytes, int wg_per_cu, int in_flight, int hint,
                       void* stream);

/* Nothing but matrix instructions: one workgroup of `waves_per_cu` (4, 8 or 16) waves per CU, every wave
 * `iters` rounds of four independent v_mfma_f32_16x16x32_f16 (16384 flop each) on registers.  Its rate,
 * cus x waves_per_cu x iters x 65536 flop over the time between two events, is what the matrix pipes reach at
 * the clock the chip settles at under them. */
int w4a16_probe_mfma(w4a16_handle* h, int waves_per_cu, int iters, void* stream);

/* The engine clock inside the kernels.  Between w4a16_probe_clock_begin and w4a16_probe_clock_end one
 * thread of every decode strip kernel launched by w4a16_gemm, and of every w4a16_probe_stream and
 * w4a16_probe_mfma launch, through this handle reads the core-clock counter and the constant-rate counter when
 * it starts and when it ends and adds the differences up (launches captured into a graph in between keep
 * recording on every replay).  `end` synchronises the stream and returns the sums: cycles / ticks x
 * ticks_per_second is the clock those kernels ran at, ticks / launches their duration.  Ordinary launches
 * carry a null pointer and record nothing.  `begin` clears the counters on `stream` with a memset, so it is called
 * outside stream capture; a handle records for one begin / end pair at a time. */
int w4a16_probe_clock_begin(w4a16_handle* h, void* stream);
int w4a16_probe_clock_end(w4a16_handle* h, unsigned long long* cycles, unsigned long long* ticks,
                          unsigned long long* launches, long long* ticks_per_second, void* stream);

/* Measurement aid (no counterpart in the reference): one persistent launch of one workgroup per CU that
 * crosses `iters` device-wide barriers of w4a16_gemm_sequence and does nothing else; time it with
 * events and divide.  tree = 1: the two-level counter tree that the sequence kernel uses; tree = 0: every
 * workgroup arrives on one counter. */
int w4a16_probe_barrier(w4a16_handle* h, int iters, int tree, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* W4A16_PROBE_H_ */
