/* Entry points of libsga_hip_bench.so, the benchmark-only companion of
 * libsga_hip.so.  They stand behind no interface of wenqingqian/SGA and are
 * NOT part of the drop-in boundary (include/sga_hip.h; libsga_hip.so exports
 * none of them): bench.py uses them to time the dominant kernels live with
 * HIP events on their launch stream and to calibrate the HBM traffic
 * counters.  libsga_hip.so holds two weak references (sga_bench_prof_begin /
 * sga_bench_prof_end) that bind to this library when it was loaded first,
 * into the global symbol scope (dlopen with RTLD_GLOBAL); without it they are
 * null and a timed launch costs the product path one pointer test.
 * Process-wide state behind a mutex.
 */
#ifndef SGA_HIP_BENCH_H_
#define SGA_HIP_BENCH_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* tags of the timed kernels */
#define SGA_PROF_TAG_FUSED_FINAL 0   /* k_fused_final (the fused step's final sweep)   */
#define SGA_PROF_TAG_SELECT_SWEEP 1  /* k_bracket_sweep (the select's one data sweep)  */
#define SGA_PROF_TAG_REPLAY_PASS3 2  /* k_replay_pass3                                  */
#define SGA_PROF_TAG_REPLAY_PASS1 3  /* the k_replay_pass1 launches of one step         */

/* enable(1) waits for event pairs still in flight, resets the table and arms
 * up to 4096 timed launches; enable(0) disarms.  read() waits for the recorded
 * events of one tag and returns their summed duration in ms and their number. */
int sga_prof_enable(int on);
/* the observer libsga_hip.so calls around a timed launch (not for callers) */
void* sga_bench_prof_begin(int tag, void* stream);
void sga_bench_prof_end(void* pair, void* stream);
/* text of the last error of this library on the calling thread */
const char* sga_bench_last_error(void);
int sga_prof_read(int tag, double* total_ms, int* launches);

/* dst[0..n) = src[0..n), fp32, n % 4 == 0: plain copy of known size used to
 * scale the HBM traffic counters. */
int sga_calib_copy(float* dst, const float* src, int64_t n, void* stream);

/* Math-free kernel with the fused final sweep's stream structure (reads bf16
 * g and fp32 r/p/m/v, rewrites r/p/m/v: 34 B per element).  Overwrites r/p/m/v
 * with meaningless values: use scratch buffers. */
int sga_calib_streams(const void* g_bf16, float* r, float* p, float* m, float* v,
                      int64_t n, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* SGA_HIP_BENCH_H_ */
