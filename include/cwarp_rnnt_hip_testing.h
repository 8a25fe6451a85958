/*
 * cwarp_rnnt_hip_testing.h -- hooks of libcwarp_rnnt_hip.so that exist for its own tests.  Not part
 * of the drop-in surface (cwarp_rnnt_hip.h): nothing here has a counterpart in the reference, and a
 * caller of the loss never needs it.
 */
#ifndef CWARP_RNNT_HIP_TESTING_H
#define CWARP_RNNT_HIP_TESTING_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* The number of polls a wave of the lattice kernel spends waiting for the neighbouring strip's wave
 * before it gives up (CWR_FLAG_INTERNAL; the sequence's cost becomes NaN and its per-row gradients
 * zero; every wave still leaves the kernel normally).  polls <= 0 restores the default (about 4
 * million).  One atomic word for the process, read once per launch.  With polls = 1 a strip that
 * finds its feeder short of the 79 steps it must be ahead gives up at its first look; the two start
 * at the same barrier, so in practice that look always comes first, but it is a matter of timing. */
void cwr_debug_wait_limit(int polls);

/* cwr_forward (same arguments, outputs and results; see cwarp_rnnt_hip.h) with a HIP event recorded
 * on `stream` in front of and behind each of its four stages.  Unlike every entry point of the
 * drop-in surface this one creates events and WAITS for the stream: a measurement hook for the
 * benchmark's latency breakdown.  stage_us (host memory, 4 floats): microseconds from event to
 * event for the offsets scan, the gather pass, the lattice walk and the gradient fill; each figure
 * holds the kernel and the dependency gap in front of it. */
int cwr_debug_forward_stage_times(const void* x, int dtype, int64_t R, int64_t V, const int32_t* lx,
                                  const int32_t* ly, const int32_t* y, int64_t y_stride, int64_t y_len, int64_t N,
                                  int32_t blank, int mode, int64_t max_u, void* workspace, size_t workspace_bytes,
                                  int64_t* row_off, int64_t* lab_off, int32_t* status, int32_t* rowinfo, float* lse,
                                  float* grads, float* costs, void* stream, float* stage_us);

#ifdef __cplusplus
}
#endif
#endif /* CWARP_RNNT_HIP_TESTING_H */
