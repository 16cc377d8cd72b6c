/*
 * n2d2hip_probe.h - in-kernel phase probes of the convolution kernels.  No counterpart in the reference.
 *
 * These two entry points exist only in a library built with -DN2D2HIP_PROFILE (python -m n2d2_amd.build --probe
 * builds it as n2d2_amd/lib/libn2d2hip_probe.so); the product library does not export them and its kernels carry no
 * probes.  In a probe build every work-group of conv_pipe_kernel, conv_patch3x3_kernel and bottleneck_kernel writes one
 * record of N2D2HIP_PROBE_RECORD 64-bit counters when it ends:
 *   [0] shader clock at the work-group's first instruction     [1] ... when its first operand load is issued
 *   [2] ... when its first ring stage has landed (first matrix instruction)   [3] ... at its end
 *   [4] shader clocks spent in epilogues    [5] / [6] the constant 100 MHz counter at its start / end
 *   [7] units of work it did (ring steps or tiles)   [8..13] bottleneck_kernel: clocks per phase
 * Records of one launch are consecutive, one per work-group in blockIdx order; n2d2hip_launch_log_entry() gives the
 * launch's first record.  Launches that do not fit the buffer any more run unprobed.
 */
#ifndef N2D2HIP_PROBE_H
#define N2D2HIP_PROBE_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define N2D2HIP_PROBE_RECORD 16

/* Hands the library a zero-filled device buffer for the records.  Checked on the host before any kernel may write there:
 * memory of the current device, 8-byte aligned, `bytes` inside one allocation.  The buffer must outlive n2d2hip_probe_end. */
int n2d2hip_probe_begin(void* device_buffer, size_t bytes);
/* Stops probing; *records_used = records handed to launches since _begin.  Synchronize the streams before reading them. */
int n2d2hip_probe_end(long long* records_used);

#ifdef __cplusplus
}
#endif
#endif
