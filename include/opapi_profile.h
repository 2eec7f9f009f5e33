/*
 * Per-kernel device timing for the MI355X operator library.
 *
 * No counterpart in the reference's headers: there, per-kernel durations come from the external `msprof op` tool
 * (docs/debug/op_debug_prof.md:35-67).  Here the library can bracket each of its own kernel launches with a pair of HIP
 * events on the stream the kernel is launched on, so that a caller (the benchmark) can read the average duration of,
 * say, the gate/up GEMM kernel alone while the whole operator chain runs.
 *
 * Timing is off by default and costs one branch per launch when off.  While on, every launch records two events and
 * keeps them until the next report; recording does not synchronise.  Not thread-safe against concurrent operator calls.
 */
#ifndef OPS_TRANSFORMER_AMD_OPAPI_PROFILE_H_
#define OPS_TRANSFORMER_AMD_OPAPI_PROFILE_H_

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Turns event recording on (non-zero) or off (zero); pending records are discarded. */
__attribute__((visibility("default"))) void opapiKernelTimerEnable(int enable);

/*
 * Waits for every recorded launch to finish, then writes one text line per kernel name,
 * "<name> <launches> <total_ms>\n", into buf (NUL-terminated, truncated to cap) and clears the records.
 * Returns the number of distinct kernel names, or -1 on a HIP error.
 */
__attribute__((visibility("default"))) int opapiKernelTimerReport(char* buf, size_t cap);

/*
 * Launches a plain copy kernel ("calibration_copy") moving `bytes` (a multiple of 16, both pointers 16-byte aligned)
 * from src to dst on `stream`.  Its HBM traffic is known exactly (bytes read + bytes written), so reading a hardware
 * traffic counter for it gives the factor that converts the counter's units to bytes for the other kernels.
 * Returns 0, or an aclnn status code for bad arguments / a failed launch.
 */
__attribute__((visibility("default"))) int opapiCalibrationCopy(void* dst, const void* src, size_t bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif
