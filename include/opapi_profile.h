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

/*
 * Matrix-pipe rate probe: runs nothing but back-to-back v_mfma_i32_32x32x32_i8 on register operands (eight waves per CU,
 * one workgroup per CU, `iterations` x 16 MFMAs per wave, one warm-up launch and one timed launch on the null stream)
 * and writes the achieved int8 operations per second (2 per multiply-add).  uniformRandomOperands = 0: all-zero operands;
 * non-zero: every operand byte uniform over [-127, 127], like the benchmark's weights.  The engine clock under matrix load
 * follows the switching activity of the operands, so the second figure is the ceiling for a GEMM on such data.  Allocates
 * and frees a few KB of device memory and synchronises: a measurement call, not for use inside a serving loop.
 * Returns 0 or an aclnn status code.
 */
__attribute__((visibility("default"))) int opapiInt8MfmaRateProbe(int uniformRandomOperands, int iterations,
                                                                  double* opsPerSecond);

/*
 * Workgroup spans of the grouped GEMM's persistent kernels: a measurement of how evenly the static deal of tiles to the
 * workgroups (hence to the eight XCDs) ends.  While on, every workgroup of a ring-kernel launch records when it started
 * and ended (the GPU's 100 MHz real-time counter) and how many tiles it computed; only the last launch of each kind
 * (gmm_swiglu, gmm_dequant, gmm_int32) is kept.  Off by default; costs one branch per workgroup when off.
 * Turning it on allocates three 24 KB device buffers on the current device (once; kept until the process ends) -- the
 * launch paths themselves never allocate -- and discards earlier records; launches on another device, or of more than
 * 1024 workgroups, are not recorded and drop their kind's record.  One launching thread at a time.
 */
__attribute__((visibility("default"))) void opapiGemmWorkgroupSpansEnable(int enable);

/*
 * Synchronises the device, then writes one text line per recorded kind into buf (NUL-terminated):
 * "<name> workgroups <n> tile_rows <r> span_us <last end - first start>" followed, per XCD x = 0..7, by
 * " xcd<x> end_us <when its last workgroup ended> busy <mean (end - start) / span of its workgroups> tiles <min>-<max>".
 * Returns the number of lines, or -1 on an error.
 */
__attribute__((visibility("default"))) int opapiGemmWorkgroupSpansReport(char* buf, size_t cap);

#ifdef __cplusplus
}
#endif
#endif
