// A plain device-to-device copy kernel of known size, used to calibrate the hardware counters that report HBM traffic:
// the same counter is read for this kernel (whose traffic is exactly `bytes` in and `bytes` out) and for the kernel
// under study, and the ratio of the two readings converts counter units to bytes.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "opapi_common.h"
#include "opapi_profile.h"

namespace {

constexpr int kCopyThreads = 256;
constexpr int kCopyBlocks = 256 * 16;  // 16 blocks per CU, grid-stride

__global__ __launch_bounds__(kCopyThreads) void CalibrationCopyKernel(uint4* __restrict__ dst,
                                                                      const uint4* __restrict__ src, size_t packets) {
    const size_t stride = static_cast<size_t>(gridDim.x) * kCopyThreads;
    for (size_t i = static_cast<size_t>(blockIdx.x) * kCopyThreads + threadIdx.x; i < packets; i += stride) {
        dst[i] = src[i];
    }
}

}  // namespace

extern "C" __attribute__((visibility("default"))) int opapiCalibrationCopy(void* dst, const void* src, size_t bytes,
                                                                           void* stream) {
    if (dst == nullptr || src == nullptr || bytes == 0 || bytes % 16 != 0 ||
        reinterpret_cast<uintptr_t>(dst) % 16 != 0 || reinterpret_cast<uintptr_t>(src) % 16 != 0) {
        return ACLNN_ERR_PARAM_INVALID;
    }
    opapi::KernelTimer timer("calibration_copy", static_cast<hipStream_t>(stream));
    hipLaunchKernelGGL(CalibrationCopyKernel, dim3(kCopyBlocks), dim3(kCopyThreads), 0, static_cast<hipStream_t>(stream),
                       static_cast<uint4*>(dst), static_cast<const uint4*>(src), bytes / 16);
    return hipGetLastError() == hipSuccess ? ACL_SUCCESS : ACLNN_ERR_INNER;
}
