// Two measurement helpers (include/opapi_profile.h), no operator code.
//
// A plain device-to-device copy kernel of known size, used to calibrate the hardware counters that report HBM traffic:
// the same counter is read for this kernel (whose traffic is exactly `bytes` in and `bytes` out) and for the kernel
// under study, and the ratio of the two readings converts counter units to bytes.
//
// A matrix-pipe rate probe: nothing but back-to-back v_mfma_i32_32x32x32_i8 on operands held in registers, eight waves
// per CU.  The engine clock this chip sustains under matrix load depends on how much the operand bits toggle: the probe
// reports the int8 rate for operands of a chosen kind (zeros, or uniform random bytes like the benchmark's weights), i.e.
// the ceiling that a GEMM on such data cannot pass however well it is fed.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <vector>

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

typedef int V4i __attribute__((ext_vector_type(4)));
typedef int V16i __attribute__((ext_vector_type(16)));
constexpr int kProbeThreads = 512;
constexpr int kProbeOperands = 12;  // 8 A fragments + 4 B fragments per lane

// 16 MFMAs per iteration on 8 independent accumulators (128 registers, the footprint of a 128 x 64 wave tile).
__global__ __launch_bounds__(kProbeThreads) void MfmaRateProbeKernel(const V4i* __restrict__ operands, int iterations, int* sink) {
    V4i a[8], b[4];
    for (int i = 0; i < 8; ++i) a[i] = operands[i * kProbeThreads + threadIdx.x];
    for (int i = 0; i < 4; ++i) b[i] = operands[(8 + i) * kProbeThreads + threadIdx.x];
    V16i acc[4][2];
    for (int m = 0; m < 4; ++m)
        for (int n = 0; n < 2; ++n)
            for (int v = 0; v < 16; ++v) acc[m][n][v] = 0;
    for (int it = 0; it < iterations; ++it) {
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
            for (int m = 0; m < 4; ++m) {
                acc[m][0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[4 * s + m], b[2 * s], acc[m][0], 0, 0, 0);
                acc[m][1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[4 * s + m], b[2 * s + 1], acc[m][1], 0, 0, 0);
            }
    }
    int x = 0;
    for (int m = 0; m < 4; ++m)
        for (int n = 0; n < 2; ++n)
            for (int v = 0; v < 16; ++v) x ^= acc[m][n][v];
    if (x == 0x12345678) sink[0] = x;  // keeps the accumulators alive
}

}  // namespace

extern "C" __attribute__((visibility("default"))) int opapiInt8MfmaRateProbe(int uniformRandomOperands, int iterations,
                                                                             double* opsPerSecond) {
    if (iterations <= 0 || opsPerSecond == nullptr) return ACLNN_ERR_PARAM_INVALID;
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) {
        return ACLNN_ERR_RUNTIME_ERROR;
    }
    const size_t words = static_cast<size_t>(kProbeOperands) * kProbeThreads * 4;
    std::vector<int32_t> host(words, 0);
    if (uniformRandomOperands) {
        uint64_t state = 0x9e3779b97f4a7c15ull;  // splitmix64: every byte uniform over [-127, 127]
        for (size_t i = 0; i < words; ++i) {
            uint32_t w = 0;
            for (int byte = 0; byte < 4; ++byte) {
                state += 0x9e3779b97f4a7c15ull;
                uint64_t z = state;
                z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
                z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
                z ^= z >> 31;
                const int v = static_cast<int>(z % 255) - 127;
                w |= static_cast<uint32_t>(v & 0xff) << (8 * byte);
            }
            host[i] = static_cast<int32_t>(w);
        }
    }
    V4i* operands = nullptr;
    int* sink = nullptr;
    hipEvent_t start = nullptr, stop = nullptr;
    int status = ACLNN_ERR_RUNTIME_ERROR;
    float ms = 0.0f;
    if (hipMalloc(&operands, words * 4) == hipSuccess && hipMalloc(&sink, 4) == hipSuccess &&
        hipMemcpy(operands, host.data(), words * 4, hipMemcpyHostToDevice) == hipSuccess &&
        hipEventCreate(&start) == hipSuccess && hipEventCreate(&stop) == hipSuccess) {
        // one untimed launch first: the clock settles under the load within it
        hipLaunchKernelGGL(MfmaRateProbeKernel, dim3(cus), dim3(kProbeThreads), 0, nullptr, operands, iterations, sink);
        if (hipEventRecord(start, nullptr) == hipSuccess) {
            hipLaunchKernelGGL(MfmaRateProbeKernel, dim3(cus), dim3(kProbeThreads), 0, nullptr, operands, iterations, sink);
            if (hipEventRecord(stop, nullptr) == hipSuccess && hipEventSynchronize(stop) == hipSuccess &&
                hipEventElapsedTime(&ms, start, stop) == hipSuccess && ms > 0.0f) {
                // 8 waves x 16 MFMAs per iteration per workgroup, 32 * 32 * 32 * 2 operations each
                *opsPerSecond = static_cast<double>(cus) * 8.0 * 16.0 * iterations * 65536.0 / (ms * 1e-3);
                status = ACL_SUCCESS;
            }
        }
    }
    if (start != nullptr) (void)hipEventDestroy(start);
    if (stop != nullptr) (void)hipEventDestroy(stop);
    if (operands != nullptr) (void)hipFree(operands);
    if (sink != nullptr) (void)hipFree(sink);
    return status;
}

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
