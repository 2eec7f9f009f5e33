// HIP-backed implementation of the small AscendCL host surface declared in include/acl/acl.h, plus the shared
// phase-2 driver and the per-thread error text of the aclnn entry points.
#include "opapi_common.h"

#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <new>

#include "opapi_profile.h"

namespace {
thread_local std::string g_lastError;

aclError FromHip(hipError_t e) {
    if (e == hipSuccess) return ACL_SUCCESS;
    opapi::SetError("HIP runtime error %d: %s", (int)e, hipGetErrorString(e));
    return e == hipErrorOutOfMemory ? ACL_ERROR_BAD_ALLOC : ACL_ERROR_RT_FAILURE;
}
}  // namespace

namespace opapi {

void SetError(const char* fmt, ...) {
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    try {
        g_lastError = buf;
    } catch (...) {  // out of host memory: the status code still reaches the caller, the text does not
        g_lastError.clear();
    }
    if (const char* v = std::getenv("OPAPI_LOG_ERRORS")) {
        if (v[0] != '\0' && v[0] != '0') fprintf(stderr, "[opapi] %s\n", buf);
    }
}

void ClearError() { g_lastError.clear(); }

std::string ShapeStr(const aclTensor* t) {
    if (t == nullptr) return "null";
    std::string s = "[";
    for (size_t i = 0; i < t->dims.size(); ++i) {
        if (i) s += ",";
        s += std::to_string(t->dims[i]);
    }
    return s + "]";
}

}  // namespace opapi

aclnnStatus aclOpExecutor::BindRaw(const aclTensor* t, void* slotAddr, const void** now) {
    *now = nullptr;
    if (t == nullptr) return ACLNN_SUCCESS;
    *now = opapi::DataPtr(t);
    if (opapi::Numel(t) == 0 || opapi::IsContiguous(t)) return ACLNN_SUCCESS;
    opapi::StagedInput s;
    s.slotAddr = slotAddr;
    s.offset = stagingBytes;
    s.src = opapi::DataPtr(t);
    s.numel = opapi::Numel(t);
    s.nd = static_cast<int32_t>(t->dims.size());
    s.elemSize = static_cast<int32_t>(opapi::ElemSize(t->dtype));
    OPAPI_CHECK(s.nd <= 8 && t->strides.size() == t->dims.size(), ACLNN_ERR_PARAM_INVALID,
                "a non-contiguous input has more than 8 dimensions or no strides");
    OPAPI_CHECK(s.elemSize > 0, ACLNN_ERR_PARAM_INVALID, "a non-contiguous input has an unsupported data type");
    for (int d = 0; d < s.nd; ++d) {
        OPAPI_CHECK(t->strides[d] >= 0, ACLNN_ERR_PARAM_INVALID, "negative strides are not supported (%s)",
                    opapi::ShapeStr(t).c_str());
        s.dims[d] = t->dims[d];
        s.strides[d] = t->strides[d];
    }
    OPAPI_CHECK(t->data != nullptr, ACLNN_ERR_PARAM_NULLPTR, "a tensor carries no device memory");
    try {
        staged.push_back(s);
    } catch (...) {
        opapi::SetError("out of host memory");
        return ACLNN_ERR_INNER;
    }
    stagingBytes += (static_cast<uint64_t>(s.numel) * static_cast<uint64_t>(s.elemSize) + 255) / 256 * 256;
    // aligned stand-in until the second phase knows the workspace address
    *now = reinterpret_cast<const void*>(static_cast<uintptr_t>(1) << 20);
    return ACLNN_SUCCESS;
}

namespace opapi {

namespace {
// dst[i] = src[sum_d index_d(i) * stride_d], i running over the view in row-major order; one element per thread.
template <typename T>
__global__ void StridedCopyKernel(StagedInput s, T* dst) {
    const int64_t step = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < s.numel; i += step) {
        int64_t rest = i, off = 0;
        for (int d = s.nd - 1; d >= 0; --d) {
            off += (rest % s.dims[d]) * s.strides[d];
            rest /= s.dims[d];
        }
        dst[i] = reinterpret_cast<const T*>(s.src)[off];
    }
}

template <typename T>
void LaunchStridedCopy(const StagedInput& s, void* dst, hipStream_t stream) {
    int64_t blocks = (s.numel + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    hipLaunchKernelGGL(StridedCopyKernel<T>, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream, s, static_cast<T*>(dst));
}
}  // namespace

aclnnStatus RunAndRelease(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor, aclrtStream stream) {
    if (executor == nullptr) {
        SetError("second-phase call: executor must not be null");
        return ACLNN_ERR_PARAM_NULLPTR;
    }
    aclnnStatus st = ACLNN_SUCCESS;
    if (executor->workspaceBytes > 0 && workspace == nullptr) {
        SetError("second-phase call: workspace is null but %llu bytes are required",
                 (unsigned long long)executor->workspaceBytes);
        st = ACLNN_ERR_PARAM_NULLPTR;
    } else if (workspaceSize < executor->workspaceBytes) {
        SetError("second-phase call: workspaceSize %llu is smaller than the required %llu",
                 (unsigned long long)workspaceSize, (unsigned long long)executor->workspaceBytes);
        st = ACLNN_ERR_PARAM_INVALID;
    } else if (!executor->staged.empty() && reinterpret_cast<uintptr_t>(workspace) % 256 != 0) {
        SetError("second-phase call: the workspace must be 256-byte aligned when non-contiguous inputs are staged in it");
        st = ACLNN_ERR_PARAM_INVALID;
    } else {
        for (const StagedInput& s : executor->staged) {
            char* const dst = static_cast<char*>(workspace) + executor->stagingBase + s.offset;
            KernelTimer timer("stage_input", static_cast<hipStream_t>(stream));
            switch (s.elemSize) {
                case 1: LaunchStridedCopy<uint8_t>(s, dst, static_cast<hipStream_t>(stream)); break;
                case 2: LaunchStridedCopy<uint16_t>(s, dst, static_cast<hipStream_t>(stream)); break;
                case 4: LaunchStridedCopy<uint32_t>(s, dst, static_cast<hipStream_t>(stream)); break;
                default: LaunchStridedCopy<uint64_t>(s, dst, static_cast<hipStream_t>(stream)); break;
            }
            void* const patched = dst;
            memcpy(s.slotAddr, &patched, sizeof(void*));
        }
        st = executor->Run(workspace, static_cast<hipStream_t>(stream));
        if (st == ACLNN_SUCCESS) {
            hipError_t e = hipGetLastError();
            if (e != hipSuccess) {
                SetError("kernel launch failed: %s", hipGetErrorString(e));
                st = ACLNN_ERR_RUNTIME_ERROR;
            }
        }
    }
    delete executor;  // phase 2 consumes the executor
    return st;
}

namespace {
struct TimedLaunch {
    const char* name;
    hipEvent_t start, stop;
};
bool g_timerOn = false;
std::mutex g_timedMutex;  // guards g_timed: operators may be enqueued from several host threads
std::vector<TimedLaunch> g_timed;

void DropTimed() {  // caller holds g_timedMutex
    for (TimedLaunch& t : g_timed) {
        (void)hipEventDestroy(t.start);
        (void)hipEventDestroy(t.stop);
    }
    g_timed.clear();
}
}  // namespace

KernelTimer::KernelTimer(const char* name, hipStream_t stream) : name_(name), stream_(stream) {
    if (!g_timerOn) return;
    if (hipEventCreate(&start_) != hipSuccess) { start_ = nullptr; return; }
    (void)hipEventRecord(start_, stream_);
}

KernelTimer::~KernelTimer() {
    if (start_ == nullptr) return;
    hipEvent_t stop = nullptr;
    if (hipEventCreate(&stop) != hipSuccess) { (void)hipEventDestroy(start_); return; }
    (void)hipEventRecord(stop, stream_);
    try {
        std::lock_guard<std::mutex> lock(g_timedMutex);
        g_timed.push_back({name_, start_, stop});
    } catch (...) {  // out of host memory: this launch goes untimed
        (void)hipEventDestroy(start_);
        (void)hipEventDestroy(stop);
    }
}

}  // namespace opapi

extern "C" {

void opapiKernelTimerEnable(int enable) {
    std::lock_guard<std::mutex> lock(opapi::g_timedMutex);
    opapi::DropTimed();
    opapi::g_timerOn = enable != 0;
}

int opapiKernelTimerReport(char* buf, size_t cap) try {
    std::lock_guard<std::mutex> lock(opapi::g_timedMutex);
    std::map<std::string, std::pair<int, double>> agg;
    int rc = 0;
    for (opapi::TimedLaunch& t : opapi::g_timed) {
        float ms = 0.0f;
        if (hipEventSynchronize(t.stop) != hipSuccess || hipEventElapsedTime(&ms, t.start, t.stop) != hipSuccess) rc = -1;
        auto& a = agg[t.name];
        a.first += 1;
        a.second += ms;
    }
    opapi::DropTimed();
    std::string out;
    for (auto& kv : agg) {
        char line[256];
        snprintf(line, sizeof(line), "%s %d %.6f\n", kv.first.c_str(), kv.second.first, kv.second.second);
        out += line;
    }
    if (buf != nullptr && cap > 0) {
        const size_t n = out.size() < cap - 1 ? out.size() : cap - 1;
        memcpy(buf, out.data(), n);
        buf[n] = '\0';
    }
    return rc < 0 ? rc : static_cast<int>(agg.size());
} catch (...) {  // out of host memory while building the report
    return -1;
}

aclError aclInit(const char*) { return ACL_SUCCESS; }
aclError aclFinalize(void) { return ACL_SUCCESS; }
aclError aclrtSetDevice(int32_t deviceId) { return FromHip(hipSetDevice(deviceId)); }
aclError aclrtResetDevice(int32_t deviceId) {
    (void)deviceId;
    return FromHip(hipDeviceSynchronize());
}
aclError aclrtCreateStream(aclrtStream* stream) {
    if (stream == nullptr) return ACL_ERROR_INVALID_PARAM;
    hipStream_t s = nullptr;
    aclError e = FromHip(hipStreamCreate(&s));
    *stream = s;
    return e;
}
aclError aclrtDestroyStream(aclrtStream stream) { return FromHip(hipStreamDestroy(static_cast<hipStream_t>(stream))); }
aclError aclrtSynchronizeStream(aclrtStream stream) {
    return FromHip(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
}
aclError aclrtMalloc(void** devPtr, size_t size, aclrtMemMallocPolicy) {
    if (devPtr == nullptr) return ACL_ERROR_INVALID_PARAM;
    return FromHip(hipMalloc(devPtr, size));
}
aclError aclrtFree(void* devPtr) { return FromHip(hipFree(devPtr)); }
aclError aclrtMemcpy(void* dst, size_t destMax, const void* src, size_t count, aclrtMemcpyKind kind) {
    if (count > destMax) return ACL_ERROR_INVALID_PARAM;
    if (count == 0) return ACL_SUCCESS;
    hipMemcpyKind k = hipMemcpyDefault;
    switch (kind) {
        case ACL_MEMCPY_HOST_TO_HOST: k = hipMemcpyHostToHost; break;
        case ACL_MEMCPY_HOST_TO_DEVICE: k = hipMemcpyHostToDevice; break;
        case ACL_MEMCPY_DEVICE_TO_HOST: k = hipMemcpyDeviceToHost; break;
        case ACL_MEMCPY_DEVICE_TO_DEVICE: k = hipMemcpyDeviceToDevice; break;
    }
    return FromHip(hipMemcpy(dst, src, count, k));
}
aclError aclrtMemset(void* devPtr, size_t maxCount, int32_t value, size_t count) {
    if (count > maxCount) return ACL_ERROR_INVALID_PARAM;
    return FromHip(hipMemset(devPtr, value, count));
}

aclTensor* aclCreateTensor(const int64_t* viewDims, uint64_t viewDimsNum, aclDataType dataType, const int64_t* stride,
                           int64_t offset, aclFormat format, const int64_t* storageDims, uint64_t storageDimsNum,
                           void* tensorData) {
    if ((viewDimsNum > 0 && viewDims == nullptr) || viewDimsNum > 8 || storageDimsNum > 8) return nullptr;
    aclTensor* t = new (std::nothrow) aclTensor();
    if (t == nullptr) return nullptr;
    try {  // no exception may cross the C boundary
        t->dims.assign(viewDims, viewDims + viewDimsNum);
        if (stride != nullptr) {
            t->strides.assign(stride, stride + viewDimsNum);
        } else {  // contiguous default
            t->strides.assign(viewDimsNum, 1);
            for (int i = (int)viewDimsNum - 2; i >= 0; --i) t->strides[i] = t->strides[i + 1] * t->dims[i + 1];
        }
        if (storageDims != nullptr) t->storage.assign(storageDims, storageDims + storageDimsNum);
    } catch (...) {
        delete t;
        return nullptr;
    }
    t->offset = offset;
    t->dtype = dataType;
    t->format = format;
    t->data = tensorData;
    return t;
}
aclnnStatus aclDestroyTensor(const aclTensor* tensor) {
    delete tensor;
    return ACLNN_SUCCESS;
}
aclTensorList* aclCreateTensorList(const aclTensor* const* value, uint64_t size) {
    if (size > 0 && value == nullptr) return nullptr;
    aclTensorList* l = new (std::nothrow) aclTensorList();
    if (l == nullptr) return nullptr;
    try {
        l->items.assign(value, value + size);
    } catch (...) {
        delete l;
        return nullptr;
    }
    return l;
}
aclnnStatus aclDestroyTensorList(const aclTensorList* tensorList) {
    if (tensorList != nullptr) {
        for (const aclTensor* t : tensorList->items) delete t;
        delete tensorList;
    }
    return ACLNN_SUCCESS;
}
aclIntArray* aclCreateIntArray(const int64_t* value, uint64_t size) {
    if (size > 0 && value == nullptr) return nullptr;
    aclIntArray* a = new (std::nothrow) aclIntArray();
    if (a == nullptr) return nullptr;
    try {
        a->values.assign(value, value + size);
    } catch (...) {
        delete a;
        return nullptr;
    }
    return a;
}
aclnnStatus aclDestroyIntArray(const aclIntArray* array) {
    delete array;
    return ACLNN_SUCCESS;
}
aclnnStatus aclDestroyAclOpExecutor(aclOpExecutor* executor) {
    delete executor;
    return ACLNN_SUCCESS;
}

const char* aclGetRecentErrMsg(void) { return g_lastError.c_str(); }
void ResetCacheThreadLocal(void) { g_lastError.clear(); }

}  // extern "C"
