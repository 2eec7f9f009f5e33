// Shared host-side plumbing of the aclnn C-ABI: descriptor objects, executors, error reporting, argument checks.
// Every aclnn entry point is two-phase (docs/context/两段式接口.md:5-20 in the reference): phase 1 validates, plans and
// returns a heap executor plus the workspace byte count; phase 2 enqueues on the caller's stream and consumes the executor.
#pragma once

#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <string>
#include <vector>

#include "acl/acl.h"

struct aclTensor {
    std::vector<int64_t> dims;     // view shape
    std::vector<int64_t> strides;  // in elements
    std::vector<int64_t> storage;  // storage shape
    int64_t offset = 0;            // in elements
    aclDataType dtype = ACL_DT_UNDEFINED;
    aclFormat format = ACL_FORMAT_ND;
    void* data = nullptr;
};

struct aclTensorList {
    std::vector<const aclTensor*> items;
};

struct aclIntArray {
    std::vector<int64_t> values;
};

namespace opapi {
// An input whose view is not contiguous is copied into the workspace (behind the operator's own part of it) at the
// start of the second phase, as the reference makes such inputs contiguous before its kernels run
// (gmm/grouped_matmul_swiglu_quant/op_host/op_api/aclnn_grouped_matmul_swiglu_quant.cpp:431-445).
struct StagedInput {
    void* slotAddr = nullptr;  // address of the executor's pointer field that the kernels read
    uint64_t offset = 0;       // byte offset of the copy inside the staging area
    const char* src = nullptr; // first element of the view
    int64_t numel = 0;
    int32_t nd = 0;
    int32_t elemSize = 0;
    int64_t dims[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    int64_t strides[8] = {0, 0, 0, 0, 0, 0, 0, 0};  // in elements
};
}  // namespace opapi

struct aclOpExecutor {
    uint64_t workspaceBytes = 0;  // what the caller provides: the operator's own workspace, then the staging area
    uint64_t stagingBase = 0;
    uint64_t stagingBytes = 0;
    std::vector<opapi::StagedInput> staged;
    virtual ~aclOpExecutor() = default;
    // Enqueue all kernels of the op on `stream`; must not synchronise with the host.
    virtual aclnnStatus Run(void* workspace, hipStream_t stream) = 0;

    // Stores into *slot the pointer the kernels are to read input `t` through: its data when the view is contiguous
    // (or absent, or empty), otherwise a 256-byte aligned stand-in that the second phase replaces by the address of a
    // contiguous copy in the workspace.  Planning decisions that look at pointer alignment therefore hold for both.
    template <typename T>
    aclnnStatus Bind(const aclTensor* t, T** slot) {
        const void* p = nullptr;
        const aclnnStatus st = BindRaw(t, slot, &p);
        *slot = static_cast<T*>(const_cast<void*>(p));
        return st;
    }
    // Adds the staging area behind `ownBytes` of operator workspace and sets workspaceBytes.
    void SealWorkspace(uint64_t ownBytes) {
        stagingBase = (ownBytes + 255) / 256 * 256;
        workspaceBytes = stagingBytes > 0 ? stagingBase + stagingBytes : ownBytes;
    }

   private:
    aclnnStatus BindRaw(const aclTensor* t, void* slotAddr, const void** now);
};

namespace opapi {

void SetError(const char* fmt, ...) __attribute__((format(printf, 1, 2)));
void ClearError();

// Phase-2 body shared by all ops: argument checks, Run, launch-error check, executor release.
aclnnStatus RunAndRelease(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor, aclrtStream stream);

inline int64_t ElemSize(aclDataType dt) {
    switch (dt) {
        case ACL_FLOAT: case ACL_INT32: case ACL_UINT32: return 4;
        case ACL_FLOAT16: case ACL_BF16: case ACL_INT16: case ACL_UINT16: return 2;
        case ACL_INT8: case ACL_UINT8: case ACL_BOOL: return 1;
        case ACL_INT64: case ACL_UINT64: case ACL_DOUBLE: return 8;
        default: return 0;
    }
}

inline int64_t Numel(const aclTensor* t) {
    int64_t n = 1;
    for (int64_t d : t->dims) n *= d;
    return n;
}

inline bool IsEmpty(const aclTensor* t) { return t == nullptr || Numel(t) == 0; }

// Extents are caller data: a negative one would make every size derived from it meaningless.
inline bool HasNegativeDim(const aclTensor* t) {
    if (t == nullptr) return false;
    for (int64_t d : t->dims) {
        if (d < 0) return true;
    }
    return false;
}

// Row-major contiguous view (dims of extent 1 may carry any stride).
inline bool IsContiguous(const aclTensor* t) {
    int64_t expect = 1;
    for (int i = (int)t->dims.size() - 1; i >= 0; --i) {
        if (t->dims[i] != 1 && t->strides[i] != expect) return false;
        expect *= t->dims[i];
    }
    return true;
}

// The last two view dims are a transpose of contiguous storage: strides (.., 1, dim[-2]).  This is how the reference
// recognises a transposed weight (gmm/grouped_matmul/op_host/op_api/aclnn_grouped_matmul_util.cpp:20-32).
inline bool IsLastTwoDimsTransposed(const aclTensor* t) {
    const int n = (int)t->dims.size();
    if (n < 2) return false;
    const int64_t d1 = t->dims[n - 1], d2 = t->dims[n - 2];
    if (t->strides[n - 2] != 1 || t->strides[n - 1] != d2) return false;
    int64_t expect = d1 * d2;
    for (int i = n - 3; i >= 0; --i) {
        if (t->dims[i] != 1 && t->strides[i] != expect) return false;
        expect *= t->dims[i];
    }
    // a [.., 1, 1] tail is both; call it not transposed
    return !(d1 == 1 && d2 == 1);
}

inline char* DataPtr(const aclTensor* t) {
    return t == nullptr ? nullptr : static_cast<char*>(t->data) + t->offset * ElemSize(t->dtype);
}

inline uint64_t AlignUp(uint64_t v, uint64_t a) { return (v + a - 1) / a * a; }

std::string ShapeStr(const aclTensor* t);

// Brackets the kernel launches made during its lifetime with HIP events on `stream` when kernel timing is enabled
// (include/opapi_profile.h); otherwise does nothing.
class KernelTimer {
   public:
    KernelTimer(const char* name, hipStream_t stream);
    ~KernelTimer();
    KernelTimer(const KernelTimer&) = delete;
    KernelTimer& operator=(const KernelTimer&) = delete;

   private:
    const char* name_;
    hipStream_t stream_;
    hipEvent_t start_ = nullptr;
};

// Raises a kernel's dynamic-LDS limit to `bytes` on the current device.  The opt-in belongs to the kernel as loaded on
// one device, so it is made once per device of the process; `done` is the caller's per-kernel bit set (one bit per device).
inline hipError_t EnsureDynamicLds(const void* kernel, int bytes, std::atomic<uint64_t>& done) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return hipErrorInvalidDevice;
    const uint64_t devBit = 1ull << (dev & 63);
    if ((done.load(std::memory_order_acquire) & devBit) != 0) return hipSuccess;
    const hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e == hipSuccess) done.fetch_or(devBit, std::memory_order_release);
    return e;
}

}  // namespace opapi

#define OPAPI_CHECK(cond, code, ...)            \
    do {                                        \
        if (!(cond)) {                          \
            ::opapi::SetError(__VA_ARGS__);     \
            return (code);                      \
        }                                       \
    } while (0)

// Rejects tensors (absent ones pass) that carry a negative extent.
#define OPAPI_CHECK_EXTENTS(...)                                                                              \
    do {                                                                                                      \
        const aclTensor* const opapiTensors_[] = {__VA_ARGS__};                                               \
        for (const aclTensor* opapiT_ : opapiTensors_) {                                                      \
            OPAPI_CHECK(!::opapi::HasNegativeDim(opapiT_), ACLNN_ERR_PARAM_INVALID,                           \
                        "%s: a tensor has a negative extent: %s", __func__, ::opapi::ShapeStr(opapiT_).c_str()); \
        }                                                                                                     \
    } while (0)

// Binds input `t` to the executor's pointer field (see aclOpExecutor::Bind); on failure the executor is released.
#define OPAPI_BIND(ex, t, slot)                             \
    do {                                                    \
        const aclnnStatus opapiBind_ = (ex)->Bind((t), (slot)); \
        if (opapiBind_ != ACLNN_SUCCESS) {                  \
            delete (ex);                                    \
            return opapiBind_;                              \
        }                                                   \
    } while (0)

#define OPAPI_CHECK_NOTNULL(ptr, name) \
    OPAPI_CHECK((ptr) != nullptr, ACLNN_ERR_PARAM_NULLPTR, "%s: argument %s must not be null", __func__, name)
