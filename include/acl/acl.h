/*
 * Minimal AscendCL-compatible host surface for the MI355X build of the quantized MoE expert-FFN path.
 *
 * The reference's examples and callers are written against CANN's "acl/acl.h" (not vendored in the reference
 * repository): runtime init, device/stream management, device memory, and the opaque descriptor objects
 * (aclTensor, aclTensorList, aclIntArray, aclOpExecutor) that every aclnn entry point takes.  This header
 * declares the subset those callers use, with the same names and argument meaning, backed by HIP:
 *   usage in the reference: moe/moe_init_routing_v2/examples/test_aclnn_moe_init_routing_v2.cpp:32-61,151-169
 *                           gmm/grouped_matmul/examples/test_aclnn_grouped_matmul.cpp:95-112,155-157
 *   descriptor semantics:   docs/context/数据结构.md:62-70  (view shape, strides, offset, dtype, format, storage shape, data)
 *   return codes:           docs/context/aclnn返回码.md:16-80
 *
 * aclrtStream is a hipStream_t passed as void*.  Device pointers are plain HIP device pointers.
 * Nothing here allocates behind the caller's back: tensors describe caller-owned memory.
 */
#ifndef OPS_TRANSFORMER_AMD_ACL_H_
#define OPS_TRANSFORMER_AMD_ACL_H_

#include <stddef.h>
#include <stdint.h>
#ifndef __cplusplus
#include <stdbool.h>
#endif

#ifdef __cplusplus
extern "C" {
#endif

#define ACL_API __attribute__((visibility("default")))
#define ACLNN_API __attribute__((visibility("default")))

typedef int aclError;
typedef int32_t aclnnStatus;
typedef void* aclrtStream;

typedef struct aclTensor aclTensor;
typedef struct aclTensorList aclTensorList;
typedef struct aclIntArray aclIntArray;
typedef struct aclOpExecutor aclOpExecutor;

/* runtime error code */
#define ACL_SUCCESS 0
#define ACL_ERROR_INVALID_PARAM 100000
#define ACL_ERROR_BAD_ALLOC 200000
#define ACL_ERROR_RT_FAILURE 500000

/* aclnn status codes (docs/context/aclnn返回码.md) */
#define ACLNN_SUCCESS 0
#define ACLNN_ERR_PARAM_NULLPTR 161001
#define ACLNN_ERR_PARAM_INVALID 161002
#define ACLNN_ERR_RUNTIME_ERROR 361001
#define ACLNN_ERR_INNER 561000
#define ACLNN_ERR_INNER_INFERSHAPE_ERROR 561001
#define ACLNN_ERR_INNER_TILING_ERROR 561002
#define ACLNN_ERR_INNER_CREATE_EXECUTOR 561101
#define ACLNN_ERR_INNER_NULLPTR 561103

/* Element types; numeric values follow ge::DataType (gmm/grouped_matmul/op_kernel/grouped_matmul_tiling_key.h:23-28). */
typedef enum {
    ACL_DT_UNDEFINED = -1,
    ACL_FLOAT = 0,
    ACL_FLOAT16 = 1,
    ACL_INT8 = 2,
    ACL_INT32 = 3,
    ACL_UINT8 = 4,
    ACL_INT16 = 6,
    ACL_UINT16 = 7,
    ACL_UINT32 = 8,
    ACL_INT64 = 9,
    ACL_UINT64 = 10,
    ACL_DOUBLE = 11,
    ACL_BOOL = 12,
    ACL_BF16 = 27,
    ACL_INT4 = 29
} aclDataType;

typedef enum {
    ACL_FORMAT_UNDEFINED = -1,
    ACL_FORMAT_NCHW = 0,
    ACL_FORMAT_NHWC = 1,
    ACL_FORMAT_ND = 2,
    ACL_FORMAT_FRACTAL_NZ = 29
} aclFormat;

typedef enum {
    ACL_MEM_MALLOC_HUGE_FIRST = 0,
    ACL_MEM_MALLOC_HUGE_ONLY = 1,
    ACL_MEM_MALLOC_NORMAL_ONLY = 2
} aclrtMemMallocPolicy;

typedef enum {
    ACL_MEMCPY_HOST_TO_HOST = 0,
    ACL_MEMCPY_HOST_TO_DEVICE = 1,
    ACL_MEMCPY_DEVICE_TO_HOST = 2,
    ACL_MEMCPY_DEVICE_TO_DEVICE = 3
} aclrtMemcpyKind;

/* ---- runtime ---- */
ACL_API aclError aclInit(const char* configPath);
ACL_API aclError aclFinalize(void);
ACL_API aclError aclrtSetDevice(int32_t deviceId);
ACL_API aclError aclrtResetDevice(int32_t deviceId);
ACL_API aclError aclrtCreateStream(aclrtStream* stream);
ACL_API aclError aclrtDestroyStream(aclrtStream stream);
ACL_API aclError aclrtSynchronizeStream(aclrtStream stream);
ACL_API aclError aclrtMalloc(void** devPtr, size_t size, aclrtMemMallocPolicy policy);
ACL_API aclError aclrtFree(void* devPtr);
ACL_API aclError aclrtMemcpy(void* dst, size_t destMax, const void* src, size_t count, aclrtMemcpyKind kind);
ACL_API aclError aclrtMemset(void* devPtr, size_t maxCount, int32_t value, size_t count);

/* ---- descriptors ---- */
/* viewDims/stride are in elements; offset is an element offset from `tensorData`; the tensor does not own the memory. */
ACL_API aclTensor* aclCreateTensor(const int64_t* viewDims, uint64_t viewDimsNum, aclDataType dataType,
                                   const int64_t* stride, int64_t offset, aclFormat format,
                                   const int64_t* storageDims, uint64_t storageDimsNum, void* tensorData);
ACL_API aclnnStatus aclDestroyTensor(const aclTensor* tensor);
/* The list keeps the tensor pointers; destroying the list destroys its tensors (CANN behaviour). */
ACL_API aclTensorList* aclCreateTensorList(const aclTensor* const* value, uint64_t size);
ACL_API aclnnStatus aclDestroyTensorList(const aclTensorList* tensorList);
ACL_API aclIntArray* aclCreateIntArray(const int64_t* value, uint64_t size);
ACL_API aclnnStatus aclDestroyIntArray(const aclIntArray* array);
/* Releases an executor whose second-phase call will never be made. */
ACL_API aclnnStatus aclDestroyAclOpExecutor(aclOpExecutor* executor);

/* Text of the most recent error raised on the calling thread by an aclnn entry point ("" if none). */
ACL_API const char* aclGetRecentErrMsg(void);
/* Looked up by the reference's dlsym-based binder (common/include/fallback/fallback.h:79-135); clears the per-thread error text. */
ACL_API void ResetCacheThreadLocal(void);

#ifdef __cplusplus
}
#endif

#endif /* OPS_TRANSFORMER_AMD_ACL_H_ */
