/*
 * aclnnGroupedMatmulV4 — MI355X build, int8 x int8 grouped GEMM split along M (the MoE down-projection).
 * Replaces: gmm/grouped_matmul/op_host/op_api/aclnn_grouped_matmul_v4.h:69-90 (same symbols, same argument order).
 *
 * Supported on this path: single-tensor lists, groupType 0 (split M), splitItem 2/3, groupListType 0 (cumsum) or 1 (counts),
 * x int8 [M,K], weight int8 [E,K,N] (ND or transposed view), and
 *   scale absent            -> out INT32 : out = acc                                           (raw accumulators)
 *   scale BF16  [E,N] + perTokenScale FP32 [M] -> out BF16 : bf16((float(acc) * scale) * perToken)
 *   scale FP32  [E,N] + perTokenScale FP32 [M] -> out FLOAT16 (reference pairing) or BF16 (extension)
 *   scale without perTokenScale                -> out = cast(float(acc) * scale)
 * actType must be 0 (none).  Every other dtype family of the reference op returns ACLNN_ERR_PARAM_INVALID.
 */
#ifndef OPS_TRANSFORMER_AMD_ACLNN_GROUPED_MATMUL_V4_H_
#define OPS_TRANSFORMER_AMD_ACLNN_GROUPED_MATMUL_V4_H_

#include "acl/acl.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
    GMM_ACT_TYPE_NONE = 0LL,
    GMM_ACT_TYPE_RELU = 1LL,
    GMM_ACT_TYPE_GELU_TANH = 2LL,
    GMM_ACT_TYPE_GELU_ERR_FUNC = 3LL,
    GMM_ACT_TYPE_FAST_GELU = 4LL,
    GMM_ACT_TYPE_SILU = 5LL,
    END_ACT_TYPE_ENUM
} GMMActType;

ACLNN_API aclnnStatus aclnnGroupedMatmulV4GetWorkspaceSize(
    const aclTensorList* x, const aclTensorList* weight, const aclTensorList* biasOptional,
    const aclTensorList* scaleOptional, const aclTensorList* offsetOptional,
    const aclTensorList* antiquantScaleOptional, const aclTensorList* antiquantOffsetOptional,
    const aclTensorList* perTokenScaleOptional, const aclTensor* groupListOptional,
    const aclTensorList* activationInputOptional, const aclTensorList* activationQuantScaleOptional,
    const aclTensorList* activationQuantOffsetOptional, int64_t splitItem, int64_t groupType, int64_t groupListType,
    int64_t actType, aclTensorList* out, aclTensorList* activationFeatureOutOptional,
    aclTensorList* dynQuantScaleOutOptional, uint64_t* workspaceSize, aclOpExecutor** executor);

ACLNN_API aclnnStatus aclnnGroupedMatmulV4(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor,
                                           aclrtStream stream);

#ifdef __cplusplus
}
#endif
#endif
