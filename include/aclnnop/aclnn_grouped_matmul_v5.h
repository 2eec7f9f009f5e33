/*
 * aclnnGroupedMatmulV5 for MI355X: aclnnGroupedMatmulV4 plus `tuningConfigOptional`.
 *
 * Replaces gmm/grouped_matmul/op_host/op_api/aclnn_grouped_matmul_v5.h:50-71 of the reference (same symbol names,
 * argument order and meaning).  It is the entry point the reference's own example
 * (gmm/grouped_matmul/examples/test_aclnn_grouped_matmul.cpp:178) and graph-mode bridge
 * (gmm/grouped_matmul/op_host/fallback_grouped_matmul.cpp:286-388) call.
 *
 * tuningConfigOptional[0], when present and positive, is the expected number of tokens per expert
 * (aclnn_grouped_matmul.cpp:1957-1992): here it picks the GEMM tile height in place of the static mean M / groups.
 * It never changes results.  Every other argument, restriction and return code is that of aclnnGroupedMatmulV4
 * (aclnn_grouped_matmul_v4.h in this directory).
 */
#ifndef OPS_TRANSFORMER_AMD_ACLNN_GROUPED_MATMUL_V5_H_
#define OPS_TRANSFORMER_AMD_ACLNN_GROUPED_MATMUL_V5_H_

#include "acl/acl.h"
#include "aclnnop/aclnn_grouped_matmul_v4.h"

#ifdef __cplusplus
extern "C" {
#endif

ACLNN_API aclnnStatus aclnnGroupedMatmulV5GetWorkspaceSize(
    const aclTensorList* x, const aclTensorList* weight, const aclTensorList* biasOptional,
    const aclTensorList* scaleOptional, const aclTensorList* offsetOptional, const aclTensorList* antiquantScaleOptional,
    const aclTensorList* antiquantOffsetOptional, const aclTensorList* perTokenScaleOptional,
    const aclTensor* groupListOptional, const aclTensorList* activationInputOptional,
    const aclTensorList* activationQuantScaleOptional, const aclTensorList* activationQuantOffsetOptional,
    int64_t splitItem, int64_t groupType, int64_t groupListType, int64_t actType, aclIntArray* tuningConfigOptional,
    aclTensorList* out, aclTensorList* activationFeatureOutOptional, aclTensorList* dynQuantScaleOutOptional,
    uint64_t* workspaceSize, aclOpExecutor** executor);

ACLNN_API aclnnStatus aclnnGroupedMatmulV5(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor,
                                           aclrtStream stream);

#ifdef __cplusplus
}
#endif
#endif
