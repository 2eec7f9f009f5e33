/*
 * aclnnGroupedMatmulWeightNz — MI355X build.
 * Replaces gmm/grouped_matmul/op_host/op_api/aclnn_grouped_matmul_weight_nz.h:52-62.
 *
 * aclnnGroupedMatmulV5 (aclnn_grouped_matmul_v5.h: same arguments, same restrictions of this build) for a weight whose
 * storage is the blocked FRACTAL_NZ layout [E, N/32, K/16, 16, 32] (storage shape that 5-D shape; view shape the same
 * or [E, K, N]), plus quantGroupSize, the group size of per-group quantisation, which is not built: pass 0.
 */
#ifndef OPS_TRANSFORMER_AMD_ACLNN_GROUPED_MATMUL_WEIGHT_NZ_H_
#define OPS_TRANSFORMER_AMD_ACLNN_GROUPED_MATMUL_WEIGHT_NZ_H_

#include "acl/acl.h"

#ifdef __cplusplus
extern "C" {
#endif

ACLNN_API aclnnStatus aclnnGroupedMatmulWeightNzGetWorkspaceSize(
    const aclTensorList* x, const aclTensorList* weight, const aclTensorList* biasOptional,
    const aclTensorList* scaleOptional, const aclTensorList* offsetOptional, const aclTensorList* antiquantScaleOptional,
    const aclTensorList* antiquantOffsetOptional, const aclTensorList* perTokenScaleOptional,
    const aclTensor* groupListOptional, const aclTensorList* activationInputOptional,
    const aclTensorList* activationQuantScaleOptional, const aclTensorList* activationQuantOffsetOptional,
    int64_t splitItem, int64_t groupType, int64_t groupListType, int64_t actType, aclIntArray* tuningConfigOptional,
    int64_t quantGroupSize, aclTensorList* out, aclTensorList* activationFeatureOutOptional,
    aclTensorList* dynQuantScaleOutOptional, uint64_t* workspaceSize, aclOpExecutor** executor);

ACLNN_API aclnnStatus aclnnGroupedMatmulWeightNz(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor,
                                                 aclrtStream stream);

#ifdef __cplusplus
}
#endif
#endif
