/*
 * aclnnGroupedMatmulFinalizeRouting / V2 / V3 — MI355X build: the int8 down projection fused with the weighted combine.
 * Replaces gmm/grouped_matmul_finalize_routing/op_host/op_api/aclnn_grouped_matmul_finalize_routing.h:47-52,
 * aclnn_grouped_matmul_finalize_routing_v2.h:51-58 and aclnn_grouped_matmul_finalize_routing_v3.h:50-57 (same symbol
 * names, argument order and meaning; arithmetic of op_kernel/grouped_matmul_finalize_routing.h:217-254,390-495).
 *
 *   out[:, :] = 0;  out[sharedInputOffset + j, :] = float(sharedInput[j, :]) * sharedInputWeight
 *   for every row r of x1 (group e = the expert whose row range holds r):
 *     out[rowIndex[r], :] += (float(acc[r, :]) * scale[e, :]) * (pertokenScale[r] * logit[r]) + logit[r] * bias[e, :]
 * acc = int32 x1[r, :] @ x2[e]; the additions into one output row arrive in no fixed order (fp32 atomics, as in the
 * reference), so results are reproducible only up to fp32 rounding of a sum of top-k terms.
 *
 * x1 INT8 [m, k]; out FLOAT [batch, n] with batch <= m; scale FLOAT or BF16 [e, n] (or [e, 1, n]); bias BF16 or FLOAT
 * [e, n]; pertokenScale, logit FLOAT [m]; rowIndex INT64 or INT32 [m]; groupList INT64 [e] (INT32 also accepted);
 * sharedInput BF16 or FLOAT16 [rows, n] with sharedInputOffset + rows <= batch; dtype must be 0 (FLOAT);
 * transposeX1 / transposeX2 false; groupListType 0 (cumsum) or 1 (count).
 *
 * aclnnGroupedMatmulFinalizeRoutingWeightNz / WeightNzV2 (replacing aclnn_grouped_matmul_finalize_routing_weight_nz.h:48-53
 * and aclnn_grouped_matmul_finalize_routing_weight_nz_v2.h:55-61) are the reference's route for INT8 weights: x2 is stored
 * in the blocked FRACTAL_NZ layout [e, n/32, k/16, 16, 32] (storage shape; the view shape is that or [e, k, n]).
 *
 * This build also takes x2 as INT8 [e, k, n] ND in the plain entry points (the K-contiguous storage seen through a
 * transposed view is the fast ND layout, as for aclnnGroupedMatmulV4).  The reference's ND entry points take only INT4
 * weights packed in INT32; those are rejected here with ACLNN_ERR_PARAM_INVALID.  bias,
 * pertokenScale, sharedInput and logit may be null (no bias / scale 1 / no shared rows / weight 1); offset and the
 * antiquant arguments must be null.
 */
#ifndef OPS_TRANSFORMER_AMD_ACLNN_GROUPED_MATMUL_FINALIZE_ROUTING_H_
#define OPS_TRANSFORMER_AMD_ACLNN_GROUPED_MATMUL_FINALIZE_ROUTING_H_

#include "acl/acl.h"

#ifdef __cplusplus
extern "C" {
#endif

ACLNN_API aclnnStatus aclnnGroupedMatmulFinalizeRoutingGetWorkspaceSize(
    const aclTensor* x, aclTensor* w, const aclTensor* scaleOptional, const aclTensor* biasOptional,
    const aclTensor* pertokenScaleOptional, const aclTensor* groupListOptional, const aclTensor* sharedInputOptional,
    const aclTensor* logitOptional, const aclTensor* rowIndexOptional, int64_t dtype, float sharedInputWeight,
    int64_t sharedInputOffset, bool transposeX, bool transposeW, int64_t groupListType, aclTensor* y,
    uint64_t* workspaceSize, aclOpExecutor** executor);
ACLNN_API aclnnStatus aclnnGroupedMatmulFinalizeRouting(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor,
                                                        aclrtStream stream);

ACLNN_API aclnnStatus aclnnGroupedMatmulFinalizeRoutingV2GetWorkspaceSize(
    const aclTensor* x1, aclTensor* x2, const aclTensor* scaleOptional, const aclTensor* biasOptional,
    const aclTensor* offsetOptional, const aclTensor* antiquantScaleOptional, const aclTensor* antiquantOffsetOptional,
    const aclTensor* pertokenScaleOptional, const aclTensor* groupListOptional, const aclTensor* sharedInputOptional,
    const aclTensor* logitOptional, const aclTensor* rowIndexOptional, int64_t dtype, float sharedInputWeight,
    int64_t sharedInputOffset, bool transposeX1, bool transposeX2, int64_t groupListType, aclTensor* out,
    uint64_t* workspaceSize, aclOpExecutor** executor);
ACLNN_API aclnnStatus aclnnGroupedMatmulFinalizeRoutingV2(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor,
                                                          aclrtStream stream);

ACLNN_API aclnnStatus aclnnGroupedMatmulFinalizeRoutingV3GetWorkspaceSize(
    const aclTensor* x1, aclTensor* x2, const aclTensor* scaleOptional, const aclTensor* biasOptional,
    const aclTensor* offsetOptional, const aclTensor* antiquantScaleOptional, const aclTensor* antiquantOffsetOptional,
    const aclTensor* pertokenScaleOptional, const aclTensor* groupListOptional, const aclTensor* sharedInputOptional,
    const aclTensor* logitOptional, const aclTensor* rowIndexOptional, int64_t dtype, float sharedInputWeight,
    int64_t sharedInputOffset, bool transposeX1, bool transposeX2, int64_t groupListType,
    const aclIntArray* tuningConfigOptional, aclTensor* out, uint64_t* workspaceSize, aclOpExecutor** executor);
ACLNN_API aclnnStatus aclnnGroupedMatmulFinalizeRoutingV3(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor,
                                                          aclrtStream stream);

ACLNN_API aclnnStatus aclnnGroupedMatmulFinalizeRoutingWeightNzGetWorkspaceSize(
    const aclTensor* x1, const aclTensor* x2, const aclTensor* scale, const aclTensor* bias,
    const aclTensor* pertokenScaleOptional, const aclTensor* groupList, const aclTensor* sharedInput, const aclTensor* logit,
    const aclTensor* rowIndex, int64_t dtype, float sharedInputWeight, int64_t sharedInputOffset, bool transposeX1,
    bool transposeX2, int64_t groupListType, aclTensor* out, uint64_t* workspaceSize, aclOpExecutor** executor);
ACLNN_API aclnnStatus aclnnGroupedMatmulFinalizeRoutingWeightNz(void* workspace, uint64_t workspaceSize,
                                                                aclOpExecutor* executor, aclrtStream stream);

ACLNN_API aclnnStatus aclnnGroupedMatmulFinalizeRoutingWeightNzV2GetWorkspaceSize(
    const aclTensor* x1, aclTensor* x2, const aclTensor* scale, const aclTensor* bias, const aclTensor* offsetOptional,
    const aclTensor* antiquantScaleOptional, const aclTensor* antiquantOffsetOptional,
    const aclTensor* pertokenScaleOptional, const aclTensor* groupList, const aclTensor* sharedInput, const aclTensor* logit,
    const aclTensor* rowIndex, int64_t dtype, float sharedInputWeight, int64_t sharedInputOffset, bool transposeX1,
    bool transposeX2, int64_t groupListType, const aclIntArray* tuningConfigOptional, aclTensor* out,
    uint64_t* workspaceSize, aclOpExecutor** executor);
ACLNN_API aclnnStatus aclnnGroupedMatmulFinalizeRoutingWeightNzV2(void* workspace, uint64_t workspaceSize,
                                                                  aclOpExecutor* executor, aclrtStream stream);

#ifdef __cplusplus
}
#endif
#endif
