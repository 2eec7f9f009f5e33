/*
 * aclnnMoeFinalizeRoutingV2 — MI355X build.
 * Replaces: moe/moe_finalize_routing_v2/op_host/op_api/aclnn_moe_finalize_routing_v2.h:26-35.
 *
 *   out[n,:] = x1[n,:] + x2[n,:] + sum_{k<K} scales[n,k] * (expandedX[idx(n,k),:] + bias[expertIdx[n,k],:])
 * accumulated in fp32 in ascending k and rounded to the dtype of expandedX (nearest even).
 * idx(n,k) = expandedRowIdx[k*T + n] for dropPadMode 0/1 (column arrangement) and expandedRowIdx[n*K + k] for 2/3 (row
 * arrangement, what aclnnMoeInitRoutingV2 emits); in modes 1/3 an index of -1 contributes nothing.
 * expandedX/x1/x2/bias/out: FLOAT, FLOAT16 or BF16 (all equal); scales: same dtype, or FLOAT with BF16 data.
 */
#ifndef OPS_TRANSFORMER_AMD_ACLNN_MOE_FINALIZE_ROUTING_V2_H_
#define OPS_TRANSFORMER_AMD_ACLNN_MOE_FINALIZE_ROUTING_V2_H_

#include "acl/acl.h"

#ifdef __cplusplus
extern "C" {
#endif

ACLNN_API aclnnStatus aclnnMoeFinalizeRoutingV2GetWorkspaceSize(
    const aclTensor* expandedX, const aclTensor* expandedRowIdx, const aclTensor* x1Optional,
    const aclTensor* x2Optional, const aclTensor* biasOptional, const aclTensor* scalesOptional,
    const aclTensor* expertIdxOptional, int64_t dropPadMode, const aclTensor* out, uint64_t* workspaceSize,
    aclOpExecutor** executor);

ACLNN_API aclnnStatus aclnnMoeFinalizeRoutingV2(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor,
                                                aclrtStream stream);

#ifdef __cplusplus
}
#endif
#endif
