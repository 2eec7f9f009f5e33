/*
 * aclnnMoeGatingTopKSoftmaxV2 — MI355X build.
 * Replaces the aclnn interface generated from moe/moe_gating_top_k_softmax_v2/op_host/moe_gating_top_k_softmax_v2_def.cpp
 * (call shape: moe/moe_gating_top_k_softmax_v2/examples/test_aclnn_moe_gating_top_k_softmax_v2.cpp:115;
 * semantics: moe/moe_gating_top_k_softmax_v2/README.md:12-30).
 *
 *   renorm 0:  p = softmax(x, axis -1) in fp32;  yOut, expertIdxOut = top-k of p (descending, equal values by ascending
 *              index);  softmaxResultOutOptional = p (FLOAT) when outputSoftmaxResultFlag is set
 *   renorm 1:  v, expertIdxOut = top-k of x;  yOut = softmax(v, axis -1)
 * Rows whose finishedOptional entry is true get expertIdxOut = x.shape[-1] in every slot (the values are still written).
 * x, yOut: FLOAT, FLOAT16 or BF16 (equal), rank 2 or 3; expertIdxOut INT32; finishedOptional BOOL of x's shape without
 * the last axis; 0 < k <= min(x.shape[-1], 1024).  This build: x.shape[-1] <= 32768.
 */
#ifndef OPS_TRANSFORMER_AMD_ACLNN_MOE_GATING_TOP_K_SOFTMAX_V2_H_
#define OPS_TRANSFORMER_AMD_ACLNN_MOE_GATING_TOP_K_SOFTMAX_V2_H_

#include "acl/acl.h"

#ifdef __cplusplus
extern "C" {
#endif

ACLNN_API aclnnStatus aclnnMoeGatingTopKSoftmaxV2GetWorkspaceSize(
    const aclTensor* x, const aclTensor* finishedOptional, int64_t k, int64_t renorm, bool outputSoftmaxResultFlag,
    const aclTensor* yOut, const aclTensor* expertIdxOut, const aclTensor* softmaxResultOutOptional,
    uint64_t* workspaceSize, aclOpExecutor** executor);

ACLNN_API aclnnStatus aclnnMoeGatingTopKSoftmaxV2(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor,
                                                  aclrtStream stream);

#ifdef __cplusplus
}
#endif
#endif
