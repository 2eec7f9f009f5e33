/*
 * aclnnGroupedMatmulSwigluQuantWeightNZ — MI355X build.
 * Replaces gmm/grouped_matmul_swiglu_quant/op_host/op_api/aclnn_grouped_matmul_swiglu_quant_weight_nz.h:37-54.
 *
 * aclnnGroupedMatmulSwigluQuant for a weight whose storage is the blocked FRACTAL_NZ layout [E, N/32, K/16, 16, 32]
 * (element (k, n) of expert e at ((n/32) * (K/16) + k/16) * 512 + (k%16) * 32 + n%32), whatever the format field of the
 * descriptor says: the storage shape must be that 5-D shape, the view shape either the same or [E, K, N].  Everything
 * else is as in aclnn_grouped_matmul_swiglu_quant.h.  The blocked layout is streamed as it lies (a 32-channel block is
 * one contiguous K x 32-byte run) and transposed on the way out of LDS; no repacked copy is made.
 */
#ifndef OPS_TRANSFORMER_AMD_ACLNN_GROUPED_MATMUL_SWIGLU_QUANT_WEIGHT_NZ_H_
#define OPS_TRANSFORMER_AMD_ACLNN_GROUPED_MATMUL_SWIGLU_QUANT_WEIGHT_NZ_H_

#include "acl/acl.h"

#ifdef __cplusplus
extern "C" {
#endif

ACLNN_API aclnnStatus aclnnGroupedMatmulSwigluQuantWeightNZGetWorkspaceSize(
    const aclTensor* x, const aclTensor* weight, const aclTensor* bias, const aclTensor* offset,
    const aclTensor* weightScale, const aclTensor* xScale, const aclTensor* groupList, aclTensor* output,
    aclTensor* outputScale, aclTensor* outputOffset, uint64_t* workspaceSize, aclOpExecutor** executor);

ACLNN_API aclnnStatus aclnnGroupedMatmulSwigluQuantWeightNZ(void* workspace, uint64_t workspaceSize,
                                                            aclOpExecutor* executor, aclrtStream stream);

#ifdef __cplusplus
}
#endif
#endif
