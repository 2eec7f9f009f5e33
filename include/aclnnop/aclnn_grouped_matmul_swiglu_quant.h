/*
 * aclnnGroupedMatmulSwigluQuant — MI355X build (A8W8 path).
 * Replaces: gmm/grouped_matmul_swiglu_quant/op_host/op_api/aclnn_grouped_matmul_swiglu_quant.h:37-52.
 *
 * For group e with rows [g[e-1], g[e]) (g = groupList, cumulative, g[-1] = 0):
 *   acc = int32(x[rows,:]) @ int32(weight[e])                       x int8 [M,K], weight int8 [E,K,N]
 *   C   = (float(acc) * xScale[row]) * float(weightScale[e,col])    weightScale [E,N] fp32/fp16/bf16, xScale [M] fp32
 *   S   = swish(C[:, :N/2]) * C[:, N/2:]
 *   outputScale[row] = max|S[row,:]| / 127 ;  output[row,:] = int8(rint(fp16(S * (1/outputScale[row]))))
 * Rows at or beyond g[E-1] are left untouched.  bias, offset and outputOffset are accepted and ignored, as in the reference.
 *
 * Differences from the reference, all widening: N above 10240 is accepted; groupList may be INT32 as well as INT64 so
 * that routing's int32 cumsum can be passed without a cast; and the weight may come in any of three layouts, all served
 * by the same LDS-DMA kernel when K is a multiple of 128:
 *   - the view [E,K,N] over K-contiguous storage [E,N,K] (strides (N*K, 1, K)): what the kernels stream fastest;
 *   - contiguous row-major ND [E,K,N] (the reference's plain layout; N/2 a multiple of 16);
 *   - ACL_FORMAT_FRACTAL_NZ, 5-D [E, N/32, K/16, 16, 32] or a 3-D view [E,K,N] whose storage shape is that (the only
 *     layout the reference's A8W8 path takes).  aclnnGroupedMatmulSwigluQuantWeightNZ
 *     (aclnn_grouped_matmul_swiglu_quant_weight_nz.h) is the same operator with the storage treated as blocked whatever
 *     the format field says.
 * Shapes off these grids (K not a multiple of 128, odd channel counts) run on a byte-wise kernel: correct, slow.
 */
#ifndef OPS_TRANSFORMER_AMD_ACLNN_GROUPED_MATMUL_SWIGLU_QUANT_H_
#define OPS_TRANSFORMER_AMD_ACLNN_GROUPED_MATMUL_SWIGLU_QUANT_H_

#include "acl/acl.h"

#ifdef __cplusplus
extern "C" {
#endif

ACLNN_API aclnnStatus aclnnGroupedMatmulSwigluQuantGetWorkspaceSize(
    const aclTensor* x, const aclTensor* weight, const aclTensor* bias, const aclTensor* offset,
    const aclTensor* weightScale, const aclTensor* xScale, const aclTensor* groupList, aclTensor* output,
    aclTensor* outputScale, aclTensor* outputOffset, uint64_t* workspaceSize, aclOpExecutor** executor);

ACLNN_API aclnnStatus aclnnGroupedMatmulSwigluQuant(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor,
                                                    aclrtStream stream);

#ifdef __cplusplus
}
#endif
#endif
