/*
 * aclnnMoeInitRoutingV3 for MI355X.
 *
 * Replaces moe/moe_init_routing_v3/op_host/op_api/aclnn_moe_init_routing_v3.h:25-47 of the reference (same symbol
 * names, argument order and meaning; semantics from moe/moe_init_routing_v3/README.md:12-66 and
 * op_host/moe_init_routing_v3_tiling.cpp:233-352).  Compared with V2: INT8 rows are a first-class input, an optional
 * per-token scale [T] is gathered into expandedScaleOut [T*K] alongside the rows (quantMode -1,
 * op_kernel/moe_v3_gather_out.h:213-221), only experts inside activeExpertRangeOptional = [start, end) are routed
 * (the other rows are dropped: -1 in the index output), the token counts are INT64 and can be counts (type 1) or
 * key/value pairs (type 2, op_kernel/moe_v3_expert_tokens_count.h:254-269), and the index output is either the
 * scatter-type map of V2 (rowIdxType 1: [source] -> destination) or the gather-type map (0: [destination] -> source).
 *
 * quantMode 1 (dynamic quantisation, op_kernel/moe_v3_gather_dynamic_quant.h:103-141): x is FLOAT/FLOAT16/BF16,
 * scaleOptional is the optional smooth scale [end - start, H] multiplied into the row of the expert it is routed to,
 * expandedXOut is INT8 with per-row scale max|v| / 127 in expandedScaleOut (always written): v / scale by true division,
 * narrowed to half precision toward zero, then to INT8 with halves away from zero.  A row of zeros gives scale 0 and
 * zeros (the reference divides 0 by 0 there).
 *
 * This build: at most 2047 active experts when the range is a proper sub-range, 2048 otherwise; expertTokensNumType 0
 * (cumsum) is accepted as an extension (the reference's tiling rejects it although the operator definition lists it),
 * because aclnnGroupedMatmulSwigluQuant takes a cumsum group list; offsetOptional is accepted and ignored, as in the
 * reference.
 */
#ifndef OPS_TRANSFORMER_AMD_ACLNN_MOE_INIT_ROUTING_V3_H_
#define OPS_TRANSFORMER_AMD_ACLNN_MOE_INIT_ROUTING_V3_H_

#include "acl/acl.h"

#ifdef __cplusplus
extern "C" {
#endif

ACLNN_API aclnnStatus aclnnMoeInitRoutingV3GetWorkspaceSize(
    const aclTensor* x, const aclTensor* expertIdx, const aclTensor* scaleOptional, const aclTensor* offsetOptional,
    int64_t activeNum, int64_t expertCapacity, int64_t expertNum, int64_t dropPadMode, int64_t expertTokensNumType,
    bool expertTokensNumFlag, int64_t quantMode, const aclIntArray* activeExpertRangeOptional, int64_t rowIdxType,
    const aclTensor* expandedXOut, const aclTensor* expandedRowIdxOut, const aclTensor* expertTokensCountOrCumsumOut,
    const aclTensor* expandedScaleOut, uint64_t* workspaceSize, aclOpExecutor** executor);

ACLNN_API aclnnStatus aclnnMoeInitRoutingV3(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor,
                                            aclrtStream stream);

#ifdef __cplusplus
}
#endif
#endif
