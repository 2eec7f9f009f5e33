/*
 * aclnnMoeInitRoutingQuantV2 — MI355X build.
 * Replaces the aclnn interface generated from moe/moe_init_routing_quant_v2/op_host/moe_init_routing_quant_v2_def.cpp
 * (call shape: moe/moe_init_routing_quant_v2/examples/test_aclnn_moe_init_routing_quant_v2.cpp:131; semantics:
 * moe/moe_init_routing_quant_v2/README.md).
 *
 * aclnnMoeInitRoutingV2 (same routing, same modes, see aclnn_moe_init_routing_v2.h) whose gathered rows are quantised to
 * INT8 on the way:
 *   quantMode 0 (static):  scaleOptional and offsetOptional are FLOAT [1]; y = int8(rint(half(half(x) * half(scale))
 *                          + half(offset))) in half arithmetic (op_kernel/moe_v2_gather_quant.h:93-133), saturated
 *   quantMode 1 (dynamic): scaleOptional is an optional smooth scale, FLOAT [1, H] or [expertNum, H]; per routed row
 *                          s = max|x * smooth| / 127 goes to dynamicQuantScaleOutOptional (FLOAT [rows of expandedXOut],
 *                          required) and y = int8(round_half_away(half_toward_zero((x * smooth) / s)))
 *                          (op_kernel/moe_v2_gather_dynamic_quant.h:120-155)
 * x FLOAT / FLOAT16 / BF16, expandedXOut INT8.  In drop/pad mode the unused capacity rows are zero and their scale 0.
 */
#ifndef OPS_TRANSFORMER_AMD_ACLNN_MOE_INIT_ROUTING_QUANT_V2_H_
#define OPS_TRANSFORMER_AMD_ACLNN_MOE_INIT_ROUTING_QUANT_V2_H_

#include "acl/acl.h"

#ifdef __cplusplus
extern "C" {
#endif

ACLNN_API aclnnStatus aclnnMoeInitRoutingQuantV2GetWorkspaceSize(
    const aclTensor* x, const aclTensor* expertIdx, const aclTensor* scaleOptional, const aclTensor* offsetOptional,
    int64_t activeNum, int64_t expertCapacity, int64_t expertNum, int64_t dropPadMode,
    int64_t expertTokensCountOrCumsumFlag, bool expertTokensBeforeCapacityFlag, int64_t quantMode,
    const aclTensor* expandedXOut, const aclTensor* expandedRowIdxOut, const aclTensor* expertTokensCountOrCumsumOutOptional,
    const aclTensor* expertTokensBeforeCapacityOutOptional, const aclTensor* dynamicQuantScaleOutOptional,
    uint64_t* workspaceSize, aclOpExecutor** executor);

ACLNN_API aclnnStatus aclnnMoeInitRoutingQuantV2(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor,
                                                 aclrtStream stream);

#ifdef __cplusplus
}
#endif
#endif
