/*
 * aclnnMoeInitRoutingV2 — MI355X build.
 * Replaces: moe/moe_init_routing_v2/op_host/op_api/aclnn_moe_init_routing_v2.h:42-56 (same symbols, same argument order).
 *
 * Expands T tokens top-K ways (flat index i = n*K + j over expertIdx[T,K], row-major), sorts the M = T*K flat entries by
 * expert id with a stable ascending sort, and returns
 *   expandedRowIdxOut[i]  = destination row of flat entry i (dropless) / e*C + rank or -1 (drop/pad),
 *   expandedXOut[dst, :]  = x[i / K, :],
 *   expertTokensCountOrCumsumOut[e] = per-expert count (flag 2) or inclusive cumsum (flag 1), int32.
 * x dtype: FLOAT, FLOAT16, BF16 as in the reference (moe_init_routing_v2_def.cpp:22-38); INT8 is accepted as an extension so
 * that already-quantized activations can be routed (a row gather is dtype-agnostic).
 */
#ifndef OPS_TRANSFORMER_AMD_ACLNN_MOE_INIT_ROUTING_V2_H_
#define OPS_TRANSFORMER_AMD_ACLNN_MOE_INIT_ROUTING_V2_H_

#include "acl/acl.h"

#ifdef __cplusplus
extern "C" {
#endif

ACLNN_API aclnnStatus aclnnMoeInitRoutingV2GetWorkspaceSize(
    const aclTensor* x, const aclTensor* expertIdx, int64_t activeNumOptional, int64_t expertCapacityOptional,
    int64_t expertNumOptional, int64_t dropPadModeOptional, int64_t expertTokensCountOrCumsumFlagOptional,
    bool expertTokensBeforeCapacityFlagOptional, const aclTensor* expandedXOut, const aclTensor* expandedRowIdxOut,
    const aclTensor* expertTokensCountOrCumsumOutOptional, const aclTensor* expertTokensBeforeCapacityOutOptional,
    uint64_t* workspaceSize, aclOpExecutor** executor);

ACLNN_API aclnnStatus aclnnMoeInitRoutingV2(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor,
                                            aclrtStream stream);

/*
 * aclnnMoeInitRoutingV2StaticWorkspace -- no counterpart in the reference.  For callers that cannot allocate device
 * memory (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc): the second phase of
 * aclnnMoeInitRoutingV2 without a workspace argument.  The sort tables live in a 4 MiB device array inside the library
 * (one copy per GPU, held until the process ends), which covers up to about 130000 expanded rows (tokens x top-k) per call with expertNum <= 2048.
 * Takes an executor made by aclnnMoeInitRoutingV2GetWorkspaceSize and consumes it like the ordinary second phase; a call
 * whose first phase asked for more than 4 MiB is refused with ACLNN_ERR_PARAM_INVALID (the executor is released).  Calls
 * no hipMalloc / hipFree.  All calls on one GPU share the array: calls that overlap on one GPU (two streams, two threads)
 * race -- serialise them.  The first call on a device looks the array's address up (hipGetSymbolAddress), so make one
 * call before starting a graph capture.
 */
ACLNN_API aclnnStatus aclnnMoeInitRoutingV2StaticWorkspace(aclOpExecutor* executor, aclrtStream stream);

#ifdef __cplusplus
}
#endif
#endif
