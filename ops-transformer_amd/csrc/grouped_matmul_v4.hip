// aclnnGroupedMatmulV4 for gfx950, restricted to the int8 x int8 split-M case of the MoE down projection.
//
// Argument checks follow gmm/grouped_matmul/op_host/op_api/aclnn_grouped_matmul.cpp:
//   :303-311   x / weight / out lists must be non-null (ACLNN_ERR_PARAM_NULLPTR) and non-empty
//   :1373-1386 the five reserved arguments must be null
//   :1397-1428 an empty list, a list holding nullptr, or one holding a shape-[0] tensor means "absent"
//   :339-361   groupList is a 1-D INT64 tensor of at most 1024 entries whose length equals weight.dim0
//   :556-588   perTokenScale is FLOAT [M]
//   :642-700   int8 pairing: scale BF16 -> out BF16, scale FLOAT -> out FLOAT16 (per-token), no scale -> out INT32
//   :1883-1916 groupListType 0/1/2 (2 = sparse [e, 2] list of (expert id, rows) pairs, groupType 0 only), actType range
//   op_kernel/grouped_matmul.h:288-345 how a sparse list is walked (pairs in order, stop at the first empty pair)
// Widenings of this build: scale FLOAT with out BF16 is accepted; groupList may be INT32.
// Group boundaries: grouped_matmul_utils.h:243-257.  The arithmetic is in grouped_gemm_i8.hip.
#include "aclnnop/aclnn_grouped_matmul_v5.h"
#include "aclnnop/aclnn_grouped_matmul_weight_nz.h"

#include <new>

#include "grouped_gemm_i8.h"
#include "opapi_common.h"

namespace {

class NoOpExecutor : public aclOpExecutor {
   public:
    aclnnStatus Run(void*, hipStream_t) override { return ACLNN_SUCCESS; }
};

class GroupedMatmulExecutor : public aclOpExecutor {
   public:
    gemm::Problem problem;
    gemm::Plan plan;
    aclnnStatus Run(void* workspace, hipStream_t stream) override {
        const hipError_t e = gemm::Enqueue(problem, plan, workspace, stream);
        if (e != hipSuccess) {
            opapi::SetError("aclnnGroupedMatmulV4: launch failed: %s", hipGetErrorString(e));
            return ACLNN_ERR_RUNTIME_ERROR;
        }
        return ACLNN_SUCCESS;
    }
};

// "absent" per the reference's ResetEmptyTensor convention
const aclTensor* SingleOrNull(const aclTensorList* l) {
    if (l == nullptr || l->items.empty() || l->items[0] == nullptr) return nullptr;
    if (l->items.size() == 1) {
        const aclTensor* t = l->items[0];
        if (t->dims.size() == 1 && t->dims[0] == 0) return nullptr;
    }
    return l->items[0];
}

bool Present(const aclTensorList* l) { return SingleOrNull(l) != nullptr; }

constexpr int64_t kMaxGroupListTensor = 1024;

}  // namespace

namespace {

// Shared first phase of V4 and V5.  expectedRowsPerGroup > 0 is V5's tuning hint (tuningConfig[0]): the expected number
// of rows per expert, which picks the tile height instead of the static mean M / groups.
aclnnStatus PlanGroupedMatmul(
    const aclTensorList* x, const aclTensorList* weight, const aclTensorList* biasOptional,
    const aclTensorList* scaleOptional, const aclTensorList* offsetOptional, const aclTensorList* antiquantScaleOptional,
    const aclTensorList* antiquantOffsetOptional, const aclTensorList* perTokenScaleOptional,
    const aclTensor* groupListOptional, const aclTensorList* activationInputOptional,
    const aclTensorList* activationQuantScaleOptional, const aclTensorList* activationQuantOffsetOptional,
    int64_t splitItem, int64_t groupType, int64_t groupListType, int64_t actType, int64_t expectedRowsPerGroup,
    bool forceNz, aclTensorList* out, aclTensorList* activationFeatureOutOptional,
    aclTensorList* dynQuantScaleOutOptional, uint64_t* workspaceSize, aclOpExecutor** executor) {
    using namespace opapi;
    ClearError();
    constexpr aclnnStatus kInvalid = ACLNN_ERR_PARAM_INVALID;
    OPAPI_CHECK(x != nullptr, ACLNN_ERR_PARAM_NULLPTR, "x must not be nullptr.");
    OPAPI_CHECK(!x->items.empty(), kInvalid, "x must not be empty tensorlist.");
    OPAPI_CHECK(weight != nullptr, ACLNN_ERR_PARAM_NULLPTR, "weight must not be nullptr.");
    OPAPI_CHECK(!weight->items.empty(), kInvalid, "weight must not be empty tensorlist.");
    OPAPI_CHECK(out != nullptr, ACLNN_ERR_PARAM_NULLPTR, "y must not be nullptr.");
    OPAPI_CHECK(!out->items.empty(), kInvalid, "y must not be empty tensorlist.");
    OPAPI_CHECK_NOTNULL(workspaceSize, "workspaceSize");
    OPAPI_CHECK_NOTNULL(executor, "executor");

    // common checks
    OPAPI_CHECK(groupType >= -1 && groupType <= 2, kInvalid, "groupType is invalid.");
    OPAPI_CHECK(splitItem >= 0 && splitItem <= 3, kInvalid, "splitItem is invalid.");
    OPAPI_CHECK(actType >= 0, kInvalid, "actType must be larger or equal to 0");
    if (actType != GMM_ACT_TYPE_NONE) {
        OPAPI_CHECK(actType != GMM_ACT_TYPE_GELU_ERR_FUNC, kInvalid, "Activation function not support GELU_ERR_FUNC now.");
        OPAPI_CHECK(actType < END_ACT_TYPE_ENUM, kInvalid, "Activation function only support RELU/GELU_TANH/FASTGELU/SILU.");
    }
    OPAPI_CHECK(groupListType == 0 || groupListType == 1 || groupListType == 2, kInvalid, "groupListType shoule be 0 or 1.");
    const size_t groupListRank = groupListType == 2 ? 2 : 1;
    OPAPI_CHECK(groupListOptional == nullptr || groupListOptional->dims.size() == groupListRank, kInvalid,
                "When groupList type is tensor, groupList dim only support 1 or 2(only when groupListType is 2), but now "
                "groupList dim is %zu, groupListType is %lld.",
                groupListOptional ? groupListOptional->dims.size() : size_t(0), (long long)groupListType);
    OPAPI_CHECK(!(groupListType == 2 && groupListOptional != nullptr && groupListOptional->dims[1] != 2), kInvalid,
                "With groupListType 2 groupList must be [e, 2] pairs of (expert id, rows), got %s",
                groupListOptional ? ShapeStr(groupListOptional).c_str() : "");
    OPAPI_CHECK(!(groupListType == 2 && groupType != 0), kInvalid,
                "When groupListType is 2 only support groupType 0, but get groupType %lld.", (long long)groupType);

    // reserved arguments
    OPAPI_CHECK(!Present(activationInputOptional), kInvalid, "activationInputOptional must be nullptr.");
    OPAPI_CHECK(!Present(activationQuantScaleOptional), kInvalid, "activationQuantScaleOptional must be nullptr.");
    OPAPI_CHECK(!Present(activationQuantOffsetOptional), kInvalid, "activationQuantOffsetOptional must be nullptr.");
    OPAPI_CHECK(!Present(activationFeatureOutOptional), kInvalid, "activationFeatureOutOptional must be nullptr.");
    OPAPI_CHECK(!Present(dynQuantScaleOutOptional), kInvalid, "dynQuantScaleOutOptional must be nullptr.");

    // the one layout built here: single x, single weight, single y, rows split by groupList
    OPAPI_CHECK(x->items.size() == 1 && weight->items.size() == 1 && out->items.size() == 1, kInvalid,
                "only single-tensor x / weight / y lists are supported (got %zu, %zu, %zu)", x->items.size(),
                weight->items.size(), out->items.size());
    OPAPI_CHECK(groupType == 0, kInvalid, "only groupType 0 (split along M) is supported, got %lld", (long long)groupType);
    OPAPI_CHECK(splitItem == 2 || splitItem == 3, kInvalid,
                "single-tensor y requires splitItem 2 or 3, got %lld", (long long)splitItem);
    const aclTensor* xt = x->items[0];
    const aclTensor* wt = weight->items[0];
    const aclTensor* yt = out->items[0];
    OPAPI_CHECK(xt != nullptr, kInvalid, "x[0] is nullptr!");
    OPAPI_CHECK(wt != nullptr, kInvalid, "weight[0] is nullptr!");
    OPAPI_CHECK(yt != nullptr, kInvalid, "y[0] is nullptr!");
    OPAPI_CHECK_EXTENTS(xt, wt, yt, groupListOptional);
    OPAPI_CHECK(xt->dtype == ACL_INT8 && wt->dtype == ACL_INT8, kInvalid,
                "only INT8 x and INT8 weight are built (got %d, %d)", (int)xt->dtype, (int)wt->dtype);
    // A blocked (FRACTAL_NZ) int8 weight is [E, N/32, K/16, 16, 32], given as that 5-D tensor or as the 3-D view
    // [E, K, N] over storage of that shape (the layout aclnn_grouped_matmul_swiglu_quant.cpp:163-168 spells out).
    const bool nz = forceNz || wt->format == ACL_FORMAT_FRACTAL_NZ;
    OPAPI_CHECK(nz || wt->format == ACL_FORMAT_ND, kInvalid, "weight must be ND or FRACTAL_NZ");
    const std::vector<int64_t>& blocked = wt->dims.size() == 5 ? wt->dims : wt->storage;
    if (nz) {
        OPAPI_CHECK((wt->dims.size() == 5 || wt->dims.size() == 3) && blocked.size() == 5 && blocked[3] == 16 && blocked[4] == 32,
                    kInvalid, "a FRACTAL_NZ weight needs the storage shape [E, N/32, K/16, 16, 32], got view %s",
                    ShapeStr(wt).c_str());
    }
    OPAPI_CHECK(actType == GMM_ACT_TYPE_NONE, kInvalid, "actType %lld is not built for the INT8 path", (long long)actType);
    OPAPI_CHECK(!Present(biasOptional), kInvalid, "bias is not supported on the INT8 per-token path of this build");
    OPAPI_CHECK(!Present(offsetOptional), kInvalid, "offset must be null in the quant case");
    OPAPI_CHECK(!Present(antiquantScaleOptional) && !Present(antiquantOffsetOptional), kInvalid,
                "antiquant parameters must be null in the quant case");

    OPAPI_CHECK(xt->dims.size() == 2, kInvalid, "x must be 2-D [M,K], got %s", ShapeStr(xt).c_str());
    OPAPI_CHECK(nz || wt->dims.size() == 3, kInvalid, "weight must be 3-D [E,K,N], got %s", ShapeStr(wt).c_str());
    OPAPI_CHECK(yt->dims.size() == 2, kInvalid, "y must be 2-D [M,N], got %s", ShapeStr(yt).c_str());
    const int64_t m = xt->dims[0], k = xt->dims[1], e = wt->dims[0];
    const int64_t n = wt->dims.size() == 5 ? wt->dims[1] * 32 : wt->dims[2];
    const int64_t wk = wt->dims.size() == 5 ? wt->dims[2] * 16 : wt->dims[1];
    OPAPI_CHECK(wk == k, kInvalid, "weight %s does not match x %s along K", ShapeStr(wt).c_str(), ShapeStr(xt).c_str());
    OPAPI_CHECK(!nz || (blocked[0] == e && blocked[1] * 32 == n && blocked[2] * 16 == k && wt->offset == 0), kInvalid,
                "the blocked weight storage must be [%lld, %lld, %lld, 16, 32] (N a multiple of 32, K of 16)", (long long)e,
                (long long)(n / 32), (long long)(k / 16));
    OPAPI_CHECK(yt->dims[0] == m && yt->dims[1] == n, kInvalid, "y must be [%lld,%lld], got %s", (long long)m, (long long)n,
                ShapeStr(yt).c_str());
    OPAPI_CHECK(k < 65536, kInvalid, "K must be lower than 65536");
    OPAPI_CHECK(m < (1ll << 31) && n < (1ll << 31), kInvalid, "M and N must fit int32");

    // group list
    OPAPI_CHECK(groupListOptional != nullptr && groupListOptional->dims[0] > 0, kInvalid,
                "groupListOptional(tensor) is required in this case, but get nullptr.");
    const int64_t groupListLen = groupListOptional->dims[0];
    OPAPI_CHECK(groupListLen <= kMaxGroupListTensor, kInvalid,
                "When groupList type is tenosr, size of groupList %lld should be less than or equal to %lld.",
                (long long)groupListLen, (long long)kMaxGroupListTensor);
    OPAPI_CHECK(groupListLen == e, kInvalid,
                "When groupList is not null, size of groupList(tensor) %lld should be equal to weight dim 0 %lld with groupType 0.",
                (long long)groupListLen, (long long)e);
    OPAPI_CHECK(groupListOptional->dtype == ACL_INT64 || groupListOptional->dtype == ACL_INT32, kInvalid,
                "Invalid dtype: Only int64 (or int32) is supported for groupList.");

    // quant parameter pairing
    const aclTensor* scale = SingleOrNull(scaleOptional);
    const aclTensor* perToken = SingleOrNull(perTokenScaleOptional);
    if (scale == nullptr) {
        OPAPI_CHECK(yt->dtype == ACL_INT32, kInvalid, "without scale the output of the INT8 case must be INT32");
        OPAPI_CHECK(perToken == nullptr, kInvalid, "perTokenScale needs scale");
    } else {
        OPAPI_CHECK(scale->dims.size() == 2 && scale->dims[0] == e && scale->dims[1] == n, kInvalid,
                    "scale must be [%lld,%lld], got %s", (long long)e, (long long)n, ShapeStr(scale).c_str());
        const bool pairOk = (scale->dtype == ACL_BF16 && yt->dtype == ACL_BF16) ||
                            (scale->dtype == ACL_FLOAT && (yt->dtype == ACL_FLOAT16 || yt->dtype == ACL_BF16));
        OPAPI_CHECK(pairOk, kInvalid, "unsupported scale/output dtype pair (%d, %d): BF16->BF16, FLOAT->FLOAT16, FLOAT->BF16",
                    (int)scale->dtype, (int)yt->dtype);
        if (perToken != nullptr) {
            OPAPI_CHECK(perToken->dtype == ACL_FLOAT, kInvalid, "perTokenScale must be FLOAT");
            OPAPI_CHECK(perToken->dims.size() == 1 && perToken->dims[0] == m, kInvalid, "perTokenScale must be [%lld], got %s",
                        (long long)m, ShapeStr(perToken).c_str());
        }
    }

    if (m == 0 || n == 0) {  // nothing to compute
        auto* noop = new (std::nothrow) NoOpExecutor();
        OPAPI_CHECK(noop != nullptr, ACLNN_ERR_INNER_CREATE_EXECUTOR, "out of host memory");
        *workspaceSize = 0;
        *executor = noop;
        return ACLNN_SUCCESS;
    }
    OPAPI_CHECK(k > 0, kInvalid, "K must be positive");

    const bool wTransposed = !nz && IsLastTwoDimsTransposed(wt);
    OPAPI_CHECK(nz || wTransposed || IsContiguous(wt), kInvalid,
                "weight must be contiguous [E,K,N] or the transposed view of contiguous [E,N,K] storage");
    OPAPI_CHECK(IsContiguous(yt), kInvalid, "y must be contiguous");  // the other tensors may be strided views
    const aclTensor* all[] = {xt, wt, yt, groupListOptional, scale, perToken};
    for (const aclTensor* t : all) {
        OPAPI_CHECK(t == nullptr || t->data != nullptr, ACLNN_ERR_PARAM_NULLPTR, "a tensor carries no device memory");
    }

    auto* ex = new (std::nothrow) GroupedMatmulExecutor();
    OPAPI_CHECK(ex != nullptr, ACLNN_ERR_INNER_CREATE_EXECUTOR, "out of host memory");
    gemm::Problem& p = ex->problem;
    OPAPI_BIND(ex, xt, &p.x);
    p.w = reinterpret_cast<const int8_t*>(DataPtr(wt));
    p.wKMajor = wTransposed;
    p.wNz = nz;
    p.M = m;
    p.K = k;
    p.N = n;
    p.groups = static_cast<int32_t>(groupListLen);
    OPAPI_BIND(ex, groupListOptional, &p.groupList);
    p.groupListIsInt64 = groupListOptional->dtype == ACL_INT64;
    p.groupListKind = groupListType == 2 ? gemm::GroupListKind::kSparse
                      : groupListType == 1 ? gemm::GroupListKind::kCount : gemm::GroupListKind::kCumsum;
    p.out = DataPtr(yt);
    p.outDtype = static_cast<int>(yt->dtype);
    if (scale == nullptr) {
        p.epilogue = gemm::Epilogue::kInt32;
    } else {
        p.epilogue = gemm::Epilogue::kDequant;
        OPAPI_BIND(ex, scale, &p.scale);
        p.scaleDtype = static_cast<int>(scale->dtype);
        OPAPI_BIND(ex, perToken, &p.rowScale);
    }
    p.expectedRowsPerGroup = expectedRowsPerGroup;
    ex->plan = gemm::MakePlan(p);
    ex->SealWorkspace(ex->plan.workspaceBytes);
    *workspaceSize = ex->workspaceBytes;
    *executor = ex;
    return ACLNN_SUCCESS;
}

}  // namespace

extern "C" aclnnStatus aclnnGroupedMatmulV4GetWorkspaceSize(
    const aclTensorList* x, const aclTensorList* weight, const aclTensorList* biasOptional,
    const aclTensorList* scaleOptional, const aclTensorList* offsetOptional, const aclTensorList* antiquantScaleOptional,
    const aclTensorList* antiquantOffsetOptional, const aclTensorList* perTokenScaleOptional,
    const aclTensor* groupListOptional, const aclTensorList* activationInputOptional,
    const aclTensorList* activationQuantScaleOptional, const aclTensorList* activationQuantOffsetOptional,
    int64_t splitItem, int64_t groupType, int64_t groupListType, int64_t actType, aclTensorList* out,
    aclTensorList* activationFeatureOutOptional, aclTensorList* dynQuantScaleOutOptional, uint64_t* workspaceSize,
    aclOpExecutor** executor) {
    return PlanGroupedMatmul(x, weight, biasOptional, scaleOptional, offsetOptional, antiquantScaleOptional,
                             antiquantOffsetOptional, perTokenScaleOptional, groupListOptional, activationInputOptional,
                             activationQuantScaleOptional, activationQuantOffsetOptional, splitItem, groupType,
                             groupListType, actType, /*expectedRowsPerGroup=*/0, /*forceNz=*/false, out, activationFeatureOutOptional,
                             dynQuantScaleOutOptional, workspaceSize, executor);
}

// V5 = V4 plus tuningConfigOptional, whose first value is the expected number of tokens per expert
// (reference: aclnn_grouped_matmul.cpp:1957-1992; it only steers tiling, never results).
extern "C" aclnnStatus aclnnGroupedMatmulV5GetWorkspaceSize(
    const aclTensorList* x, const aclTensorList* weight, const aclTensorList* biasOptional,
    const aclTensorList* scaleOptional, const aclTensorList* offsetOptional, const aclTensorList* antiquantScaleOptional,
    const aclTensorList* antiquantOffsetOptional, const aclTensorList* perTokenScaleOptional,
    const aclTensor* groupListOptional, const aclTensorList* activationInputOptional,
    const aclTensorList* activationQuantScaleOptional, const aclTensorList* activationQuantOffsetOptional,
    int64_t splitItem, int64_t groupType, int64_t groupListType, int64_t actType, aclIntArray* tuningConfigOptional,
    aclTensorList* out, aclTensorList* activationFeatureOutOptional, aclTensorList* dynQuantScaleOutOptional,
    uint64_t* workspaceSize, aclOpExecutor** executor) {
    int64_t expected = 0;
    if (tuningConfigOptional != nullptr && !tuningConfigOptional->values.empty() &&
        tuningConfigOptional->values[0] > 0) {
        expected = tuningConfigOptional->values[0];
    }
    return PlanGroupedMatmul(x, weight, biasOptional, scaleOptional, offsetOptional, antiquantScaleOptional,
                             antiquantOffsetOptional, perTokenScaleOptional, groupListOptional, activationInputOptional,
                             activationQuantScaleOptional, activationQuantOffsetOptional, splitItem, groupType,
                             groupListType, actType, expected, /*forceNz=*/false, out, activationFeatureOutOptional,
                             dynQuantScaleOutOptional, workspaceSize, executor);
}

extern "C" aclnnStatus aclnnGroupedMatmulV5(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor,
                                            aclrtStream stream) {
    return opapi::RunAndRelease(workspace, workspaceSize, executor, stream);
}

extern "C" aclnnStatus aclnnGroupedMatmulV4(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor,
                                            aclrtStream stream) {
    return opapi::RunAndRelease(workspace, workspaceSize, executor, stream);
}

// V5 for a weight whose storage is the blocked FRACTAL_NZ layout, plus quantGroupSize (per-group quantisation: must be 0
// here) -- reference: aclnn_grouped_matmul.cpp:1918-1956.
extern "C" aclnnStatus aclnnGroupedMatmulWeightNzGetWorkspaceSize(
    const aclTensorList* x, const aclTensorList* weight, const aclTensorList* biasOptional,
    const aclTensorList* scaleOptional, const aclTensorList* offsetOptional, const aclTensorList* antiquantScaleOptional,
    const aclTensorList* antiquantOffsetOptional, const aclTensorList* perTokenScaleOptional,
    const aclTensor* groupListOptional, const aclTensorList* activationInputOptional,
    const aclTensorList* activationQuantScaleOptional, const aclTensorList* activationQuantOffsetOptional,
    int64_t splitItem, int64_t groupType, int64_t groupListType, int64_t actType, aclIntArray* tuningConfigOptional,
    int64_t quantGroupSize, aclTensorList* out, aclTensorList* activationFeatureOutOptional,
    aclTensorList* dynQuantScaleOutOptional, uint64_t* workspaceSize, aclOpExecutor** executor) {
    if (quantGroupSize != 0) {
        opapi::ClearError();
        opapi::SetError("aclnnGroupedMatmulWeightNz: per-group quantisation (quantGroupSize %lld) is not built; pass 0",
                        (long long)quantGroupSize);
        return ACLNN_ERR_PARAM_INVALID;
    }
    int64_t expected = 0;
    if (tuningConfigOptional != nullptr && !tuningConfigOptional->values.empty() &&
        tuningConfigOptional->values[0] > 0) {
        expected = tuningConfigOptional->values[0];
    }
    return PlanGroupedMatmul(x, weight, biasOptional, scaleOptional, offsetOptional, antiquantScaleOptional,
                             antiquantOffsetOptional, perTokenScaleOptional, groupListOptional, activationInputOptional,
                             activationQuantScaleOptional, activationQuantOffsetOptional, splitItem, groupType,
                             groupListType, actType, expected, /*forceNz=*/true, out, activationFeatureOutOptional,
                             dynQuantScaleOutOptional, workspaceSize, executor);
}

extern "C" aclnnStatus aclnnGroupedMatmulWeightNz(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor,
                                                  aclrtStream stream) {
    return opapi::RunAndRelease(workspace, workspaceSize, executor, stream);
}
