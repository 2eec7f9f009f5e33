// aclnnGroupedMatmulSwigluQuant (A8W8) for gfx950.
//
// Argument checks follow gmm/grouped_matmul_swiglu_quant/op_host/op_api/aclnn_grouped_matmul_swiglu_quant.cpp:75-350,
// 365-409 (required tensors, ranks, shapes, dtypes, groupList length <= E, K < 65536, N even) and :425-429 (an empty
// output / groupList / outputScale succeeds with no work).  The N <= 10240 ceiling and the FRACTAL_NZ-only weight rule
// of the reference are not carried over: ND weights are taken as well.  A FRACTAL_NZ weight is the 5-D tensor
// [E, N/32, K/16, 16, 32] (:163-181), or through aclnnGroupedMatmulSwigluQuantWeightNZ any tensor whose storage shape
// is that (:483-516).  The arithmetic is in grouped_gemm_i8.hip (kSwiglu epilogue + requantisation).
//
// All state lives in the executor; the reference's two sticky file-scope switches
// (aclnn_grouped_matmul_swiglu_quant.cpp:61-62) have no counterpart here.
#include "aclnnop/aclnn_grouped_matmul_swiglu_quant.h"
#include "aclnnop/aclnn_grouped_matmul_swiglu_quant_weight_nz.h"

#include <new>

#include "grouped_gemm_i8.h"
#include "opapi_common.h"

namespace {

class NoOpExecutor : public aclOpExecutor {
   public:
    aclnnStatus Run(void*, hipStream_t) override { return ACLNN_SUCCESS; }
};

class SwigluQuantExecutor : public aclOpExecutor {
   public:
    gemm::Problem problem;
    gemm::Plan plan;
    aclnnStatus Run(void* workspace, hipStream_t stream) override {
        const hipError_t e = gemm::Enqueue(problem, plan, workspace, stream);
        if (e != hipSuccess) {
            opapi::SetError("aclnnGroupedMatmulSwigluQuant: launch failed: %s", hipGetErrorString(e));
            return ACLNN_ERR_RUNTIME_ERROR;
        }
        return ACLNN_SUCCESS;
    }
};

constexpr int64_t kKLimit = 65536;

// forceNz: the WeightNZ entry point, where the storage is blocked whatever the descriptor's format field says.
aclnnStatus PlanSwigluQuant(const aclTensor* x, const aclTensor* weight, const aclTensor* bias, const aclTensor* offset,
                            const aclTensor* weightScale, const aclTensor* xScale, const aclTensor* groupList,
                            aclTensor* output, aclTensor* outputScale, aclTensor* outputOffset, bool forceNz,
                            uint64_t* workspaceSize, aclOpExecutor** executor) {
    using namespace opapi;
    ClearError();
    (void)bias;          // accepted and ignored, as in the reference's A8W8 path (only a warning there)
    (void)offset;
    (void)outputOffset;
    OPAPI_CHECK_NOTNULL(x, "x");
    OPAPI_CHECK_NOTNULL(weight, "weight");
    OPAPI_CHECK_NOTNULL(weightScale, "weightScale");
    OPAPI_CHECK_NOTNULL(xScale, "xScale");
    OPAPI_CHECK_NOTNULL(groupList, "groupList");
    OPAPI_CHECK_NOTNULL(output, "output");
    OPAPI_CHECK_NOTNULL(outputScale, "outputScale");
    OPAPI_CHECK_NOTNULL(workspaceSize, "workspaceSize");
    OPAPI_CHECK_NOTNULL(executor, "executor");
    OPAPI_CHECK_EXTENTS(x, weight, weightScale, xScale, groupList, output, outputScale);
    constexpr aclnnStatus kInvalid = ACLNN_ERR_PARAM_INVALID;

    OPAPI_CHECK(x->dtype == ACL_INT8 && weight->dtype == ACL_INT8, kInvalid,
                "only the A8W8 path is built: x and weight must be INT8 (got %d, %d)", (int)x->dtype, (int)weight->dtype);
    const bool nz = forceNz || weight->format == ACL_FORMAT_FRACTAL_NZ;
    OPAPI_CHECK(nz || weight->format == ACL_FORMAT_ND, kInvalid, "weight Format expect is ND or FRACTAL_NZ, but got [%d].",
                (int)weight->format);
    OPAPI_CHECK(x->dims.size() == 2, kInvalid, "x must be 2-D [M,K], got %s", ShapeStr(x).c_str());
    // a blocked weight is described either by its 5-D shape [E, N/32, K/16, 16, 32] or by the 3-D view [E, K, N] over
    // storage of that shape
    const std::vector<int64_t>& blocked = weight->dims.size() == 5 ? weight->dims : weight->storage;
    if (nz) {
        OPAPI_CHECK(weight->dims.size() == 5 || weight->dims.size() == 3, kInvalid,
                    "a FRACTAL_NZ weight must be 5-D [E,N/32,K/16,16,32] or a 3-D view of such storage, got %s",
                    ShapeStr(weight).c_str());
        OPAPI_CHECK(blocked.size() == 5 && blocked[3] == 16 && blocked[4] == 32, kInvalid,
                    "The dimnum of storageShape for second input (weight) must be 5 with the last two dims (16, 32).");
    } else {
        OPAPI_CHECK(weight->dims.size() == 3, kInvalid, "weight must be 3-D [E,K,N], got %s", ShapeStr(weight).c_str());
    }
    OPAPI_CHECK(weightScale->dims.size() == 2, kInvalid, "weightScale must be 2-D [E,N], got %s",
                ShapeStr(weightScale).c_str());
    OPAPI_CHECK(xScale->dims.size() == 1, kInvalid, "xScale must be 1-D [M], got %s", ShapeStr(xScale).c_str());
    OPAPI_CHECK(groupList->dims.size() == 1, kInvalid, "groupList must be 1-D, got %s", ShapeStr(groupList).c_str());
    OPAPI_CHECK(output->dims.size() == 2, kInvalid, "output must be 2-D [M,N/2], got %s", ShapeStr(output).c_str());
    OPAPI_CHECK(outputScale->dims.size() == 1, kInvalid, "outputScale must be 1-D [M], got %s",
                ShapeStr(outputScale).c_str());

    const int64_t e = weight->dims[0], m = x->dims[0], k = x->dims[1];
    const int64_t n = weight->dims.size() == 5 ? weight->dims[1] * 32 : weight->dims[2];
    const int64_t wk = weight->dims.size() == 5 ? weight->dims[2] * 16 : weight->dims[1];
    OPAPI_CHECK(wk == k, kInvalid, "weight %s does not match x %s along K", ShapeStr(weight).c_str(), ShapeStr(x).c_str());
    if (nz) {
        OPAPI_CHECK(blocked[0] == e && blocked[1] * 32 == n && blocked[2] * 16 == k, kInvalid,
                    "the blocked weight storage must be [%lld, %lld, %lld, 16, 32] (N a multiple of 32, K of 16)",
                    (long long)e, (long long)(n / 32), (long long)(k / 16));
    }
    OPAPI_CHECK(n % 2 == 0, kInvalid, "N is %lld , which must even number.", (long long)n);
    OPAPI_CHECK(weightScale->dims[0] == e && weightScale->dims[1] == n, kInvalid, "weightScale must be [%lld,%lld], got %s",
                (long long)e, (long long)n, ShapeStr(weightScale).c_str());
    OPAPI_CHECK(xScale->dims[0] == m, kInvalid, "xScale must be [%lld], got %s", (long long)m, ShapeStr(xScale).c_str());
    OPAPI_CHECK(output->dims[0] == m && output->dims[1] == n / 2, kInvalid, "output must be [%lld,%lld], got %s",
                (long long)m, (long long)(n / 2), ShapeStr(output).c_str());
    OPAPI_CHECK(outputScale->dims[0] == m, kInvalid, "outputScale must be [%lld], got %s", (long long)m,
                ShapeStr(outputScale).c_str());
    const int64_t groupListLen = groupList->dims[0];
    OPAPI_CHECK(groupListLen <= e, kInvalid, "Length of 'groupList' out of range (expected to be in range of [1, %lld], but got %lld)",
                (long long)e, (long long)groupListLen);
    OPAPI_CHECK(groupListLen <= 1024, kInvalid, "groupList longer than 1024 groups is not supported");
    OPAPI_CHECK(k < kKLimit, kInvalid, "The tail axis dimension of input0(x) is %lld, which need lower than %lld.",
                (long long)k, (long long)kKLimit);
    OPAPI_CHECK(m < (1ll << 31) && n < (1ll << 31), kInvalid, "M and N must fit int32");

    OPAPI_CHECK(weightScale->dtype == ACL_FLOAT || weightScale->dtype == ACL_FLOAT16 || weightScale->dtype == ACL_BF16,
                kInvalid, "weightScale must be FLOAT, FLOAT16 or BF16");
    OPAPI_CHECK(xScale->dtype == ACL_FLOAT, kInvalid, "xScale must be FLOAT");
    OPAPI_CHECK(groupList->dtype == ACL_INT64 || groupList->dtype == ACL_INT32, kInvalid,
                "groupList must be INT64 (or INT32)");
    OPAPI_CHECK(output->dtype == ACL_INT8, kInvalid, "output must be INT8");
    OPAPI_CHECK(outputScale->dtype == ACL_FLOAT, kInvalid, "outputScale must be FLOAT");

    if (IsEmpty(output) || IsEmpty(groupList) || IsEmpty(outputScale)) {
        auto* noop = new (std::nothrow) NoOpExecutor();
        OPAPI_CHECK(noop != nullptr, ACLNN_ERR_INNER_CREATE_EXECUTOR, "out of host memory");
        *workspaceSize = 0;
        *executor = noop;
        return ACLNN_SUCCESS;
    }
    OPAPI_CHECK(k > 0, kInvalid, "K must be positive");

    const bool wTransposed = !nz && IsLastTwoDimsTransposed(weight);
    OPAPI_CHECK(nz || wTransposed || IsContiguous(weight), kInvalid,
                "weight must be contiguous [E,K,N] or the transposed view of contiguous [E,N,K] storage");
    OPAPI_CHECK(!nz || weight->offset == 0, kInvalid, "a FRACTAL_NZ weight must start at its storage");
    OPAPI_CHECK(IsContiguous(output) && IsContiguous(outputScale), kInvalid,
                "output and outputScale must be contiguous");  // the inputs other than weight may be strided views
    const aclTensor* all[] = {x, weight, weightScale, xScale, groupList, output, outputScale};
    for (const aclTensor* t : all) {
        OPAPI_CHECK(t->data != nullptr, ACLNN_ERR_PARAM_NULLPTR, "a tensor carries no device memory");
    }

    auto* ex = new (std::nothrow) SwigluQuantExecutor();
    OPAPI_CHECK(ex != nullptr, ACLNN_ERR_INNER_CREATE_EXECUTOR, "out of host memory");
    gemm::Problem& p = ex->problem;
    OPAPI_BIND(ex, x, &p.x);
    p.w = reinterpret_cast<const int8_t*>(DataPtr(weight));
    p.wKMajor = wTransposed;
    p.wNz = nz;
    p.M = m;
    p.K = k;
    p.N = n;
    p.groups = static_cast<int32_t>(groupListLen);
    OPAPI_BIND(ex, groupList, &p.groupList);
    p.groupListIsInt64 = groupList->dtype == ACL_INT64;
    p.groupListKind = gemm::GroupListKind::kCumsum;
    p.epilogue = gemm::Epilogue::kSwiglu;
    OPAPI_BIND(ex, weightScale, &p.scale);
    p.scaleDtype = static_cast<int>(weightScale->dtype);
    OPAPI_BIND(ex, xScale, &p.rowScale);
    p.quantOut = reinterpret_cast<int8_t*>(DataPtr(output));
    p.quantScaleOut = reinterpret_cast<float*>(DataPtr(outputScale));
    ex->plan = gemm::MakePlan(p);
    ex->SealWorkspace(ex->plan.workspaceBytes);
    *workspaceSize = ex->workspaceBytes;
    *executor = ex;
    return ACLNN_SUCCESS;
}

}  // namespace

extern "C" aclnnStatus aclnnGroupedMatmulSwigluQuantGetWorkspaceSize(
    const aclTensor* x, const aclTensor* weight, const aclTensor* bias, const aclTensor* offset,
    const aclTensor* weightScale, const aclTensor* xScale, const aclTensor* groupList, aclTensor* output,
    aclTensor* outputScale, aclTensor* outputOffset, uint64_t* workspaceSize, aclOpExecutor** executor) {
    return PlanSwigluQuant(x, weight, bias, offset, weightScale, xScale, groupList, output, outputScale, outputOffset,
                           /*forceNz=*/false, workspaceSize, executor);
}

extern "C" aclnnStatus aclnnGroupedMatmulSwigluQuantWeightNZGetWorkspaceSize(
    const aclTensor* x, const aclTensor* weight, const aclTensor* bias, const aclTensor* offset,
    const aclTensor* weightScale, const aclTensor* xScale, const aclTensor* groupList, aclTensor* output,
    aclTensor* outputScale, aclTensor* outputOffset, uint64_t* workspaceSize, aclOpExecutor** executor) {
    return PlanSwigluQuant(x, weight, bias, offset, weightScale, xScale, groupList, output, outputScale, outputOffset,
                           /*forceNz=*/true, workspaceSize, executor);
}

extern "C" aclnnStatus aclnnGroupedMatmulSwigluQuantWeightNZ(void* workspace, uint64_t workspaceSize,
                                                             aclOpExecutor* executor, aclrtStream stream) {
    return opapi::RunAndRelease(workspace, workspaceSize, executor, stream);
}

extern "C" aclnnStatus aclnnGroupedMatmulSwigluQuant(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor,
                                                     aclrtStream stream) {
    return opapi::RunAndRelease(workspace, workspaceSize, executor, stream);
}
