// aclnnGroupedMatmulFinalizeRouting / V2 / V3 for gfx950: the int8 down projection of the MoE FFN fused with the weighted
// combine (scatter-add of every expanded row into its token's output row).
//
// Reference behaviour restated: gmm/grouped_matmul_finalize_routing/op_kernel/grouped_matmul_finalize_routing.h
//   :217-254  output initialisation: zero outside the shared rows, float(sharedInput) * sharedInputWeight inside
//   :458-495  per row: perToken * logit broadcast; bias row scaled by logit
//   :390-417  (acc * scale) * (perToken * logit) [+ logit * bias]
//   :321-342  atomic fp32 add into out[rowIndex[r], :]
// Argument rules follow op_host/op_api/aclnn_grouped_matmul_finalize_routing.cpp:240-300 (dtypes), :345-380 (ranks),
// :395-500 (extents), :560-572 (out / sharedInputOffset / groupListType), :1100-1111 (dtype 0, no transposes).
// The GEMM itself is the shared grouped int8 engine (grouped_gemm_i8.hip) with its dequantising epilogue in
// scatter-add mode; two small kernels prepare its inputs: the output initialisation and the per-row factor
// perToken * logit.
#include "aclnnop/aclnn_grouped_matmul_finalize_routing.h"

#include <hip/hip_fp16.h>

#include <new>

#include "grouped_gemm_i8.h"
#include "opapi_common.h"

namespace {

struct InitArgs {
    float* out;
    const uint16_t* shared;  // optional
    int32_t sharedIsBf16;
    float sharedWeight;
    int64_t sharedOffset, sharedRows;
    int64_t batch, n;
};

// One thread per four output floats (n is a multiple of 4 on this path, else one per element).
template <int kVec>
__global__ __launch_bounds__(256) void InitCombineOutputKernel(InitArgs a) {
    const int64_t perRow = a.n / kVec;
    const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= a.batch * perRow) return;
    const int64_t row = i / perRow, col = (i % perRow) * kVec;
    float v[kVec];
#pragma unroll
    for (int e = 0; e < kVec; ++e) v[e] = 0.0f;
    if (a.shared != nullptr && row >= a.sharedOffset && row < a.sharedOffset + a.sharedRows) {
        const uint16_t* src = a.shared + (row - a.sharedOffset) * a.n + col;
#pragma unroll
        for (int e = 0; e < kVec; ++e) {
            const float f = a.sharedIsBf16 ? __uint_as_float(static_cast<uint32_t>(src[e]) << 16)
                                           : __half2float(__ushort_as_half(src[e]));
            v[e] = __fmul_rn(f, a.sharedWeight);
        }
    }
    float* dst = a.out + row * a.n + col;
    if constexpr (kVec == 4) *reinterpret_cast<float4*>(dst) = make_float4(v[0], v[1], v[2], v[3]);
    else dst[0] = v[0];
}

// rowFactor[r] = perToken[r] * logit[r] (either may be absent: factor 1).
__global__ void RowFactorKernel(const float* perToken, const float* logit, float* rowFactor, int64_t m) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= m) return;
    const float p = perToken != nullptr ? perToken[i] : 1.0f;
    rowFactor[i] = logit != nullptr ? __fmul_rn(p, logit[i]) : p;
}

class CombineExecutor : public aclOpExecutor {
   public:
    gemm::Problem problem;
    gemm::Plan plan;
    InitArgs init{};
    const float* perToken = nullptr;
    const float* logit = nullptr;
    uint64_t offRowFactor = 0;
    bool needRowFactor = false;

    aclnnStatus Run(void* workspace, hipStream_t stream) override {
        char* ws = static_cast<char*>(workspace);
        if (init.batch > 0 && init.n > 0) {
            opapi::KernelTimer timer("combine_init", stream);
            const bool wide = init.n % 4 == 0 && reinterpret_cast<uintptr_t>(init.out) % 16 == 0;
            const int64_t threads = init.batch * (wide ? init.n / 4 : init.n);
            const unsigned blocks = static_cast<unsigned>((threads + 255) / 256);
            if (wide) hipLaunchKernelGGL(InitCombineOutputKernel<4>, dim3(blocks), dim3(256), 0, stream, init);
            else hipLaunchKernelGGL(InitCombineOutputKernel<1>, dim3(blocks), dim3(256), 0, stream, init);
        }
        if (problem.M == 0) return ACLNN_SUCCESS;
        problem.combineWeight = logit;
        problem.rowScale = perToken;
        if (needRowFactor) {
            float* rowFactor = reinterpret_cast<float*>(ws + offRowFactor);
            hipLaunchKernelGGL(RowFactorKernel, dim3(static_cast<unsigned>((problem.M + 255) / 256)), dim3(256), 0, stream,
                               perToken, logit, rowFactor, problem.M);
            problem.rowScale = rowFactor;
        }
        const hipError_t e = gemm::Enqueue(problem, plan, workspace, stream);
        if (e != hipSuccess) {
            opapi::SetError("aclnnGroupedMatmulFinalizeRouting: launch failed: %s", hipGetErrorString(e));
            return ACLNN_ERR_RUNTIME_ERROR;
        }
        return ACLNN_SUCCESS;
    }
};

aclnnStatus PlanCombine(const char* api, const aclTensor* x1, const aclTensor* x2, const aclTensor* scale,
                        const aclTensor* bias, const aclTensor* offset, const aclTensor* antiquantScale,
                        const aclTensor* antiquantOffset, const aclTensor* perToken, const aclTensor* groupList,
                        const aclTensor* sharedInput, const aclTensor* logit, const aclTensor* rowIndex, int64_t dtype,
                        float sharedInputWeight, int64_t sharedInputOffset, bool transposeX1, bool transposeX2,
                        int64_t groupListType, const aclIntArray* tuningConfig, bool forceNz, const aclTensor* out,
                        uint64_t* workspaceSize, aclOpExecutor** executor) {
    using namespace opapi;
    ClearError();
    constexpr aclnnStatus kInvalid = ACLNN_ERR_PARAM_INVALID;
    OPAPI_CHECK(x1 != nullptr && x2 != nullptr && scale != nullptr && groupList != nullptr && rowIndex != nullptr &&
                    out != nullptr, ACLNN_ERR_PARAM_NULLPTR,
                "%s do not support input nullptr (x1, x2, scale, groupList, rowIndex, out).", api);
    OPAPI_CHECK_NOTNULL(workspaceSize, "workspaceSize");
    OPAPI_CHECK_NOTNULL(executor, "executor");
    OPAPI_CHECK_EXTENTS(x1, x2, scale, bias, perToken, groupList, sharedInput, logit, rowIndex, out);
    OPAPI_CHECK(antiquantScale == nullptr && antiquantOffset == nullptr, ACLNN_ERR_PARAM_NULLPTR,
                "%s: antiquantScale / antiquantOffset are not enabled and must be nullptr.", api);
    OPAPI_CHECK(dtype == 0, kInvalid, "%s dtype must be 0, but is %lld.", api, (long long)dtype);
    OPAPI_CHECK(!transposeX1 && !transposeX2, kInvalid, "%s transpose should be false", api);

    // dtypes
    OPAPI_CHECK(x1->dtype == ACL_INT8, kInvalid, "x1 must be INT8");
    OPAPI_CHECK(x2->dtype != ACL_INT32 && x2->dtype != ACL_INT4, kInvalid,
                "INT4 weights (packed in INT32) are not built here: this build's fused combine takes INT8 weights");
    OPAPI_CHECK(x2->dtype == ACL_INT8, kInvalid, "x1 and x2 dtype should be same (INT8), actual x2 dtype is %d.", (int)x2->dtype);
    // a blocked (FRACTAL_NZ) INT8 weight: [E, N/32, K/16, 16, 32] as a 5-D tensor or as the 3-D view [E, K, N] over
    // storage of that shape; the WeightNz entry points take the storage shape as the only evidence
    const bool nz = forceNz || x2->format == ACL_FORMAT_FRACTAL_NZ;
    OPAPI_CHECK(nz || x2->format == ACL_FORMAT_ND, kInvalid, "x2's format should be ND or FRACTAL_NZ. actual is [%d].",
                (int)x2->format);
    const std::vector<int64_t>& blocked = x2->dims.size() == 5 ? x2->dims : x2->storage;
    OPAPI_CHECK(!nz || ((x2->dims.size() == 5 || x2->dims.size() == 3) && blocked.size() == 5 && blocked[3] == 16 &&
                        blocked[4] == 32), kInvalid,
                "x2'format only support NZ, but now x2's format is not NZ: the storage shape must be [E, N/32, K/16, 16, 32].");
    OPAPI_CHECK(offset == nullptr, kInvalid, "offset belongs to the INT4 case and must be nullptr with INT8 weights");
    OPAPI_CHECK(scale->dtype == ACL_FLOAT || scale->dtype == ACL_BF16, kInvalid, "scale must be FLOAT or BF16");
    OPAPI_CHECK(bias == nullptr || bias->dtype == ACL_BF16 || bias->dtype == ACL_FLOAT, kInvalid, "bias must be BF16 or FLOAT");
    OPAPI_CHECK(perToken == nullptr || perToken->dtype == ACL_FLOAT, kInvalid, "pertokenScale must be FLOAT");
    OPAPI_CHECK(groupList->dtype == ACL_INT64 || groupList->dtype == ACL_INT32, kInvalid, "groupList must be INT64 (or INT32)");
    OPAPI_CHECK(sharedInput == nullptr || sharedInput->dtype == ACL_BF16 || sharedInput->dtype == ACL_FLOAT16, kInvalid,
                "sharedInput must be BF16 or FLOAT16");
    OPAPI_CHECK(logit == nullptr || logit->dtype == ACL_FLOAT, kInvalid, "logit must be FLOAT");
    OPAPI_CHECK(rowIndex->dtype == ACL_INT64 || rowIndex->dtype == ACL_INT32, kInvalid, "rowIndex must be INT64 or INT32");
    OPAPI_CHECK(out->dtype == ACL_FLOAT, kInvalid, "out must be FLOAT");

    // ranks and extents
    OPAPI_CHECK(x1->dims.size() == 2, kInvalid, "input x Dims is %zu, weight Dims is %zu.", x1->dims.size(), x2->dims.size());
    OPAPI_CHECK(x2->dims.size() == 3 || (nz && x2->dims.size() == 5), kInvalid, "input x Dims is %zu, weight Dims is %zu.",
                x1->dims.size(), x2->dims.size());
    OPAPI_CHECK(out->dims.size() == 2, kInvalid, "Out dim num should be equal to 2, but is %zu.", out->dims.size());
    const int64_t m = x1->dims[0], k = x1->dims[1], e = x2->dims[0], batch = out->dims[0];
    const int64_t n = x2->dims.size() == 5 ? x2->dims[1] * 32 : x2->dims[2];
    const int64_t wk = x2->dims.size() == 5 ? x2->dims[2] * 16 : x2->dims[1];
    OPAPI_CHECK(wk == k, kInvalid, "x1 k dim and x2 k dim should be same, but are %lld and %lld.", (long long)k, (long long)wk);
    OPAPI_CHECK(!nz || (blocked[0] == e && blocked[1] * 32 == n && blocked[2] * 16 == k && x2->offset == 0), kInvalid,
                "the blocked weight storage must be [%lld, %lld, %lld, 16, 32] (N a multiple of 32, K of 16)", (long long)e,
                (long long)(n / 32), (long long)(k / 16));
    const bool scale2d = scale->dims.size() == 2 && scale->dims[0] == e && scale->dims[1] == n;
    const bool scale3d = scale->dims.size() == 3 && scale->dims[0] == e && scale->dims[1] == 1 && scale->dims[2] == n;
    OPAPI_CHECK(scale->dims.empty() || scale->dims[0] == e, kInvalid,
                "Scale fisrt dim should equal to weight EDim %lld, but actual is %lld.", (long long)e, (long long)scale->dims[0]);
    OPAPI_CHECK(scale2d || scale3d, kInvalid, "scale must be [%lld, %lld] or [%lld, 1, %lld], got %s", (long long)e,
                (long long)n, (long long)e, (long long)n, ShapeStr(scale).c_str());
    OPAPI_CHECK(bias == nullptr || (bias->dims.size() == 2 && bias->dims[0] == e && bias->dims[1] == n), kInvalid,
                "bias's dim value should be (e, n) = (%lld, %lld), got %s", (long long)e, (long long)n,
                bias ? ShapeStr(bias).c_str() : "");
    OPAPI_CHECK(perToken == nullptr || (perToken->dims.size() == 1 && perToken->dims[0] == m), kInvalid,
                "pertokenScale fisrt dim should equal to x MDim %lld, but actual is %s.", (long long)m,
                perToken ? ShapeStr(perToken).c_str() : "");
    OPAPI_CHECK(groupList->dims.size() == 1 && groupList->dims[0] == e, kInvalid,
                "groupList fisrt dim should equal to weight EDim %lld, but actual is %s.", (long long)e, ShapeStr(groupList).c_str());
    OPAPI_CHECK(logit == nullptr || (logit->dims.size() == 1 && logit->dims[0] == m), kInvalid,
                "logit fisrt dim should equal to x MDim %lld, but actual is %s.", (long long)m, logit ? ShapeStr(logit).c_str() : "");
    OPAPI_CHECK(rowIndex->dims.size() == 1 && rowIndex->dims[0] == m, kInvalid,
                "rowIndex fisrt dim should equal to x MDim %lld, but actual is %s.", (long long)m, ShapeStr(rowIndex).c_str());
    OPAPI_CHECK(batch <= m && batch >= 0, kInvalid,
                "Out 1st dim should be less than or equal to x MDim , but out 1st dim is %lld", (long long)batch);
    OPAPI_CHECK(out->dims[1] == n, kInvalid, "Out 2nd dim should be equal to weight NDim %lld, but is %lld.", (long long)n,
                (long long)out->dims[1]);
    OPAPI_CHECK(sharedInputOffset >= 0, kInvalid, "sharedInputOffset should bigger than or equal to 0");
    int64_t sharedRows = 0;
    if (sharedInput != nullptr) {
        OPAPI_CHECK(sharedInput->dims.size() == 2 && sharedInput->dims[1] == n, kInvalid,
                    "sharedInput must be [rows, %lld], got %s", (long long)n, ShapeStr(sharedInput).c_str());
        sharedRows = sharedInput->dims[0];
        OPAPI_CHECK(sharedRows <= batch, kInvalid,
                    "shareInput fisrt dim should less than or equal to outputBS %lld, but actual is %lld.", (long long)batch,
                    (long long)sharedRows);
        OPAPI_CHECK(sharedInputOffset + sharedRows <= batch, kInvalid,
                    "sharedInputOffset %lld plus the shared rows %lld exceeds outputBS %lld.", (long long)sharedInputOffset,
                    (long long)sharedRows, (long long)batch);
    }
    OPAPI_CHECK(groupListType == 0 || groupListType == 1, kInvalid, "groupListType should be 0 or 1, but is %lld",
                (long long)groupListType);
    OPAPI_CHECK(e <= 1024, kInvalid, "at most 1024 groups are supported, got %lld", (long long)e);
    OPAPI_CHECK(k > 0 && k < 65536, kInvalid, "K must be in [1, 65535], got %lld", (long long)k);
    OPAPI_CHECK(m < (1ll << 31) && n < (1ll << 31) && n > 0, kInvalid, "M and N must fit int32 and N must be positive");
    int64_t expected = 0;
    if (tuningConfig != nullptr && !tuningConfig->values.empty()) {
        expected = tuningConfig->values[0];
        OPAPI_CHECK(expected >= 0 && expected <= m, kInvalid,
                    "GroupedMatmulFinalizeRouting Invalid tuningConfigOptional (%lld)! It should be a non-negative num and less than or equal to x MDim.",
                    (long long)expected);
    }

    const bool wTransposed = !nz && IsLastTwoDimsTransposed(x2);
    OPAPI_CHECK(nz || wTransposed || IsContiguous(x2), kInvalid,
                "x2 must be contiguous [E,K,N] or the transposed view of contiguous [E,N,K] storage");
    OPAPI_CHECK(IsContiguous(out), kInvalid, "out must be contiguous");  // inputs other than x2 may be strided views
    const aclTensor* all[] = {x1, x2, scale, bias, perToken, groupList, sharedInput, logit, rowIndex, out};
    for (const aclTensor* t : all) {
        OPAPI_CHECK(t == nullptr || Numel(t) == 0 || t->data != nullptr, ACLNN_ERR_PARAM_NULLPTR,
                    "a tensor carries no device memory");
    }

    auto* ex = new (std::nothrow) CombineExecutor();
    OPAPI_CHECK(ex != nullptr, ACLNN_ERR_INNER_CREATE_EXECUTOR, "out of host memory");
    ex->init.out = reinterpret_cast<float*>(DataPtr(out));
    OPAPI_BIND(ex, sharedInput, &ex->init.shared);
    ex->init.sharedIsBf16 = sharedInput != nullptr && sharedInput->dtype == ACL_BF16 ? 1 : 0;
    ex->init.sharedWeight = sharedInputWeight;
    ex->init.sharedOffset = sharedInputOffset;
    ex->init.sharedRows = sharedRows;
    ex->init.batch = batch;
    ex->init.n = n;
    OPAPI_BIND(ex, perToken, &ex->perToken);
    OPAPI_BIND(ex, logit, &ex->logit);
    gemm::Problem& p = ex->problem;
    OPAPI_BIND(ex, x1, &p.x);
    p.w = reinterpret_cast<const int8_t*>(DataPtr(x2));
    p.wKMajor = wTransposed;
    p.wNz = nz;
    p.M = batch == 0 ? 0 : m;
    p.K = k;
    p.N = n;
    p.groups = static_cast<int32_t>(e);
    OPAPI_BIND(ex, groupList, &p.groupList);
    p.groupListIsInt64 = groupList->dtype == ACL_INT64;
    p.groupListKind = groupListType == 1 ? gemm::GroupListKind::kCount : gemm::GroupListKind::kCumsum;
    p.expectedRowsPerGroup = expected;
    p.epilogue = gemm::Epilogue::kDequant;
    p.out = DataPtr(out);
    p.outDtype = static_cast<int>(ACL_FLOAT);
    OPAPI_BIND(ex, scale, &p.scale);
    p.scaleDtype = static_cast<int>(scale->dtype);
    OPAPI_BIND(ex, rowIndex, &p.combineIndex);
    p.combineIndexIsInt64 = rowIndex->dtype == ACL_INT64;
    p.combineRows = batch;
    p.combineWeight = ex->logit;  // both refreshed in Run, where staged inputs have their final address
    OPAPI_BIND(ex, bias, &p.bias);
    p.biasDtype = bias != nullptr ? static_cast<int>(bias->dtype) : 0;
    ex->plan = gemm::MakePlan(p);
    // the row factor: perToken alone can be used as it is; anything involving logit is multiplied out first
    ex->needRowFactor = logit != nullptr;
    p.rowScale = ex->perToken;
    uint64_t bytes = ex->plan.workspaceBytes;
    if (ex->needRowFactor) {
        ex->offRowFactor = AlignUp(bytes, 256);
        bytes = ex->offRowFactor + AlignUp(static_cast<uint64_t>(m) * 4, 256);
    }
    ex->SealWorkspace(p.M == 0 ? 0 : bytes);
    *workspaceSize = ex->workspaceBytes;
    *executor = ex;
    return ACLNN_SUCCESS;
}

}  // namespace

extern "C" aclnnStatus aclnnGroupedMatmulFinalizeRoutingGetWorkspaceSize(
    const aclTensor* x, aclTensor* w, const aclTensor* scaleOptional, const aclTensor* biasOptional,
    const aclTensor* pertokenScaleOptional, const aclTensor* groupListOptional, const aclTensor* sharedInputOptional,
    const aclTensor* logitOptional, const aclTensor* rowIndexOptional, int64_t dtype, float sharedInputWeight,
    int64_t sharedInputOffset, bool transposeX, bool transposeW, int64_t groupListType, aclTensor* y,
    uint64_t* workspaceSize, aclOpExecutor** executor) {
    return PlanCombine("GroupedMatmulFinalizeRouting weightNd", x, w, scaleOptional, biasOptional, nullptr, nullptr, nullptr,
                       pertokenScaleOptional, groupListOptional, sharedInputOptional, logitOptional, rowIndexOptional, dtype,
                       sharedInputWeight, sharedInputOffset, transposeX, transposeW, groupListType, nullptr, /*forceNz=*/false, y,
                       workspaceSize, executor);
}

extern "C" aclnnStatus aclnnGroupedMatmulFinalizeRouting(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor,
                                                         aclrtStream stream) {
    return opapi::RunAndRelease(workspace, workspaceSize, executor, stream);
}

extern "C" aclnnStatus aclnnGroupedMatmulFinalizeRoutingV2GetWorkspaceSize(
    const aclTensor* x1, aclTensor* x2, const aclTensor* scaleOptional, const aclTensor* biasOptional,
    const aclTensor* offsetOptional, const aclTensor* antiquantScaleOptional, const aclTensor* antiquantOffsetOptional,
    const aclTensor* pertokenScaleOptional, const aclTensor* groupListOptional, const aclTensor* sharedInputOptional,
    const aclTensor* logitOptional, const aclTensor* rowIndexOptional, int64_t dtype, float sharedInputWeight,
    int64_t sharedInputOffset, bool transposeX1, bool transposeX2, int64_t groupListType, aclTensor* out,
    uint64_t* workspaceSize, aclOpExecutor** executor) {
    return PlanCombine("GroupedMatmulFinalizeRoutingV2 weightNd", x1, x2, scaleOptional, biasOptional, offsetOptional,
                       antiquantScaleOptional, antiquantOffsetOptional, pertokenScaleOptional, groupListOptional,
                       sharedInputOptional, logitOptional, rowIndexOptional, dtype, sharedInputWeight, sharedInputOffset,
                       transposeX1, transposeX2, groupListType, nullptr, /*forceNz=*/false, out, workspaceSize, executor);
}

extern "C" aclnnStatus aclnnGroupedMatmulFinalizeRoutingV2(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor,
                                                           aclrtStream stream) {
    return opapi::RunAndRelease(workspace, workspaceSize, executor, stream);
}

extern "C" aclnnStatus aclnnGroupedMatmulFinalizeRoutingV3GetWorkspaceSize(
    const aclTensor* x1, aclTensor* x2, const aclTensor* scaleOptional, const aclTensor* biasOptional,
    const aclTensor* offsetOptional, const aclTensor* antiquantScaleOptional, const aclTensor* antiquantOffsetOptional,
    const aclTensor* pertokenScaleOptional, const aclTensor* groupListOptional, const aclTensor* sharedInputOptional,
    const aclTensor* logitOptional, const aclTensor* rowIndexOptional, int64_t dtype, float sharedInputWeight,
    int64_t sharedInputOffset, bool transposeX1, bool transposeX2, int64_t groupListType,
    const aclIntArray* tuningConfigOptional, aclTensor* out, uint64_t* workspaceSize, aclOpExecutor** executor) {
    return PlanCombine("aclnnGroupedMatmulFinalizeRoutingV3 weightNd", x1, x2, scaleOptional, biasOptional, offsetOptional,
                       antiquantScaleOptional, antiquantOffsetOptional, pertokenScaleOptional, groupListOptional,
                       sharedInputOptional, logitOptional, rowIndexOptional, dtype, sharedInputWeight, sharedInputOffset,
                       transposeX1, transposeX2, groupListType, tuningConfigOptional, /*forceNz=*/false, out, workspaceSize,
                       executor);
}

extern "C" aclnnStatus aclnnGroupedMatmulFinalizeRoutingV3(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor,
                                                           aclrtStream stream) {
    return opapi::RunAndRelease(workspace, workspaceSize, executor, stream);
}

// The FRACTAL_NZ entry points (aclnn_grouped_matmul_finalize_routing.cpp:943-1083): the reference's route for INT8 weights.
extern "C" aclnnStatus aclnnGroupedMatmulFinalizeRoutingWeightNzGetWorkspaceSize(
    const aclTensor* x1, const aclTensor* x2, const aclTensor* scale, const aclTensor* bias,
    const aclTensor* pertokenScaleOptional, const aclTensor* groupList, const aclTensor* sharedInput, const aclTensor* logit,
    const aclTensor* rowIndex, int64_t dtype, float sharedInputWeight, int64_t sharedInputOffset, bool transposeX1,
    bool transposeX2, int64_t groupListType, aclTensor* out, uint64_t* workspaceSize, aclOpExecutor** executor) {
    return PlanCombine("GroupedMatmulFinalizeRoutingWeightNz", x1, x2, scale, bias, nullptr, nullptr, nullptr,
                       pertokenScaleOptional, groupList, sharedInput, logit, rowIndex, dtype, sharedInputWeight,
                       sharedInputOffset, transposeX1, transposeX2, groupListType, nullptr, /*forceNz=*/true, out,
                       workspaceSize, executor);
}

extern "C" aclnnStatus aclnnGroupedMatmulFinalizeRoutingWeightNz(void* workspace, uint64_t workspaceSize,
                                                                 aclOpExecutor* executor, aclrtStream stream) {
    return opapi::RunAndRelease(workspace, workspaceSize, executor, stream);
}

extern "C" aclnnStatus aclnnGroupedMatmulFinalizeRoutingWeightNzV2GetWorkspaceSize(
    const aclTensor* x1, aclTensor* x2, const aclTensor* scale, const aclTensor* bias, const aclTensor* offsetOptional,
    const aclTensor* antiquantScaleOptional, const aclTensor* antiquantOffsetOptional,
    const aclTensor* pertokenScaleOptional, const aclTensor* groupList, const aclTensor* sharedInput, const aclTensor* logit,
    const aclTensor* rowIndex, int64_t dtype, float sharedInputWeight, int64_t sharedInputOffset, bool transposeX1,
    bool transposeX2, int64_t groupListType, const aclIntArray* tuningConfigOptional, aclTensor* out,
    uint64_t* workspaceSize, aclOpExecutor** executor) {
    return PlanCombine("GroupedMatmulFinalizeRoutingWeightNzV2", x1, x2, scale, bias, offsetOptional, antiquantScaleOptional,
                       antiquantOffsetOptional, pertokenScaleOptional, groupList, sharedInput, logit, rowIndex, dtype,
                       sharedInputWeight, sharedInputOffset, transposeX1, transposeX2, groupListType, tuningConfigOptional,
                       /*forceNz=*/true, out, workspaceSize, executor);
}

extern "C" aclnnStatus aclnnGroupedMatmulFinalizeRoutingWeightNzV2(void* workspace, uint64_t workspaceSize,
                                                                   aclOpExecutor* executor, aclrtStream stream) {
    return opapi::RunAndRelease(workspace, workspaceSize, executor, stream);
}
