// aclnnMoeGatingTopKSoftmaxV2 for gfx950: the router in front of the MoE expert FFN (softmax over the expert logits and
// top-k selection, in either order).
//
// Reference behaviour restated: moe/moe_gating_top_k_softmax_v2/op_kernel/moe_gating_top_k_softmax_v2_ek_fullload.h
// (:309-412 softmax then top-k with the inputs widened to fp32; :414-545 top-k then softmax over the k values;
// results narrowed with CAST_ROUND, :211-262) and moe_gating_top_k_softmax_v2_perf.h:603-637 (finished rows: every
// index becomes the expert count).  Validation follows op_host/moe_gating_top_k_softmax_v2_tiling_base.cpp:40-260.
//
// One workgroup owns one row.  The row lives in LDS as order-preserving 32-bit keys (a float's bits mapped so that
// unsigned comparison equals float comparison; key 0 marks "already taken", below every real value including -inf).
// Selection is k rounds of a workgroup arg-max over 64-bit (key, ~index) pairs, which yields descending values with
// equal values in ascending index order without sorting the whole row: k is small next to the expert count.
#include "opapi_common.h"

#include <hip/hip_fp16.h>

#include "aclnnop/aclnn_moe_gating_top_k_softmax_v2.h"

namespace {

constexpr int kWave = 64;
constexpr int64_t kMaxK = 1024;
constexpr int64_t kMaxCols = 32768;

struct GatingArgs {
    const void* x;
    const uint8_t* finished;  // optional, one byte per row
    void* y;
    int32_t* expertIdx;
    float* softmaxOut;        // optional
    int64_t rows;
    int32_t cols;
    int32_t k;
    int32_t renorm;
};

__device__ __forceinline__ uint32_t KeyOf(float f) {
    const uint32_t u = __float_as_uint(f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float ValueOf(uint32_t key) {
    return __uint_as_float((key & 0x80000000u) ? (key & 0x7fffffffu) : ~key);
}

// Narrowing with ties away from zero (the reference's CAST_ROUND).
struct F32Out {
    using Storage = float;
    __device__ static float Load(Storage v) { return v; }
    __device__ static Storage Store(float f) { return f; }
};
struct Bf16Out {
    using Storage = uint16_t;
    __device__ static float Load(Storage v) { return __uint_as_float(static_cast<uint32_t>(v) << 16); }
    __device__ static Storage Store(float f) {
        const uint32_t u = __float_as_uint(f);
        if ((u & 0x7fffffffu) > 0x7f800000u) return static_cast<Storage>((u >> 16) | 0x40);
        return static_cast<Storage>((u + 0x8000u) >> 16);  // sign-magnitude: adding half an ulp rounds ties outward
    }
};
struct F16Out {
    using Storage = uint16_t;
    __device__ static float Load(Storage v) { return __half2float(__ushort_as_half(v)); }
    __device__ static Storage Store(float f) {
        const uint16_t near = __half_as_ushort(__float2half_rn(f));  // ties to even
        if ((near & 0x7fffu) >= 0x7c00u) return near;
        // an exact tie that went toward zero moves one step outward
        const float lo = fabsf(Load(near)), hi = fabsf(Load(static_cast<uint16_t>(near + 1))), mag = fabsf(f);
        return (lo < mag && mag - lo == hi - mag) ? static_cast<uint16_t>(near + 1) : near;
    }
};

template <int kWaves>
__device__ __forceinline__ float BlockMax(float v, float* scratch) {
    for (int d = 32; d > 0; d >>= 1) v = fmaxf(v, __shfl_xor(v, d));
    if constexpr (kWaves == 1) return v;
    __syncthreads();
    if (threadIdx.x % kWave == 0) scratch[threadIdx.x / kWave] = v;
    __syncthreads();
    float r = scratch[0];
    for (int w = 1; w < kWaves; ++w) r = fmaxf(r, scratch[w]);
    return r;
}

// Sum in a fixed order (lane tree, then waves in ascending order): the same on every launch.
template <int kWaves>
__device__ __forceinline__ float BlockSum(float v, float* scratch) {
    for (int d = 32; d > 0; d >>= 1) v += __shfl_xor(v, d);
    if constexpr (kWaves == 1) return v;
    __syncthreads();
    if (threadIdx.x % kWave == 0) scratch[threadIdx.x / kWave] = v;
    __syncthreads();
    float r = scratch[0];
    for (int w = 1; w < kWaves; ++w) r += scratch[w];
    return r;
}

template <int kWaves>
__device__ __forceinline__ uint64_t BlockArgMax(uint64_t v, uint64_t* scratch) {
    for (int d = 32; d > 0; d >>= 1) {
        const uint32_t hi = __shfl_xor(static_cast<uint32_t>(v >> 32), d);
        const uint32_t lo = __shfl_xor(static_cast<uint32_t>(v), d);
        const uint64_t other = (static_cast<uint64_t>(hi) << 32) | lo;
        v = other > v ? other : v;
    }
    if constexpr (kWaves == 1) return v;
    __syncthreads();
    if (threadIdx.x % kWave == 0) scratch[threadIdx.x / kWave] = v;
    __syncthreads();
    uint64_t r = scratch[0];
    for (int w = 1; w < kWaves; ++w) r = scratch[w] > r ? scratch[w] : r;
    return r;
}

template <typename Codec, int kWaves>
__global__ __launch_bounds__(kWave * kWaves) void GatingTopKKernel(GatingArgs a) {
    extern __shared__ __attribute__((aligned(16))) unsigned char ldsRaw[];
    constexpr int kThreads = kWave * kWaves;
    // layout: keys[cols] | topKey[k] | topIdx[k] | reduction scratch (8-byte aligned)
    uint32_t* keys = reinterpret_cast<uint32_t*>(ldsRaw);
    uint32_t* topKey = keys + a.cols;
    int32_t* topIdx = reinterpret_cast<int32_t*>(topKey + a.k);
    uint64_t* scratch = reinterpret_cast<uint64_t*>(ldsRaw + ((static_cast<size_t>(a.cols) + 2 * a.k) * 4 + 7) / 8 * 8);
    float* scratchF = reinterpret_cast<float*>(scratch);

    const int64_t row = blockIdx.x;
    const int tid = threadIdx.x;
    const typename Codec::Storage* x = static_cast<const typename Codec::Storage*>(a.x) + row * a.cols;

    float localMax = -INFINITY;
    for (int c = tid; c < a.cols; c += kThreads) {
        const float v = Codec::Load(x[c]);
        keys[c] = __float_as_uint(v);  // raw values for now
        localMax = fmaxf(localMax, v);
    }
    if (a.renorm == 0) {
        const float rowMax = BlockMax<kWaves>(localMax, scratchF);
        float localSum = 0.f;
        for (int c = tid; c < a.cols; c += kThreads) {
            const float e = expf(__uint_as_float(keys[c]) - rowMax);
            keys[c] = __float_as_uint(e);
            localSum += e;
        }
        const float sum = BlockSum<kWaves>(localSum, scratchF);
        for (int c = tid; c < a.cols; c += kThreads) {
            const float p = __uint_as_float(keys[c]) / sum;
            if (a.softmaxOut != nullptr) a.softmaxOut[row * a.cols + c] = p;
            keys[c] = KeyOf(p);
        }
    } else {
        for (int c = tid; c < a.cols; c += kThreads) keys[c] = KeyOf(__uint_as_float(keys[c]));
    }
    __syncthreads();

    for (int j = 0; j < a.k; ++j) {
        uint64_t best = 0;
        for (int c = tid; c < a.cols; c += kThreads) {
            const uint64_t cand = (static_cast<uint64_t>(keys[c]) << 32) | (0xffffffffu - static_cast<uint32_t>(c));
            best = cand > best ? cand : best;
        }
        best = BlockArgMax<kWaves>(best, scratch);
        const int32_t idx = static_cast<int32_t>(0xffffffffu - static_cast<uint32_t>(best));
        if (tid == idx % kThreads) {  // the lane that scans this column retires it and records the pick
            keys[idx] = 0u;
            topKey[j] = static_cast<uint32_t>(best >> 32);
            topIdx[j] = idx;
        }
        __syncthreads();
    }

    const bool done = a.finished != nullptr && a.finished[row] != 0;
    typename Codec::Storage* y = static_cast<typename Codec::Storage*>(a.y) + row * a.k;
    int32_t* outIdx = a.expertIdx + row * a.k;
    if (a.renorm == 0) {
        for (int j = tid; j < a.k; j += kThreads) {
            y[j] = Codec::Store(ValueOf(topKey[j]));
            outIdx[j] = done ? a.cols : topIdx[j];
        }
    } else {
        const float top = ValueOf(topKey[0]);  // the largest selected logit
        __syncthreads();                        // every wave has read it before slot 0 is overwritten below
        float localSum = 0.f;
        for (int j = tid; j < a.k; j += kThreads) {
            const float e = expf(ValueOf(topKey[j]) - top);
            topKey[j] = __float_as_uint(e);
            localSum += e;
        }
        const float sum = BlockSum<kWaves>(localSum, scratchF);
        for (int j = tid; j < a.k; j += kThreads) {
            y[j] = Codec::Store(__uint_as_float(topKey[j]) / sum);
            outIdx[j] = done ? a.cols : topIdx[j];
        }
    }
}

class GatingExecutor : public aclOpExecutor {
   public:
    GatingArgs args{};
    aclDataType dtype = ACL_FLOAT;

    static constexpr size_t LdsBytes(int64_t cols, int64_t k, int waves) {
        return ((static_cast<size_t>(cols) + 2 * static_cast<size_t>(k)) * 4 + 7) / 8 * 8 + static_cast<size_t>(waves) * 8;
    }

    template <typename Codec, int kWaves>
    hipError_t Launch(hipStream_t stream) const {
        auto kernel = GatingTopKKernel<Codec, kWaves>;
        const size_t lds = LdsBytes(args.cols, args.k, kWaves);
        if (lds > 48 * 1024) {
            static std::atomic<uint64_t> optedIn{0};
            const hipError_t attr = opapi::EnsureDynamicLds(reinterpret_cast<const void*>(kernel),
                                                            static_cast<int>(LdsBytes(kMaxCols, kMaxK, kWaves)), optedIn);
            if (attr != hipSuccess) return attr;
        }
        hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(args.rows)), dim3(kWave * kWaves), lds, stream, args);
        return hipGetLastError();
    }

    template <typename Codec>
    hipError_t LaunchForWidth(hipStream_t stream) const {
        if (args.cols <= 512) return Launch<Codec, 1>(stream);
        if (args.cols <= 4096) return Launch<Codec, 4>(stream);
        return Launch<Codec, 16>(stream);
    }

    aclnnStatus Run(void*, hipStream_t stream) override {
        if (args.rows == 0) return ACLNN_SUCCESS;
        opapi::KernelTimer timer("gating_topk_softmax", stream);
        hipError_t err;
        if (dtype == ACL_FLOAT) err = LaunchForWidth<F32Out>(stream);
        else if (dtype == ACL_FLOAT16) err = LaunchForWidth<F16Out>(stream);
        else err = LaunchForWidth<Bf16Out>(stream);
        if (err != hipSuccess) {
            opapi::SetError("aclnnMoeGatingTopKSoftmaxV2: launch failed: %s", hipGetErrorString(err));
            return ACLNN_ERR_RUNTIME_ERROR;
        }
        return ACLNN_SUCCESS;
    }
};

// out has x's shape with the last axis replaced by `last`.
bool SameButLast(const aclTensor* out, const aclTensor* x, int64_t last) {
    if (out->dims.size() != x->dims.size()) return false;
    for (size_t i = 0; i + 1 < x->dims.size(); ++i) {
        if (out->dims[i] != x->dims[i]) return false;
    }
    return out->dims.back() == last;
}

}  // namespace

extern "C" aclnnStatus aclnnMoeGatingTopKSoftmaxV2GetWorkspaceSize(
    const aclTensor* x, const aclTensor* finishedOptional, int64_t k, int64_t renorm, bool outputSoftmaxResultFlag,
    const aclTensor* yOut, const aclTensor* expertIdxOut, const aclTensor* softmaxResultOutOptional,
    uint64_t* workspaceSize, aclOpExecutor** executor) {
    using namespace opapi;
    ClearError();
    OPAPI_CHECK_NOTNULL(x, "x");
    OPAPI_CHECK_NOTNULL(yOut, "yOut");
    OPAPI_CHECK_NOTNULL(expertIdxOut, "expertIdxOut");
    OPAPI_CHECK_NOTNULL(workspaceSize, "workspaceSize");
    OPAPI_CHECK_NOTNULL(executor, "executor");
    OPAPI_CHECK_EXTENTS(x, finishedOptional, yOut, expertIdxOut, softmaxResultOutOptional);

    constexpr aclnnStatus kInvalid = ACLNN_ERR_PARAM_INVALID;
    OPAPI_CHECK(x->dtype == ACL_FLOAT || x->dtype == ACL_FLOAT16 || x->dtype == ACL_BF16, kInvalid,
                "x data type error, only supports float32,half,bf16");
    OPAPI_CHECK(x->dims.size() == 2 || x->dims.size() == 3, kInvalid, "x shape dim(=%zu) is not 2 or 3", x->dims.size());
    const int64_t cols = x->dims.back();
    OPAPI_CHECK(cols != 0, kInvalid, "x shape last dim is zero");
    for (int64_t d : x->dims) OPAPI_CHECK(d <= 2147483647ll, kInvalid, "x shape larger than (=2147483647)");
    int64_t rows = 1;
    for (size_t i = 0; i + 1 < x->dims.size(); ++i) rows *= x->dims[i];
    if (finishedOptional != nullptr) {
        OPAPI_CHECK(finishedOptional->dtype == ACL_BOOL, kInvalid, "finished type error, should be BOOL");
        OPAPI_CHECK(finishedOptional->dims.size() == x->dims.size() - 1, kInvalid,
                    "finished dim num (=%zu) error, should be (=%zu)", finishedOptional->dims.size(), x->dims.size() - 1);
        for (size_t i = 0; i + 1 < x->dims.size(); ++i) {
            OPAPI_CHECK(finishedOptional->dims[i] == x->dims[i], kInvalid, "finished and x shape not equal");
        }
    }
    OPAPI_CHECK(k > 0 && k <= cols, kInvalid, "attr k(=%lld) is wrong. col=%lld", (long long)k, (long long)cols);
    OPAPI_CHECK(k <= kMaxK, kInvalid, "attr k(=%lld) is too large", (long long)k);
    OPAPI_CHECK(renorm == 0 || renorm == 1, kInvalid, "attr renorm(=%lld) is wrong", (long long)renorm);
    OPAPI_CHECK(yOut->dtype == x->dtype, kInvalid, "y data type error, should be same with x data type");
    OPAPI_CHECK(SameButLast(yOut, x, k), kInvalid, "y shape %s must be x's shape %s with last dim k", ShapeStr(yOut).c_str(),
                ShapeStr(x).c_str());
    OPAPI_CHECK(expertIdxOut->dtype == ACL_INT32, kInvalid, "expertIdx data type error, only supports int32");
    OPAPI_CHECK(SameButLast(expertIdxOut, x, k), kInvalid, "expertIdx shape %s must be x's shape %s with last dim k",
                ShapeStr(expertIdxOut).c_str(), ShapeStr(x).c_str());
    const bool wantSoftmax = renorm == 0 && outputSoftmaxResultFlag;
    if (wantSoftmax) {
        OPAPI_CHECK(softmaxResultOutOptional != nullptr, ACLNN_ERR_PARAM_NULLPTR, "softmax is nullptr");
        OPAPI_CHECK(softmaxResultOutOptional->dtype == ACL_FLOAT, kInvalid, "softmax result type error, should be float");
        OPAPI_CHECK(SameButLast(softmaxResultOutOptional, x, cols), kInvalid, "softmaxResult and x shape not equal");
        OPAPI_CHECK(IsContiguous(softmaxResultOutOptional), kInvalid, "softmaxResult must be contiguous");
    }
    OPAPI_CHECK(cols <= kMaxCols, kInvalid, "this build handles at most %lld experts per row", (long long)kMaxCols);
    OPAPI_CHECK(IsContiguous(yOut) && IsContiguous(expertIdxOut), kInvalid,
                "the outputs must be contiguous");  // x and finished may be strided views
    if (rows > 0) {
        OPAPI_CHECK(x->data != nullptr && yOut->data != nullptr && expertIdxOut->data != nullptr, ACLNN_ERR_PARAM_NULLPTR,
                    "x / yOut / expertIdxOut carry no device memory");
        OPAPI_CHECK(finishedOptional == nullptr || finishedOptional->data != nullptr, ACLNN_ERR_PARAM_NULLPTR,
                    "finished carries no device memory");
        OPAPI_CHECK(!wantSoftmax || softmaxResultOutOptional->data != nullptr, ACLNN_ERR_PARAM_NULLPTR,
                    "softmaxResult carries no device memory");
    }

    auto* ex = new (std::nothrow) GatingExecutor();
    OPAPI_CHECK(ex != nullptr, ACLNN_ERR_INNER_CREATE_EXECUTOR, "out of host memory");
    ex->dtype = x->dtype;
    OPAPI_BIND(ex, x, &ex->args.x);
    OPAPI_BIND(ex, finishedOptional, &ex->args.finished);
    ex->args.y = DataPtr(yOut);
    ex->args.expertIdx = reinterpret_cast<int32_t*>(DataPtr(expertIdxOut));
    ex->args.softmaxOut = wantSoftmax ? reinterpret_cast<float*>(DataPtr(softmaxResultOutOptional)) : nullptr;
    ex->args.rows = rows;
    ex->args.cols = static_cast<int32_t>(cols);
    ex->args.k = static_cast<int32_t>(k);
    ex->args.renorm = static_cast<int32_t>(renorm);
    ex->SealWorkspace(0);
    *workspaceSize = ex->workspaceBytes;
    *executor = ex;
    return ACLNN_SUCCESS;
}

extern "C" aclnnStatus aclnnMoeGatingTopKSoftmaxV2(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor,
                                                   aclrtStream stream) {
    return opapi::RunAndRelease(workspace, workspaceSize, executor, stream);
}
