// aclnnMoeFinalizeRoutingV2 for gfx950: weighted top-k un-permute and reduce.
//
// Reference behaviour restated: moe/moe_finalize_routing_v2/op_kernel/moe_finalize_routing_v2_bf16.h:286-609 (bf16 data,
// fp32 accumulation, one RINT cast at the end) and moe_finalize_routing_v2_fp_db.h:265-269,393-440 (fp32 / fp16 data
// combined in their own arithmetic).  Index arrangement by dropPadMode: moe_finalize_routing_v2_bf16.h:361-366.
// Validation follows op_host/moe_finalize_routing_v2_tiling_membase.cpp:182-350.
//
// The reference needs thirteen kernel variants to fit rows into its vector core's local buffer; here it is a single
// bandwidth-bound kernel: a group of lanes owns one token, reads the K gathered rows with 16-byte loads and keeps the
// running sum in registers, adding terms in ascending k with separate multiply and add (no fused multiply-add) so
// that the result does not depend on how the row is split across lanes.
#include "opapi_common.h"

#include <type_traits>

#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>

#include "aclnnop/aclnn_moe_finalize_routing_v2.h"

namespace {

struct FinalizeArgs {
    const void* expandedX;
    const int32_t* expandedRowIdx;
    const void* x1;
    const void* x2;
    const void* bias;
    const void* scales;
    const int32_t* expertIdx;
    void* out;
    int64_t tokens;
    int64_t hidden;
    int64_t expandedRows;  // rows of expandedX viewed as 2-D; indices outside [0, expandedRows) are ignored
    int64_t biasRows;      // rows of bias; an expert id outside [0, biasRows) adds no bias
    int32_t topK;
    int32_t dropPadMode;
};

// Element codecs: Load widens to the arithmetic type, Round applies the storage type's rounding to an intermediate.
struct Bf16Codec {
    using Storage = uint16_t;
    static constexpr bool kRoundEveryOp = false;
    __device__ static float Load(Storage v) { return __uint_as_float(static_cast<uint32_t>(v) << 16); }
    __device__ static Storage Store(float f) {
        uint32_t u = __float_as_uint(f);
        if ((u & 0x7fffffffu) > 0x7f800000u) return static_cast<Storage>((u >> 16) | 0x40);
        u += 0x7fffu + ((u >> 16) & 1u);
        return static_cast<Storage>(u >> 16);
    }
    __device__ static float Round(float f) { return f; }
};
struct F16Codec {
    using Storage = uint16_t;
    static constexpr bool kRoundEveryOp = true;
    __device__ static float Load(Storage v) { return __half2float(__ushort_as_half(v)); }
    __device__ static Storage Store(float f) { return __half_as_ushort(__float2half_rn(f)); }
    __device__ static float Round(float f) { return __half2float(__float2half_rn(f)); }
};
struct F32Codec {
    using Storage = float;
    static constexpr bool kRoundEveryOp = false;
    __device__ static float Load(Storage v) { return v; }
    __device__ static Storage Store(float f) { return f; }
    __device__ static float Round(float f) { return f; }
};

template <typename Codec, int kVec>
struct alignas(sizeof(typename Codec::Storage) * kVec) Packet {
    typename Codec::Storage v[kVec];
};

// acc[0 .. kVec) -> one packet in the storage type.  bf16 pairs go through v_cvt_pk_bf16_f32 (round to nearest even, NaN
// kept quiet: the same values as Bf16Codec::Store element by element, in a fifth of the instructions).
template <typename Codec, int kVec>
__device__ __forceinline__ Packet<Codec, kVec> PackPacket(const float (&acc)[kVec]) {
    Packet<Codec, kVec> o;
    if constexpr (std::is_same<Codec, Bf16Codec>::value && kVec % 2 == 0) {
        typedef float Float2 __attribute__((ext_vector_type(2)));
        typedef __bf16 Bf16x2 __attribute__((ext_vector_type(2)));
#pragma unroll
        for (int i = 0; i < kVec; i += 2) {
            const Float2 f = {acc[i], acc[i + 1]};
            const uint32_t pk = __builtin_bit_cast(uint32_t, __builtin_convertvector(f, Bf16x2));
            o.v[i] = static_cast<uint16_t>(pk & 0xffffu);
            o.v[i + 1] = static_cast<uint16_t>(pk >> 16);
        }
    } else {
#pragma unroll
        for (int i = 0; i < kVec; ++i) o.v[i] = Codec::Store(acc[i]);
    }
    return o;
}

__device__ __forceinline__ float ScaleAt(const void* scales, int64_t i, int scaleIsF32, int dataIsF16) {
    if (scaleIsF32) return static_cast<const float*>(scales)[i];
    const uint16_t raw = static_cast<const uint16_t*>(scales)[i];
    return dataIsF16 ? F16Codec::Load(raw) : Bf16Codec::Load(raw);
}

// kLanesPerToken lanes cooperate on one token; a workgroup of 256 threads handles 256 / kLanesPerToken tokens.
template <typename Codec, int kVec, int kLanesPerToken>
__global__ __launch_bounds__(256) void FinalizeKernel(FinalizeArgs a, int scaleIsF32) {
    using P = Packet<Codec, kVec>;
    const int64_t token = static_cast<int64_t>(blockIdx.x) * (256 / kLanesPerToken) + threadIdx.x / kLanesPerToken;
    if (token >= a.tokens) return;
    const int lane = threadIdx.x % kLanesPerToken;
    const int64_t packets = a.hidden / kVec;
    const bool columnArrangement = a.dropPadMode == 0 || a.dropPadMode == 1;
    const bool skipsAllowed = a.dropPadMode == 1 || a.dropPadMode == 3;
    constexpr int dataIsF16 = Codec::kRoundEveryOp ? 1 : 0;

    // gridDim.y workgroups share a token's row: slice y takes packets y * lanes + lane, + lanes * gridDim.y, ...
    for (int64_t pk = lane + static_cast<int64_t>(blockIdx.y) * kLanesPerToken; pk < packets;
         pk += static_cast<int64_t>(kLanesPerToken) * gridDim.y) {
        float acc[kVec];
        bool init = false;
        if (a.x1 != nullptr) {
            const P p1 = static_cast<const P*>(a.x1)[token * packets + pk];
            if (a.x2 != nullptr) {
                const P p2 = static_cast<const P*>(a.x2)[token * packets + pk];
#pragma unroll
                for (int i = 0; i < kVec; ++i) acc[i] = Codec::Round(__fadd_rn(Codec::Load(p1.v[i]), Codec::Load(p2.v[i])));
            } else {
#pragma unroll
                for (int i = 0; i < kVec; ++i) acc[i] = __fadd_rn(Codec::Load(p1.v[i]), 0.0f);
            }
            init = true;
        } else if (a.x2 != nullptr) {
            const P p2 = static_cast<const P*>(a.x2)[token * packets + pk];
#pragma unroll
            for (int i = 0; i < kVec; ++i) acc[i] = __fadd_rn(Codec::Load(p2.v[i]), 0.0f);
            init = true;
        }
        for (int k = 0; k < a.topK; ++k) {
            const int64_t d = columnArrangement ? a.expandedRowIdx[static_cast<int64_t>(k) * a.tokens + token]
                                                : a.expandedRowIdx[token * a.topK + k];
            if (d < 0 || d >= a.expandedRows) {
                // -1 marks a dropped row in the drop/pad arrangements; any other out-of-range index is ignored for safety
                if (skipsAllowed && !init) {
#pragma unroll
                    for (int i = 0; i < kVec; ++i) acc[i] = 0.0f;
                    init = true;
                }
                continue;
            }
            const float s = a.scales != nullptr ? ScaleAt(a.scales, token * a.topK + k, scaleIsF32, dataIsF16) : 1.0f;
            const P row = static_cast<const P*>(a.expandedX)[d * packets + pk];
            float v[kVec];
#pragma unroll
            for (int i = 0; i < kVec; ++i) v[i] = Codec::Load(row.v[i]);
            if (a.bias != nullptr) {
                const int64_t e = a.expertIdx[token * a.topK + k];
                if (e >= 0 && e < a.biasRows) {  // expert ids are caller data: never index the bias table with a bad one
                    const P b = static_cast<const P*>(a.bias)[e * packets + pk];
#pragma unroll
                    for (int i = 0; i < kVec; ++i) v[i] = Codec::Round(__fadd_rn(v[i], Codec::Load(b.v[i])));
                }
            }
#pragma unroll
            for (int i = 0; i < kVec; ++i) {
                const float t = Codec::Round(__fmul_rn(v[i], s));
                acc[i] = init ? Codec::Round(__fadd_rn(acc[i], t)) : t;
            }
            init = true;
        }
        P o;
#pragma unroll
        for (int i = 0; i < kVec; ++i) o.v[i] = Codec::Store(init ? acc[i] : 0.0f);
        static_cast<P*>(a.out)[token * packets + pk] = o;
    }
}

// The common case -- no bias, at most kMaxK experts per token, 16-byte packets, one packet per lane -- with every load of a
// token's K row indices and weights loaded up front (wave-uniform loads) and the K row packets requested two at a time,
// one pair ahead of the sum, which runs in ascending k with the same separate multiply and add as the general kernel
// (bit-identical results).  The general kernel makes 2 K dependent memory round trips per lane, this one K / 2 + 1.
template <typename Codec, int kVec, int kMaxK>
__global__ __launch_bounds__(256) void FinalizeBatchedKernel(FinalizeArgs a, int scaleIsF32) {
    using P = Packet<Codec, kVec>;
    // consecutive workgroups take the slices of one token: neighbouring pieces of the same K rows are read together
    const int64_t packets = a.hidden / kVec;
    // 32-bit index arithmetic: the grid is tokens x slices workgroups, and a 64-bit division costs a hundred scalar
    // instructions in a kernel whose whole sum is two hundred
    const uint32_t slices = static_cast<uint32_t>((packets + 255) / 256);
    const uint32_t tokenIndex = blockIdx.x / slices;
    const int64_t token = tokenIndex;
    const int64_t pk = static_cast<int64_t>((blockIdx.x - tokenIndex * slices) * 256u + threadIdx.x);
    if (pk >= packets) return;
    const bool columnArrangement = a.dropPadMode == 0 || a.dropPadMode == 1;
    const bool skipsAllowed = a.dropPadMode == 1 || a.dropPadMode == 3;
    constexpr int dataIsF16 = Codec::kRoundEveryOp ? 1 : 0;
    const int topK = a.topK;

    int64_t d[kMaxK];
    float s[kMaxK];
#pragma unroll
    for (int k = 0; k < kMaxK; ++k) {
        d[k] = -1;
        s[k] = 1.0f;
        if (k < topK) {
            d[k] = columnArrangement ? a.expandedRowIdx[static_cast<int64_t>(k) * a.tokens + token]
                                     : a.expandedRowIdx[token * topK + k];
            if (a.scales != nullptr) s[k] = ScaleAt(a.scales, token * topK + k, scaleIsF32, dataIsF16);
        }
    }
    // The plain call -- exactly kMaxK experts per token, every index in range, no skip inputs -- as straight-line code:
    // the general form below spends more instructions on its (wave-uniform) case distinctions than on the sum, and at
    // sixteen bytes per lane that, not the memory system, was what bounded the kernel.
    bool plain = topK == kMaxK && a.x1 == nullptr && a.x2 == nullptr;
#pragma unroll
    for (int k = 0; k < kMaxK; ++k) plain = plain && d[k] >= 0 && d[k] < a.expandedRows;
    if (plain) {
        const P* const x = static_cast<const P*>(a.expandedX) + pk;
        P row[2][2];
        row[0][0] = x[d[0] * packets];
        row[0][1] = x[d[1] * packets];
        float acc[kVec];
#pragma unroll
        for (int k0 = 0; k0 < kMaxK; k0 += 2) {
            const int cur = (k0 >> 1) & 1;
            if (k0 + 2 < kMaxK) {
                row[cur ^ 1][0] = x[d[k0 + 2] * packets];
                row[cur ^ 1][1] = x[d[k0 + 3 < kMaxK ? k0 + 3 : k0 + 2] * packets];
            }
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int k = k0 + j;
                if (k >= kMaxK) continue;
#pragma unroll
                for (int i = 0; i < kVec; ++i) {
                    const float t = Codec::Round(__fmul_rn(Codec::Load(row[cur][j].v[i]), s[k]));
                    acc[i] = k == 0 ? t : Codec::Round(__fadd_rn(acc[i], t));
                }
            }
        }
        static_cast<P*>(a.out)[token * packets + pk] = PackPacket<Codec, kVec>(acc);
        return;
    }
    P p1{}, p2{};
    if (a.x1 != nullptr) p1 = static_cast<const P*>(a.x1)[token * packets + pk];
    if (a.x2 != nullptr) p2 = static_cast<const P*>(a.x2)[token * packets + pk];
    // row packets travel in pairs, the next pair requested before the current one is added
    P row[2][2];
    auto request = [&](int k0, int slot) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int k = k0 + j;
            const bool valid = k < kMaxK && k < topK && d[k < kMaxK ? k : 0] >= 0 && d[k < kMaxK ? k : 0] < a.expandedRows;
            if (valid) row[slot][j] = static_cast<const P*>(a.expandedX)[d[k] * packets + pk];
        }
    };
    request(0, 0);
    float acc[kVec];
    bool init = false;
    if (a.x1 != nullptr && a.x2 != nullptr) {
#pragma unroll
        for (int i = 0; i < kVec; ++i) acc[i] = Codec::Round(__fadd_rn(Codec::Load(p1.v[i]), Codec::Load(p2.v[i])));
        init = true;
    } else if (a.x1 != nullptr || a.x2 != nullptr) {
        const P& only = a.x1 != nullptr ? p1 : p2;
#pragma unroll
        for (int i = 0; i < kVec; ++i) acc[i] = __fadd_rn(Codec::Load(only.v[i]), 0.0f);
        init = true;
    }
#pragma unroll
    for (int k0 = 0; k0 < kMaxK; k0 += 2) {
        if (k0 + 2 < kMaxK) request(k0 + 2, ((k0 >> 1) + 1) & 1);
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int k = k0 + j;
            if (k >= topK) continue;
            if (d[k] < 0 || d[k] >= a.expandedRows) {
                if (skipsAllowed && !init) {
#pragma unroll
                    for (int i = 0; i < kVec; ++i) acc[i] = 0.0f;
                    init = true;
                }
                continue;
            }
#pragma unroll
            for (int i = 0; i < kVec; ++i) {
                const float t = Codec::Round(__fmul_rn(Codec::Load(row[(k0 >> 1) & 1][j].v[i]), s[k]));
                acc[i] = init ? Codec::Round(__fadd_rn(acc[i], t)) : t;
            }
            init = true;
        }
    }
    P o;
#pragma unroll
    for (int i = 0; i < kVec; ++i) o.v[i] = Codec::Store(init ? acc[i] : 0.0f);
    static_cast<P*>(a.out)[token * packets + pk] = o;
}

class FinalizeExecutor : public aclOpExecutor {
   public:
    FinalizeArgs args{};
    aclDataType dtype = ACL_BF16;
    int scaleIsF32 = 0;
    bool vectorOk = false;  // 16-byte packets are usable

    template <typename Codec, int kVec>
    void Launch(hipStream_t stream) {
        const int64_t packets = args.hidden / kVec;
        if (kVec > 1 && args.bias == nullptr && args.topK <= 8 && packets > 64) {
            const unsigned slices = static_cast<unsigned>((packets + 255) / 256);
            hipLaunchKernelGGL((FinalizeBatchedKernel<Codec, kVec, 8>), dim3(static_cast<unsigned>(args.tokens * slices)),
                               dim3(256), 0, stream, args, scaleIsF32);
            return;
        }
        if (packets <= 64) {
            const unsigned blocks = static_cast<unsigned>((args.tokens + 3) / 4);
            hipLaunchKernelGGL((FinalizeKernel<Codec, kVec, 64>), dim3(blocks), dim3(256), 0, stream, args, scaleIsF32);
        } else {
            // one 256-lane slice of the row per workgroup: short rows of work, many of them in flight
            const unsigned slices = static_cast<unsigned>((packets + 255) / 256);
            hipLaunchKernelGGL((FinalizeKernel<Codec, kVec, 256>), dim3(static_cast<unsigned>(args.tokens), slices), dim3(256),
                               0, stream, args, scaleIsF32);
        }
    }

    aclnnStatus Run(void*, hipStream_t stream) override {
        if (args.tokens == 0 || args.hidden == 0) return ACLNN_SUCCESS;
        opapi::KernelTimer timer("finalize", stream);
        if (dtype == ACL_BF16) {
            if (vectorOk) Launch<Bf16Codec, 8>(stream); else Launch<Bf16Codec, 1>(stream);
        } else if (dtype == ACL_FLOAT16) {
            if (vectorOk) Launch<F16Codec, 8>(stream); else Launch<F16Codec, 1>(stream);
        } else {
            if (vectorOk) Launch<F32Codec, 4>(stream); else Launch<F32Codec, 1>(stream);
        }
        return ACLNN_SUCCESS;
    }
};

}  // namespace

extern "C" aclnnStatus aclnnMoeFinalizeRoutingV2GetWorkspaceSize(
    const aclTensor* expandedX, const aclTensor* expandedRowIdx, const aclTensor* x1Optional,
    const aclTensor* x2Optional, const aclTensor* biasOptional, const aclTensor* scalesOptional,
    const aclTensor* expertIdxOptional, int64_t dropPadMode, const aclTensor* out, uint64_t* workspaceSize,
    aclOpExecutor** executor) {
    using namespace opapi;
    ClearError();
    OPAPI_CHECK_NOTNULL(expandedX, "expandedX");
    OPAPI_CHECK_NOTNULL(expandedRowIdx, "expandedRowIdx");
    OPAPI_CHECK_NOTNULL(out, "out");
    OPAPI_CHECK_NOTNULL(workspaceSize, "workspaceSize");
    OPAPI_CHECK_NOTNULL(executor, "executor");
    OPAPI_CHECK_EXTENTS(expandedX, expandedRowIdx, x1Optional, x2Optional, biasOptional, scalesOptional, expertIdxOptional, out);
    constexpr aclnnStatus kInvalid = ACLNN_ERR_PARAM_INVALID;

    const aclDataType dt = expandedX->dtype;
    OPAPI_CHECK(dt == ACL_FLOAT || dt == ACL_FLOAT16 || dt == ACL_BF16, kInvalid,
                "expandedX dtype %d is not supported (FLOAT, FLOAT16, BF16)", (int)dt);
    OPAPI_CHECK(expandedRowIdx->dtype == ACL_INT32, kInvalid, "expandedRowIdx must be INT32");
    OPAPI_CHECK(dropPadMode >= 0 && dropPadMode <= 3, kInvalid, "the value of drop_pad_mode should be [0,3].");
    OPAPI_CHECK(expandedRowIdx->dims.size() == 1, kInvalid, "the expanded_row_idx of input should be 1D tensor.");
    const int64_t nk = expandedRowIdx->dims[0];
    int64_t k = 1;
    if (scalesOptional != nullptr) {
        OPAPI_CHECK(scalesOptional->dims.size() == 2, kInvalid, "the scales of input should be 2D tensor.");
        k = scalesOptional->dims[1];
        OPAPI_CHECK(k != 0, kInvalid, "K can not be 0.");
        OPAPI_CHECK(scalesOptional->dtype == dt || (scalesOptional->dtype == ACL_FLOAT && dt == ACL_BF16), kInvalid,
                    "scales dtype must equal expandedX dtype (or FLOAT with BF16 data)");
    }
    const int64_t n = nk / k;
    int64_t e = 0, h = 0;
    if (dropPadMode == 0 || dropPadMode == 2) {
        OPAPI_CHECK(expandedX->dims.size() == 2, kInvalid,
                    "the expanded_x of input should be 2D tensor when drop_pad_mode is 0 or 2.");
        h = expandedX->dims[1];
    } else {
        OPAPI_CHECK(expandedX->dims.size() == 3, kInvalid,
                    "the expanded_x of input should be 3D tensor when drop_pad_mode is 1 or 3.");
        e = expandedX->dims[0];
        h = expandedX->dims[2];
    }
    if (scalesOptional != nullptr) {
        OPAPI_CHECK(scalesOptional->dims[0] == n, kInvalid, "the dim 0 of scales should be %lld.", (long long)n);
    }
    auto checkSkip = [&](const aclTensor* t, const char* name) -> aclnnStatus {
        OPAPI_CHECK(t->dims.size() == 2, kInvalid, "the %s of input should be 2D tensor.", name);
        OPAPI_CHECK(t->dims[0] == n, kInvalid, "the dim 0 of %s should be %lld.", name, (long long)n);
        OPAPI_CHECK(t->dims[1] == h, kInvalid, "the dim 1 of %s should be %lld.", name, (long long)h);
        OPAPI_CHECK(t->dtype == dt, kInvalid, "the dtype of %s should be same with expanded_x.", name);
        return ACLNN_SUCCESS;
    };
    if (x1Optional != nullptr) {
        aclnnStatus st = checkSkip(x1Optional, "x1");
        if (st != ACLNN_SUCCESS) return st;
    }
    if (x2Optional != nullptr) {
        OPAPI_CHECK(x1Optional != nullptr, kInvalid,
                    "In the case of x1 parameter is not input, x2 parameter can't be inputted either.");
        aclnnStatus st = checkSkip(x2Optional, "x2");
        if (st != ACLNN_SUCCESS) return st;
    }
    if (biasOptional != nullptr) {
        OPAPI_CHECK(expertIdxOptional != nullptr, kInvalid, "the expert_idx must exist when bias exist.");
        OPAPI_CHECK(biasOptional->dims.size() == 2, kInvalid, "the bias of input should be 2D tensor.");
        if (dropPadMode == 1 || dropPadMode == 3) {
            OPAPI_CHECK(biasOptional->dims[0] == e, kInvalid, "the dim 0 of bias should be %lld when drop_pad_mode is 1 or 3.",
                        (long long)e);
        }
        OPAPI_CHECK(biasOptional->dims[1] == h, kInvalid, "the dim 1 of bias should be %lld.", (long long)h);
        OPAPI_CHECK(biasOptional->dtype == dt, kInvalid, "the dtype of bias should be same with expanded_x.");
    }
    if (expertIdxOptional != nullptr) {
        OPAPI_CHECK(expertIdxOptional->dims.size() == 2, kInvalid, "the expert_idx of input should be 2D tensor.");
        OPAPI_CHECK(expertIdxOptional->dims[0] == n, kInvalid, "the dim 0 of expert_idx should be %lld.", (long long)n);
        OPAPI_CHECK(expertIdxOptional->dims[1] == k, kInvalid, "the dim 1 of expert_idx should be %lld.", (long long)k);
        OPAPI_CHECK(expertIdxOptional->dtype == ACL_INT32, kInvalid, "expert_idx must be INT32");
    }
    if (biasOptional != nullptr && expertIdxOptional != nullptr) {
        OPAPI_CHECK(biasOptional->dims[0] >= expertIdxOptional->dims[1], kInvalid, "E should be larger than or equal to K.");
        OPAPI_CHECK(biasOptional->dims[0] != 0, kInvalid, "E can not be 0.");
    }
    OPAPI_CHECK(out->dims.size() == 2, kInvalid, "the y should be 2D tensor.");
    OPAPI_CHECK(out->dtype == dt, kInvalid, "the dtype of y should be same with expanded_x.");
    OPAPI_CHECK(out->dims[0] == n, kInvalid, "the dim 0 of output should be %lld.", (long long)n);
    OPAPI_CHECK(out->dims[1] == h, kInvalid, "the dim 1 of output should be %lld.", (long long)h);
    const aclTensor* all[] = {expandedX, expandedRowIdx, x1Optional, x2Optional, biasOptional, scalesOptional,
                              expertIdxOptional, out};
    for (const aclTensor* t : all) {
        if (t == nullptr) continue;
        OPAPI_CHECK(t != out || IsContiguous(t), kInvalid, "out must be contiguous");  // inputs may be strided views
        OPAPI_CHECK(Numel(t) == 0 || t->data != nullptr, ACLNN_ERR_PARAM_NULLPTR, "a tensor carries no device memory");
    }

    auto* ex = new (std::nothrow) FinalizeExecutor();
    OPAPI_CHECK(ex != nullptr, ACLNN_ERR_INNER_CREATE_EXECUTOR, "out of host memory");
    ex->dtype = dt;
    ex->scaleIsF32 = (scalesOptional != nullptr && scalesOptional->dtype == ACL_FLOAT) ? 1 : 0;
    FinalizeArgs& a = ex->args;
    OPAPI_BIND(ex, expandedX, &a.expandedX);
    OPAPI_BIND(ex, expandedRowIdx, &a.expandedRowIdx);
    OPAPI_BIND(ex, x1Optional, &a.x1);
    OPAPI_BIND(ex, x2Optional, &a.x2);
    OPAPI_BIND(ex, biasOptional, &a.bias);
    OPAPI_BIND(ex, scalesOptional, &a.scales);
    OPAPI_BIND(ex, expertIdxOptional, &a.expertIdx);
    a.out = DataPtr(out);
    a.tokens = n;
    a.hidden = h;
    a.expandedRows = h > 0 ? Numel(expandedX) / h : 0;
    a.biasRows = biasOptional != nullptr ? biasOptional->dims[0] : 0;
    a.topK = static_cast<int32_t>(k);
    a.dropPadMode = static_cast<int32_t>(dropPadMode);
    const int vec = dt == ACL_FLOAT ? 4 : 8;
    uintptr_t align = reinterpret_cast<uintptr_t>(a.expandedX) | reinterpret_cast<uintptr_t>(a.out) |
                      reinterpret_cast<uintptr_t>(a.x1) | reinterpret_cast<uintptr_t>(a.x2) |
                      reinterpret_cast<uintptr_t>(a.bias);
    ex->vectorOk = (h % vec == 0) && (align % 16 == 0);
    ex->SealWorkspace(0);
    *workspaceSize = ex->workspaceBytes;
    *executor = ex;
    return ACLNN_SUCCESS;
}

extern "C" aclnnStatus aclnnMoeFinalizeRoutingV2(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor,
                                                 aclrtStream stream) {
    return opapi::RunAndRelease(workspace, workspaceSize, executor, stream);
}
