/*
 * CPU oracle for the quantized MoE expert-FFN path.  TEST INFRASTRUCTURE ONLY.
 *
 * A plain-C restatement (OpenMP over rows) of the numerics of the four reference operators on the path:
 *   MoeInitRoutingV2 -> GroupedMatmulSwigluQuant -> GroupedMatmul (int8 down projection) -> MoeFinalizeRoutingV2,
 * and of the operators around it that the library also provides: MoeGatingTopKSoftmaxV2, MoeInitRoutingV3 (with and
 * without dynamic quantisation), MoeInitRoutingQuantV2 and GroupedMatmulFinalizeRouting.
 * It exists to check the HIP kernels and to be timed as the CPU baseline.  Nothing in the shipped library links,
 * loads or calls it; only the test-suite, the smoke check and the benchmark's cpu_baseline leg may.
 *
 * The reference kernels are Ascend C and need the CANN toolkit (headers and the tikicpulib simulator), which is not
 * part of the reference repository, so no reference binary can be built; each function below cites the reference
 * lines it restates.
 *
 * How each function is pinned (tests/test_oracle_*.py):
 *   routing        : numpy argsort(kind="stable") + bincount; brute force; the drop/pad example literal
 *                    (moe/moe_init_routing_v2/examples/test_aclnn_moe_init_routing_v2.cpp:71-96).
 *   int32 GEMMs    : exact float64 BLAS matmul per group (|acc| < 2^53).
 *   fp16/bf16 casts: exhaustive / randomized comparison with numpy float16 and torch bfloat16.
 *   SwiGLU+requant : float64 evaluation within tolerance, invariants (max|q| == 127, scale == max/127).
 *                    PARITY UNPINNED at the last-ulp level: the reference's SwiGLU exp/divide rounding lives in the
 *                    CANN library and no reference test holds expected numbers for this op.
 *   down epilogue  : closed form in numpy/torch (two fp32 multiplies, RNE cast).
 *   finalize       : numpy fp32 closed form; example literal
 *                    (moe/moe_finalize_routing_v2/examples/test_aclnn_moe_finalize_routing_v2.cpp:102-110);
 *                    column/row arrangement equivalence; the reference generator's shapes.
 *   gating         : float64 numpy softmax + stable descending argsort; closed form of the example's input
 *                    (moe/moe_gating_top_k_softmax_v2/examples/test_aclnn_moe_gating_top_k_softmax_v2.cpp:93); the
 *                    ties-away narrowing against every half-precision midpoint.
 *                    PARITY UNPINNED at the last-ulp level and in the order among equal values: SoftMax, TopK and
 *                    Sort32 live in the CANN library and the reference holds no numbers for this operator.
 *   routing V3     : numpy stable argsort of the in-range positions; equality with the V2 function on the whole
 *                    range; dynamic quantisation against a numpy restatement bit for bit.
 *   routing QuantV2: static mode against numpy float16 arithmetic bit for bit (saturation and ties included); dynamic
 *                    mode against the V3 function on the whole range; the example's literals
 *                    (moe/moe_init_routing_quant_v2/examples/test_aclnn_moe_init_routing_quant_v2.cpp:71-108).
 *   fused combine  : float64 numpy (exact matmul per group + np.add.at); equality with "dequantise, then scatter".
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORACLE_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------------------------------------ casts */

static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

/* bf16 <-> fp32, round to nearest even (CAST_RINT, grouped_matmul_quant_mixcore.h:282, moe_finalize_routing_v2_bf16.h:593). */
static inline float bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }
static inline uint16_t f32_to_bf16(float f) {
    uint32_t u = f2u(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40); /* NaN stays NaN */
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

static inline float f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    if (exp == 0) {
        if (man == 0) return u2f(sign);
        float v = (float)man * 0x1p-24f; /* subnormal: man * 2^-24, exact */
        return sign ? -v : v;
    }
    if (exp == 31) return u2f(sign | 0x7f800000u | (man << 13));
    return u2f(sign | ((exp + 112u) << 23) | (man << 13));
}

/* fp32 -> fp16, round to nearest even, overflow to inf, gradual underflow. */
static inline uint16_t f32_to_f16(float f) {
    uint32_t u = f2u(f);
    uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    uint32_t a = u & 0x7fffffffu;
    if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);
    if (a >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u); /* >= 65520 rounds to inf */
    if (a < 0x38800000u) {                                   /* below 2^-14: subnormal half */
        if (a < 0x33000000u) return sign;                    /* below 2^-25 -> 0 (2^-25 itself ties to even 0) */
        uint32_t e = a >> 23;
        uint32_t m = (a & 0x7fffffu) | 0x800000u;
        uint32_t shift = 126u - e; /* result = m >> shift in units of 2^-24 */
        uint32_t q = m >> shift;
        uint32_t rem = m & ((1u << shift) - 1u);
        uint32_t half = 1u << (shift - 1u);
        if (rem > half || (rem == half && (q & 1u))) q++;
        return (uint16_t)(sign | q);
    }
    uint32_t r = a + 0xfffu + ((a >> 13) & 1u);
    return (uint16_t)(sign | ((r - 0x38000000u) >> 13));
}

ORACLE_API void oracle_f32_to_bf16(const float* in, uint16_t* out, int64_t n) {
    for (int64_t i = 0; i < n; i++) out[i] = f32_to_bf16(in[i]);
}
ORACLE_API void oracle_f32_to_f16(const float* in, uint16_t* out, int64_t n) {
    for (int64_t i = 0; i < n; i++) out[i] = f32_to_f16(in[i]);
}
ORACLE_API void oracle_f16_to_f32(const uint16_t* in, float* out, int64_t n) {
    for (int64_t i = 0; i < n; i++) out[i] = f16_to_f32(in[i]);
}
ORACLE_API void oracle_bf16_to_f32(const uint16_t* in, float* out, int64_t n) {
    for (int64_t i = 0; i < n; i++) out[i] = bf16_to_f32(in[i]);
}

enum { DT_F32 = 0, DT_F16 = 1, DT_BF16 = 27 }; /* ge::DataType codes */

static inline float load_as_f32(const void* p, int64_t i, int dt) {
    if (dt == DT_F32) return ((const float*)p)[i];
    if (dt == DT_F16) return f16_to_f32(((const uint16_t*)p)[i]);
    return bf16_to_f32(((const uint16_t*)p)[i]);
}
static inline void store_from_f32(void* p, int64_t i, int dt, float v) {
    if (dt == DT_F32) ((float*)p)[i] = v;
    else if (dt == DT_F16) ((uint16_t*)p)[i] = f32_to_f16(v);
    else ((uint16_t*)p)[i] = f32_to_bf16(v);
}

/* ------------------------------------------------------------------------------------------------ gating */

/* fp32 -> 16-bit with ties away from zero (Ascend C RoundMode::CAST_ROUND), done on the magnitude bits. */
static inline uint16_t f32_to_bf16_away(float f) {
    uint32_t u = f2u(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
    return (uint16_t)((u + 0x8000u) >> 16);
}
static inline uint16_t f32_to_f16_away(float f) {
    const uint32_t u = f2u(f), sign = (u >> 16) & 0x8000u, mag = u & 0x7fffffffu;
    if (mag > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);
    if (mag >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);            /* >= 65520: beyond the largest half */
    const int32_t e = (int32_t)(mag >> 23) - 127;
    if (e < -25) return (uint16_t)sign;                                   /* below half of the smallest subnormal */
    uint32_t m = (mag & 0x7fffffu) | 0x800000u;                           /* 24-bit significand, value = m * 2^(e-23) */
    /* target unit: 2^-24 for subnormals (e < -14), 2^(e-10) for normals */
    const int shift = e < -14 ? (-24 - (e - 23)) : 13;                     /* bits dropped from m */
    uint32_t q = (m + (1u << (shift - 1))) >> shift;                       /* add half, truncate: ties go outward */
    if (e < -14) return (uint16_t)(sign | q);                              /* q may reach 0x400 = smallest normal */
    /* q in [0x400, 0x800]; 0x800 carries into the exponent */
    return (uint16_t)(sign | (((uint32_t)(e + 15) << 10) + (q - 0x400u)));
}
ORACLE_API void oracle_f32_to_f16_away(const float* in, uint16_t* out, int64_t n) {
    for (int64_t i = 0; i < n; i++) out[i] = f32_to_f16_away(in[i]);
}
ORACLE_API void oracle_f32_to_bf16_away(const float* in, uint16_t* out, int64_t n) {
    for (int64_t i = 0; i < n; i++) out[i] = f32_to_bf16_away(in[i]);
}

/* MoeGatingTopKSoftmaxV2 (moe/moe_gating_top_k_softmax_v2/README.md:12-30).
 *   renorm 0 : p = softmax(x) (x widened to fp32, max subtracted, exp, sum, divide:
 *              op_kernel/moe_gating_top_k_softmax_v2_ek_fullload.h:309-412); top-k of p, descending, equal values by
 *              ascending index; softmaxOut = p when given
 *   renorm 1 : top-k of x, then softmax over the k picked values (:414-545)
 *   y is narrowed to x's dtype with ties away from zero (CAST_ROUND, :211-262)
 *   finished[row] != 0 : every index of the row becomes cols (op_kernel/moe_gating_top_k_softmax_v2_perf.h:603-637)
 * The exp/sum arithmetic and the order among equal values live in the CANN library (SoftMax, TopK, Sort32): the
 * last-ulp behaviour here is this restatement's own. */
ORACLE_API void oracle_moe_gating_top_k_softmax_v2(const void* x, int dtype, const uint8_t* finished, int64_t rows,
                                                   int64_t cols, int64_t k, int64_t renorm, void* y, int32_t* idx,
                                                   float* softmaxOut) {
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; r++) {
        float* v = (float*)malloc(sizeof(float) * (size_t)cols);
        char* taken = (char*)calloc((size_t)cols, 1);
        float* picked = (float*)malloc(sizeof(float) * (size_t)k);
        for (int64_t c = 0; c < cols; c++) v[c] = load_as_f32(x, r * cols + c, dtype);
        if (renorm == 0) {
            float mx = v[0];
            double wide = 0.0;   /* the sum of the fp32 terms, rounded once: independent of any reduction order */
            for (int64_t c = 1; c < cols; c++) mx = v[c] > mx ? v[c] : mx;
            for (int64_t c = 0; c < cols; c++) { v[c] = expf(v[c] - mx); wide += v[c]; }
            const float sum = (float)wide;
            for (int64_t c = 0; c < cols; c++) { v[c] = v[c] / sum; if (softmaxOut) softmaxOut[r * cols + c] = v[c]; }
        }
        for (int64_t j = 0; j < k; j++) {                       /* selection: first strictly greater wins */
            int64_t best = -1;
            for (int64_t c = 0; c < cols; c++) {
                if (!taken[c] && (best < 0 || v[c] > v[best])) best = c;
            }
            taken[best] = 1;
            picked[j] = v[best];
            idx[r * k + j] = (finished && finished[r]) ? (int32_t)cols : (int32_t)best;
        }
        if (renorm == 1) {
            double wide = 0.0;
            const float mx = picked[0];
            for (int64_t j = 0; j < k; j++) { picked[j] = expf(picked[j] - mx); wide += picked[j]; }
            const float sum = (float)wide;
            for (int64_t j = 0; j < k; j++) picked[j] = picked[j] / sum;
        }
        for (int64_t j = 0; j < k; j++) {
            if (dtype == DT_F32) ((float*)y)[r * k + j] = picked[j];
            else if (dtype == DT_F16) ((uint16_t*)y)[r * k + j] = f32_to_f16_away(picked[j]);
            else ((uint16_t*)y)[r * k + j] = f32_to_bf16_away(picked[j]);
        }
        free(v); free(taken); free(picked);
    }
}

/* ------------------------------------------------------------------------------------------------ routing */

/*
 * MoeInitRoutingV2.
 *   sort        : stable ascending by expert id over the row-major flattening of expertIdx[T,K]
 *                 (moe_v2_sort_one_core.h:64-113; stability per the golden, moe_init_routing_quant_v2_data/gen_data.py:38-39)
 *   inverse map : expandedRowIdx[order[d]] = d                         (moe_v2_src_to_dst_op.h:92-108)
 *   drop/pad    : rank r within expert; r < C ? e*C + r : -1; unused capacity rows zero
 *                 (moe_v2_src_to_dst_with_capacity.h:113-194)
 *   counts      : hist over [0,E); flag 1 -> inclusive cumsum, flag 2 -> hist; drop mode + beforeCapacity -> hist
 *                 (moe_v2_expert_token_out.h:125-280)
 *   gather      : expandedX[dst,:] = x[i / K,:], skipping dst == -1 and dst >= activeRows
 *                 (moe_v2_gather_out.h:87-138; activeRows = activeNum == 0 ? M : min(M, activeNum),
 *                  moe_init_routing_v2_tiling.cpp:152-154)
 * x is handled as opaque rows of rowBytes bytes.  Outputs that a mode does not write may be NULL.
 * Returns 0, or -1 on an expert id outside [0, E) when E > 0 (the reference leaves that undefined).
 */
ORACLE_API int oracle_moe_init_routing_v2(const void* x, int64_t rowBytes, const int32_t* expertIdx, int64_t T, int64_t K,
                                          int64_t activeNum, int64_t capacity, int64_t expertNum, int64_t dropPadMode,
                                          int64_t countFlag, int beforeCapacityFlag, void* expandedX,
                                          int32_t* expandedRowIdx, int32_t* countOrCumsum, int32_t* beforeCapacity) {
    const int64_t M = T * K;
    if (dropPadMode == 1) countFlag = 0; else beforeCapacityFlag = 0;
    int64_t* order = (int64_t*)malloc(sizeof(int64_t) * (size_t)(M > 0 ? M : 1));
    /* stable counting sort when the id range is known, otherwise a stable merge-free insertion via qsort on (key, index) */
    int32_t kmin = 0, kmax = -1;
    for (int64_t i = 0; i < M; i++) {
        if (i == 0) { kmin = kmax = expertIdx[0]; }
        if (expertIdx[i] < kmin) kmin = expertIdx[i];
        if (expertIdx[i] > kmax) kmax = expertIdx[i];
    }
    if (M > 0 && expertNum > 0 && (kmin < 0 || kmax >= expertNum)) { free(order); return -1; }
    const int64_t range = (M > 0) ? ((int64_t)kmax - kmin + 1) : 1;
    int64_t* start = (int64_t*)calloc((size_t)range + 1, sizeof(int64_t));
    for (int64_t i = 0; i < M; i++) start[(int64_t)expertIdx[i] - kmin + 1]++;
    for (int64_t r = 0; r < range; r++) start[r + 1] += start[r];
    int64_t* cursor = (int64_t*)malloc(sizeof(int64_t) * (size_t)range);
    memcpy(cursor, start, sizeof(int64_t) * (size_t)range);
    for (int64_t i = 0; i < M; i++) order[cursor[(int64_t)expertIdx[i] - kmin]++] = i; /* ascending i => stable */

    if (expertNum > 0 && (countFlag > 0 || beforeCapacityFlag)) {
        int64_t run = 0;
        for (int64_t e = 0; e < expertNum; e++) {
            int64_t r = e - kmin;
            int64_t h = (M > 0 && r >= 0 && r < range) ? start[r + 1] - start[r] : 0;
            run += h;
            if (countFlag == 1 && countOrCumsum) countOrCumsum[e] = (int32_t)run;
            if (countFlag == 2 && countOrCumsum) countOrCumsum[e] = (int32_t)h;
            if (beforeCapacityFlag && beforeCapacity) beforeCapacity[e] = (int32_t)h;
        }
    }

    if (dropPadMode == 0) {
        const int64_t activeRows = (activeNum == 0) ? M : (activeNum < M ? activeNum : M);
        for (int64_t d = 0; d < M; d++) expandedRowIdx[order[d]] = (int32_t)d;
        for (int64_t i = 0; i < M; i++) {
            int64_t d = expandedRowIdx[i];
            if (d < activeRows && expandedX && rowBytes > 0)
                memcpy((char*)expandedX + d * rowBytes, (const char*)x + (i / K) * rowBytes, (size_t)rowBytes);
        }
    } else {
        if (expandedX && rowBytes > 0) memset(expandedX, 0, (size_t)(expertNum * capacity * rowBytes));
        for (int64_t d = 0; d < M; d++) {
            int64_t i = order[d];
            int64_t e = expertIdx[i];
            int64_t r = d - start[e - kmin];
            if (r < capacity) {
                int64_t dst = e * capacity + r;
                expandedRowIdx[i] = (int32_t)dst;
                if (expandedX && rowBytes > 0)
                    memcpy((char*)expandedX + dst * rowBytes, (const char*)x + (i / K) * rowBytes, (size_t)rowBytes);
            } else {
                expandedRowIdx[i] = -1;
            }
        }
    }
    free(order); free(start); free(cursor);
    return 0;
}

/* MoeInitRoutingV3, dropless, no quantisation (moe/moe_init_routing_v3/README.md:12-66;
 * op_kernel/moe_v3_gather_out.h:213-231 row and scale gather; op_kernel/moe_v3_expert_tokens_count.h:254-269 counts).
 * Rows whose expert lies in [start, end) are sorted (stable) by expert and packed from destination 0; the others are
 * dropped.  rowIdxType 1: idx[source] = destination (-1 when dropped; the reference leaves those uninitialised);
 * rowIdxType 0: idx[destination] = source for the packed rows, -1 behind them.
 * countMode 0 cumsum, 1 count (int64 [end-start]); 2 key/value pairs of the non-empty experts, zero-filled, written
 * for min(end-start+1, expertNum) pairs.  Untouched output rows keep their previous contents. */
ORACLE_API int oracle_moe_init_routing_v3(const void* x, int64_t rowBytes, const int32_t* expertIdx, const float* scale,
                                          int64_t T, int64_t K, int64_t expertNum, int64_t start, int64_t end,
                                          int64_t countMode, int64_t rowIdxType, void* expandedX, int32_t* idxOut,
                                          int64_t* counts, float* expandedScale) {
    const int64_t M = T * K, active = end - start;
    int64_t* hist = (int64_t*)calloc((size_t)active + 1, sizeof(int64_t));
    for (int64_t i = 0; i < M; i++) {
        const int64_t e = expertIdx[i];
        if (e >= start && e < end) hist[e - start + 1]++;
    }
    if (countMode == 2) {
        const int64_t pairs = (active + 1 < expertNum) ? active + 1 : expertNum;
        memset(counts, 0, sizeof(int64_t) * 2 * (size_t)pairs);
        int64_t slot = 0;
        for (int64_t e = 0; e < active; e++) {
            if (hist[e + 1] != 0 && slot < pairs) { counts[2 * slot] = start + e; counts[2 * slot + 1] = hist[e + 1]; slot++; }
        }
    }
    int64_t run = 0;
    for (int64_t e = 0; e < active; e++) {
        run += hist[e + 1];
        if (countMode == 0) counts[e] = run;
        if (countMode == 1) counts[e] = hist[e + 1];
    }
    for (int64_t e = 0; e < active; e++) hist[e + 1] += hist[e];   /* hist[e] = first destination of expert start+e */
    for (int64_t i = 0; i < M; i++) idxOut[i] = -1;
    for (int64_t i = 0; i < M; i++) {                                /* ascending source index => stable */
        const int64_t e = expertIdx[i];
        if (e < start || e >= end) continue;
        const int64_t d = hist[e - start]++;
        if (rowIdxType == 1) idxOut[i] = (int32_t)d; else idxOut[d] = (int32_t)i;
        if (expandedX && rowBytes > 0) memcpy((char*)expandedX + d * rowBytes, (const char*)x + (i / K) * rowBytes, (size_t)rowBytes);
        if (scale && expandedScale) expandedScale[d] = scale[i / K];
    }
    free(hist);
    return 0;
}

/* fp32 -> fp16 toward zero (Ascend C CAST_TRUNC), on the magnitude bits; the result decoded back to fp32. */
static inline float f32_to_f16_trunc_value(float f) {
    const uint32_t u = f2u(f), sign = u & 0x80000000u, mag = u & 0x7fffffffu;
    if (mag >= 0x7f800000u) return f;                                      /* inf / nan pass through */
    if (mag >= 0x477fe000u) return u2f(sign | 0x477fe000u);                /* beyond 65504: clamp to the largest half */
    const int32_t e = (int32_t)(mag >> 23) - 127;
    if (e < -24) return u2f(sign);                                          /* below the smallest subnormal */
    const int drop = e < -14 ? 13 + (-14 - e) : 13;                         /* mantissa bits a half cannot hold */
    const uint32_t m = (mag & 0x7fffffu) | 0x800000u;
    const uint32_t kept = (m >> drop) << drop;                              /* chop */
    if (kept == 0) return u2f(sign);
    /* rebuild: value = kept * 2^(e-23) */
    return u2f(sign | f2u(ldexpf((float)kept, e - 23)));
}

/* MoeInitRoutingV3 with dynamic quantisation (quantMode 1): routing as oracle_moe_init_routing_v3, and per routed row
 *   v = float(x[token,:]) * smooth[expert - start,:] (smooth optional);  s = max|v| / 127;  q = v / s (true divide);
 *   expandedX[dst,:] = int8(round-half-away(fp16-toward-zero(q)));  expandedScale[dst] = s
 * (moe/moe_init_routing_v3/op_kernel/moe_v3_gather_dynamic_quant.h:103-141).  A row of zeros: s = 0, zeros (the
 * reference computes 0/0 there). */
ORACLE_API int oracle_moe_init_routing_v3_quant(const void* x, int dtype, int64_t cols, const int32_t* expertIdx,
                                                const float* smooth, int64_t T, int64_t K, int64_t expertNum, int64_t start,
                                                int64_t end, int64_t countMode, int64_t rowIdxType, int8_t* expandedX,
                                                int32_t* idxOut, int64_t* counts, float* expandedScale) {
    const int64_t M = T * K;
    int32_t* scatter = (int32_t*)malloc(sizeof(int32_t) * (size_t)(M > 0 ? M : 1));
    oracle_moe_init_routing_v3(NULL, 0, expertIdx, NULL, T, K, expertNum, start, end, countMode, 1, NULL, scatter, counts, NULL);
    if (rowIdxType == 0) for (int64_t i = 0; i < M; i++) idxOut[i] = -1;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < M; i++) {
        const int64_t d = scatter[i];
        if (rowIdxType == 1) idxOut[i] = (int32_t)d;
        if (d < 0) continue;
        if (rowIdxType == 0) idxOut[d] = (int32_t)i;
        const float* sm = smooth ? smooth + (expertIdx[i] - start) * cols : NULL;
        float mx = 0.f;
        for (int64_t c = 0; c < cols; c++) {
            float v = load_as_f32(x, (i / K) * cols + c, dtype);
            if (sm) v = v * sm[c];
            mx = fabsf(v) > mx ? fabsf(v) : mx;
        }
        const float s = mx / 127.0f;
        expandedScale[d] = s;
        for (int64_t c = 0; c < cols; c++) {
            float v = load_as_f32(x, (i / K) * cols + c, dtype);
            if (sm) v = v * sm[c];
            float r = mx == 0.f ? 0.f : roundf(f32_to_f16_trunc_value(v / s));   /* roundf: halves away from zero */
            r = r > 127.f ? 127.f : (r < -128.f ? -128.f : r);
            expandedX[d * cols + c] = (int8_t)r;
        }
    }
    free(scatter);
    return 0;
}

ORACLE_API void oracle_f32_to_f16_trunc_value(const float* in, float* out, int64_t n) {
    for (int64_t i = 0; i < n; i++) out[i] = f32_to_f16_trunc_value(in[i]);
}

/* MoeInitRoutingQuantV2: the routing of oracle_moe_init_routing_v2 with the gathered rows quantised to int8.
 *   quantMode 0 (static, moe/moe_init_routing_quant_v2/op_kernel/moe_v2_gather_quant.h:93-133): every step in half
 *     precision, each rounding to nearest even: h = half(x); h = h * half(scale); h = h + half(offset);
 *     y = int8(rint(h)), saturated.  (A half product or sum formed in fp32 and rounded to half once more equals the
 *     directly rounded half result: fp32 carries 24 >= 2 * 11 + 2 significand bits.)
 *   quantMode 1 (dynamic, op_kernel/moe_v2_gather_dynamic_quant.h:120-155): as oracle_moe_init_routing_v3_quant;
 *     smooth is [smoothRows, cols] with smoothRows 1 (one row for all experts) or expertNum.
 * Drop/pad mode: unused capacity rows are zero with scale 0.  Rows at or beyond activeRows are not written. */
ORACLE_API int oracle_moe_init_routing_quant_v2(const void* x, int dtype, int64_t cols, const int32_t* expertIdx, int64_t T,
                                                int64_t K, int64_t activeNum, int64_t capacity, int64_t expertNum,
                                                int64_t dropPadMode, int64_t countFlag, int beforeCapacityFlag,
                                                int64_t quantMode, const float* scale, const float* offset,
                                                int64_t smoothRows, int8_t* expandedX, int32_t* expandedRowIdx,
                                                int32_t* countOrCumsum, int32_t* beforeCapacity, float* dynScale) {
    const int64_t M = T * K;
    const int rc = oracle_moe_init_routing_v2(NULL, 0, expertIdx, T, K, activeNum, capacity, expertNum, dropPadMode, countFlag,
                                              beforeCapacityFlag, NULL, expandedRowIdx, countOrCumsum, beforeCapacity);
    if (rc != 0) return rc;
    const int64_t limit = dropPadMode == 1 ? expertNum * capacity : (activeNum == 0 ? M : (activeNum < M ? activeNum : M));
    if (dropPadMode == 1) {
        memset(expandedX, 0, (size_t)(limit * cols));
        if (quantMode == 1) for (int64_t d = 0; d < limit; d++) dynScale[d] = 0.f;
    }
    const float hs = quantMode == 0 ? f16_to_f32(f32_to_f16(scale[0])) : 0.f;
    const float ho = quantMode == 0 ? f16_to_f32(f32_to_f16(offset[0])) : 0.f;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < M; i++) {
        const int64_t d = expandedRowIdx[i];
        if (d < 0 || d >= limit) continue;
        const void* row = x;
        const int64_t base = (i / K) * cols;
        if (quantMode == 0) {
            for (int64_t c = 0; c < cols; c++) {
                float h = f16_to_f32(f32_to_f16(load_as_f32(row, base + c, dtype)));
                h = f16_to_f32(f32_to_f16(h * hs));
                h = f16_to_f32(f32_to_f16(h + ho));
                float r = rintf(h);
                r = r > 127.f ? 127.f : (r < -128.f ? -128.f : r);
                expandedX[d * cols + c] = (int8_t)r;
            }
            continue;
        }
        const float* sm = scale ? scale + (smoothRows == 1 ? 0 : (int64_t)expertIdx[i] * cols) : NULL;
        float mx = 0.f;
        for (int64_t c = 0; c < cols; c++) {
            float v = load_as_f32(row, base + c, dtype);
            if (sm) v = v * sm[c];
            mx = fabsf(v) > mx ? fabsf(v) : mx;
        }
        const float s = mx / 127.0f;
        dynScale[d] = s;
        for (int64_t c = 0; c < cols; c++) {
            float v = load_as_f32(row, base + c, dtype);
            if (sm) v = v * sm[c];
            float r = mx == 0.f ? 0.f : roundf(f32_to_f16_trunc_value(v / s));
            r = r > 127.f ? 127.f : (r < -128.f ? -128.f : r);
            expandedX[d * cols + c] = (int8_t)r;
        }
    }
    return 0;
}

/* ------------------------------------------------------------------------------------------------ grouped GEMM */

/* Group boundaries from groupList: type 0 = inclusive cumsum, type 1 = per-group counts (grouped_matmul_utils.h:243-257). */
static void group_bounds(const int64_t* groupList, int64_t G, int64_t listType, int64_t* begin /*[G+1]*/) {
    begin[0] = 0;
    for (int64_t e = 0; e < G; e++) begin[e + 1] = (listType == 0) ? groupList[e] : begin[e] + groupList[e];
}
static int64_t find_group(const int64_t* begin, int64_t G, int64_t row) {
    for (int64_t e = 0; e < G; e++) if (row >= begin[e] && row < begin[e + 1]) return e;
    return -1;
}

/* One int8 x int8 -> int32 output row.  w is [K,N] (wTrans == 0) or [N,K] storage (wTrans == 1) for the row's group. */
static void gemm_row_i32(const int8_t* xrow, const int8_t* w, int wTrans, int64_t K, int64_t N, int32_t* acc) {
    if (wTrans) {
        for (int64_t n = 0; n < N; n++) {
            const int8_t* wr = w + n * K;
            int32_t s = 0;
            for (int64_t k = 0; k < K; k++) s += (int32_t)xrow[k] * (int32_t)wr[k];
            acc[n] = s;
        }
    } else {
        for (int64_t n = 0; n < N; n++) acc[n] = 0;
        for (int64_t k = 0; k < K; k++) {
            const int32_t a = xrow[k];
            if (a == 0) continue;
            const int8_t* wr = w + k * N;
            for (int64_t n = 0; n < N; n++) acc[n] += a * (int32_t)wr[n];
        }
    }
}

/*
 * Raw accumulators of the grouped GEMM (the cube step of both GEMM ops):
 *   acc[r,c] = sum_k int32(x[r,k]) * int32(w[e,k,c]) for r in group e
 *   (grouped_matmul_swiglu_quant.h:159-182,232-262; grouped_matmul.h:250-282; grouped_matmul_quant_mixcore.h:175-215).
 * rows == NULL: all M rows, out is [M,N] and rows beyond the last group are left untouched.
 * rows != NULL: out is [nrows,N] for the listed expanded rows; a listed row outside every group is left untouched.
 */
ORACLE_API void oracle_grouped_matmul_i32(const int8_t* x, const int8_t* w, int wTrans, int64_t M, int64_t K, int64_t N,
                                          int64_t G, const int64_t* groupList, int64_t listType, const int64_t* rows,
                                          int64_t nrows, int32_t* out) {
    int64_t* begin = (int64_t*)malloc(sizeof(int64_t) * (size_t)(G + 1));
    group_bounds(groupList, G, listType, begin);
    const int64_t cnt = rows ? nrows : M;
#pragma omp parallel for schedule(dynamic, 4)
    for (int64_t i = 0; i < cnt; i++) {
        const int64_t r = rows ? rows[i] : i;
        if (r < 0 || r >= M) continue;
        const int64_t e = find_group(begin, G, r);
        if (e < 0) continue;
        gemm_row_i32(x + r * K, w + e * K * N, wTrans, K, N, out + i * N);
    }
    free(begin);
}

/*
 * GroupedMatmulSwigluQuant, A8W8 (grouped_matmul_swiglu_quant.h):
 *   dequant  C = (float(acc) * xScale[r]) * float(wScale[e,c])    :368-399 (per-token Muls first), :446-456 (per-channel Mul)
 *   swiglu   S[j] = (a / (1 + exp(-a))) * b, a = C[j], b = C[j + N/2]   :459-474 (README.md:63-65)
 *   requant  mx = max_j |S[j]|; yScale = mx / 127; inv = 1 / yScale; q = int8(rint(fp16(S[j] * inv)))   :477-513,
 *            grouped_matmul_swiglu_quant_utils.h:308-316 (fp32 -> fp16 RINT, fp16 -> int8 RINT)
 * An all-zero row gives yScale = 0 and inv = inf in the reference (0 * inf = NaN, undefined int8); here it yields q = 0.
 * wScaleDtype: 0 fp32, 1 fp16, 27 bf16.  rows / nrows as in oracle_grouped_matmul_i32; outputs are [cnt, N/2] and [cnt].
 * sOut (optional, [cnt, N/2] fp32) receives S before requantisation.
 */
ORACLE_API void oracle_grouped_matmul_swiglu_quant(const int8_t* x, const int8_t* w, int wTrans, const void* wScale,
                                                   int wScaleDtype, const float* xScale, int64_t M, int64_t K, int64_t N,
                                                   int64_t G, const int64_t* groupList, const int64_t* rows, int64_t nrows,
                                                   int8_t* y, float* yScale, float* sOut) {
    int64_t* begin = (int64_t*)malloc(sizeof(int64_t) * (size_t)(G + 1));
    group_bounds(groupList, G, 0, begin);
    const int64_t cnt = rows ? nrows : M;
    const int64_t I = N / 2;
#pragma omp parallel
    {
        int32_t* acc = (int32_t*)malloc(sizeof(int32_t) * (size_t)N);
        float* S = (float*)malloc(sizeof(float) * (size_t)(I > 0 ? I : 1));
#pragma omp for schedule(dynamic, 4)
        for (int64_t i = 0; i < cnt; i++) {
            const int64_t r = rows ? rows[i] : i;
            if (r < 0 || r >= M) continue;
            const int64_t e = find_group(begin, G, r);
            if (e < 0) continue;
            gemm_row_i32(x + r * K, w + e * K * N, wTrans, K, N, acc);
            const float xs = xScale[r];
            float mx = 0.0f;
            for (int64_t j = 0; j < I; j++) {
                const float a = ((float)acc[j] * xs) * load_as_f32(wScale, e * N + j, wScaleDtype);
                const float b = ((float)acc[j + I] * xs) * load_as_f32(wScale, e * N + j + I, wScaleDtype);
                const float s = (a / (1.0f + expf(-a))) * b;
                S[j] = s;
                const float as = fabsf(s);
                if (as > mx) mx = as;
            }
            const float ys = mx / 127.0f;
            const float inv = 1.0f / ys;
            yScale[i] = ys;
            for (int64_t j = 0; j < I; j++) {
                if (sOut) sOut[i * I + j] = S[j];
                if (mx == 0.0f) { y[i * I + j] = 0; continue; }
                const float h = f16_to_f32(f32_to_f16(S[j] * inv));
                y[i * I + j] = (int8_t)lrintf(h); /* default rounding mode: nearest even */
            }
        }
        free(acc); free(S);
    }
    free(begin);
}

/*
 * GroupedMatmul int8 quant epilogue (grouped_matmul_quant_mixcore.h:248-291,293-310):
 *   Y = (float(acc) * float(scale[e,c])) * perToken[r]   (per-channel AscendDequant first, then the per-token Mul)
 *   out = bf16 RINT / fp16 cast.  perToken may be NULL (static quant: Y = float(acc) * scale).
 * scaleDtype 0 fp32 / 27 bf16; outDtype 27 bf16 / 1 fp16 / 0 fp32.
 */
ORACLE_API void oracle_grouped_matmul_dequant(const int8_t* x, const int8_t* w, int wTrans, const void* scale, int scaleDtype,
                                              const float* perToken, int64_t M, int64_t K, int64_t N, int64_t G,
                                              const int64_t* groupList, int64_t listType, const int64_t* rows,
                                              int64_t nrows, void* out, int outDtype) {
    int64_t* begin = (int64_t*)malloc(sizeof(int64_t) * (size_t)(G + 1));
    group_bounds(groupList, G, listType, begin);
    const int64_t cnt = rows ? nrows : M;
#pragma omp parallel
    {
        int32_t* acc = (int32_t*)malloc(sizeof(int32_t) * (size_t)N);
#pragma omp for schedule(dynamic, 4)
        for (int64_t i = 0; i < cnt; i++) {
            const int64_t r = rows ? rows[i] : i;
            if (r < 0 || r >= M) continue;
            const int64_t e = find_group(begin, G, r);
            if (e < 0) continue;
            gemm_row_i32(x + r * K, w + e * K * N, wTrans, K, N, acc);
            for (int64_t c = 0; c < N; c++) {
                float v = (float)acc[c] * load_as_f32(scale, e * N + c, scaleDtype);
                if (perToken) v = v * perToken[r];
                store_from_f32(out, i * N + c, outDtype, v);
            }
        }
        free(acc);
    }
    free(begin);
}

/* GroupedMatmulFinalizeRouting with INT8 weights (gmm/grouped_matmul_finalize_routing/op_kernel/
 * grouped_matmul_finalize_routing.h): out [batch, N] fp32 starts at zero, rows [sharedOffset, sharedOffset + sharedRows)
 * at float(shared) * sharedWeight (:217-254); every row r of x in group e adds
 *   (float(acc[r, c]) * scale[e, c]) * (perToken[r] * logit[r])  [+ logit[r] * float(bias[e, c])]        (:390-417, :458-495)
 * to out[rowIndex[r], c] (:321-342).  The reference adds with fp32 atomics in no fixed order; here rows are added in
 * ascending r.  perToken, logit, bias, shared may be NULL (factor 1 / none). */
ORACLE_API void oracle_grouped_matmul_finalize_routing(const int8_t* x, const int8_t* w, int wTrans, const void* scale,
                                                       int scaleDtype, const void* bias, int biasDtype, const float* perToken,
                                                       const float* logit, const int64_t* rowIndex, int64_t M, int64_t K,
                                                       int64_t N, int64_t G, const int64_t* groupList, int64_t listType,
                                                       const uint16_t* shared, int sharedDtype, int64_t sharedRows,
                                                       int64_t sharedOffset, float sharedWeight, int64_t batch, float* out) {
    int64_t* begin = (int64_t*)malloc(sizeof(int64_t) * (size_t)(G + 1));
    group_bounds(groupList, G, listType, begin);
    for (int64_t i = 0; i < batch * N; i++) out[i] = 0.f;
    for (int64_t j = 0; j < sharedRows; j++) {
        for (int64_t c = 0; c < N; c++) out[(sharedOffset + j) * N + c] = load_as_f32(shared, j * N + c, sharedDtype) * sharedWeight;
    }
    float* contrib = (float*)malloc(sizeof(float) * (size_t)(M > 0 ? M : 1) * (size_t)N);
#pragma omp parallel
    {
        int32_t* acc = (int32_t*)malloc(sizeof(int32_t) * (size_t)N);
#pragma omp for schedule(dynamic, 4)
        for (int64_t r = 0; r < M; r++) {
            const int64_t e = find_group(begin, G, r);
            if (e < 0) { for (int64_t c = 0; c < N; c++) contrib[r * N + c] = 0.f; continue; }
            gemm_row_i32(x + r * K, w + e * K * N, wTrans, K, N, acc);
            float factor = perToken ? perToken[r] : 1.0f;
            if (logit) factor = factor * logit[r];
            for (int64_t c = 0; c < N; c++) {
                float v = ((float)acc[c] * load_as_f32(scale, e * N + c, scaleDtype)) * factor;
                if (bias) v = v + (logit ? logit[r] : 1.0f) * load_as_f32(bias, e * N + c, biasDtype);
                contrib[r * N + c] = v;
            }
        }
        free(acc);
    }
    for (int64_t r = 0; r < M; r++) {
        if (find_group(begin, G, r) < 0) continue;
        const int64_t d = rowIndex[r];
        if (d < 0 || d >= batch) continue;
        for (int64_t c = 0; c < N; c++) out[d * N + c] += contrib[r * N + c];
    }
    free(contrib);
    free(begin);
}

/* ------------------------------------------------------------------------------------------------ finalize */

/*
 * MoeFinalizeRoutingV2 (moe_finalize_routing_v2_bf16.h:286-609):
 *   acc = float(x1) + float(x2)  (one absent: the other; both absent: the first processed term initialises acc)
 *   for k ascending: d = idx[n*K + k] (modes 2,3) or idx[k*T + n] (modes 0,1)            :361-366
 *       d == -1 in modes 1,3: term skipped (as the first term with no skips it sets acc = 0)   :457-476
 *       v = float(expandedX[d]) (+ float(bias[expertIdx[n,k]]));  v = v * scale[n,k];  acc = acc + v   (separate mul and add)
 *   out = cast RINT to dtype                                                               :593
 * dtype: 0 fp32, 1 fp16, 27 bf16 for expandedX/x1/x2/bias/out; scaleDtype likewise (fp32 scales with bf16 data allowed).
 * bf16 data is widened to fp32 and rounded once at the end; fp32 and fp16 data are combined in their own arithmetic
 * (moe_finalize_routing_v2_fp_db.h:265-269,393-440: Add / Muls on LocalTensor<T>), i.e. fp16 rounds after every operation.
 * scales == NULL: K = 1 and the weight is 1.0.
 */
ORACLE_API void oracle_moe_finalize_routing_v2(const void* expandedX, const int32_t* expandedRowIdx, const void* x1,
                                               const void* x2, const void* bias, const void* scales,
                                               const int32_t* expertIdx, int64_t dropPadMode, int64_t T, int64_t K,
                                               int64_t H, int dtype, int scaleDtype, void* out) {
    /* fp16 data is combined in fp16 arithmetic: rounding an fp32 sum/product of two fp16 values to fp16 is the correctly
       rounded fp16 operation (24 >= 2*11+2 bits). */
#define RND(v) (dtype == DT_F16 ? f16_to_f32(f32_to_f16(v)) : (v))
#pragma omp parallel
    {
        float* acc = (float*)malloc(sizeof(float) * (size_t)(H > 0 ? H : 1));
#pragma omp for schedule(static)
        for (int64_t n = 0; n < T; n++) {
            int init = 0;
            if (x1 && x2) { for (int64_t h = 0; h < H; h++) acc[h] = RND(load_as_f32(x1, n * H + h, dtype) + load_as_f32(x2, n * H + h, dtype)); init = 1; }
            else if (x1) { for (int64_t h = 0; h < H; h++) acc[h] = load_as_f32(x1, n * H + h, dtype) + 0.0f; init = 1; }
            else if (x2) { for (int64_t h = 0; h < H; h++) acc[h] = load_as_f32(x2, n * H + h, dtype) + 0.0f; init = 1; }
            for (int64_t k = 0; k < K; k++) {
                const int64_t d = (dropPadMode >= 2) ? expandedRowIdx[n * K + k] : expandedRowIdx[k * T + n];
                const int skip = (d == -1) && (dropPadMode == 1 || dropPadMode == 3);
                const float s = scales ? load_as_f32(scales, n * K + k, scaleDtype) : 1.0f;
                const int64_t be = (bias && expertIdx) ? expertIdx[n * K + k] : 0;
                if (skip) {
                    if (!init) { for (int64_t h = 0; h < H; h++) acc[h] = 0.0f; init = 1; }
                    continue;
                }
                for (int64_t h = 0; h < H; h++) {
                    float v = load_as_f32(expandedX, d * H + h, dtype);
                    if (bias) v = RND(v + load_as_f32(bias, be * H + h, dtype));
                    v = RND(v * s);
                    acc[h] = init ? RND(acc[h] + v) : v;
                }
                init = 1;
            }
            for (int64_t h = 0; h < H; h++) store_from_f32(out, n * H + h, dtype, init ? acc[h] : 0.0f);
        }
        free(acc);
    }
#undef RND
}

/* Number of OpenMP threads the timed baseline will use. */
#ifdef _OPENMP
#include <omp.h>
ORACLE_API int oracle_num_threads(void) { return omp_get_max_threads(); }
#else
ORACLE_API int oracle_num_threads(void) { return 1; }
#endif
