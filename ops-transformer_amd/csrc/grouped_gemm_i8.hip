// Expert-grouped int8 x int8 -> int32 GEMM for gfx950 (CDNA4) with fused epilogues.
//
// Computes, for every group e and every row r of that group, acc[r, c] = sum_k x[r, k] * w[e, k, c] on
// v_mfma_i32_32x32x32_i8 and applies one of three epilogues in registers:
//   kInt32   raw accumulators                                   (aclnnGroupedMatmulV4, int32 output)
//   kDequant (float(acc) * scale[e, c]) * rowScale[r] -> bf16 / fp16 / fp32
//            (reference order: gmm/grouped_matmul/op_kernel/grouped_matmul_quant_mixcore.h:248-291,293-310)
//   kSwiglu  C = (float(acc) * rowScale[r]) * scale[e, c];  S = swish(C[:, j]) * C[:, j + N/2]
//            (reference order: gmm/grouped_matmul_swiglu_quant/op_kernel/grouped_matmul_swiglu_quant.h:368-399,446-474),
//            S is written as fp32 together with a per-row running max |S| (atomic max on the bit pattern); a second,
//            bandwidth-trivial kernel turns S into int8 with the row scale max/127 (same file :477-513).
//
// Structure.  Group sizes live in device memory, so a one-workgroup scheduling kernel turns groupList into
// (row start, rows, m-tile prefix) per group; the GEMM grid is launched with a static upper bound of workgroups and
// each workgroup finds its (group, m-tile, n-tile) by binary search, surplus workgroups exit at once.  Workgroup ids
// are dealt round-robin to the 8 XCDs by the hardware, so logical tile index = xcd * ceil(total / 8) + id / 8 keeps
// the tiles of one expert (which share activation rows and, across m-tiles, weight columns) on one XCD's L2.
//
// Tile: (32 * subTilesM * wavesM) rows x 256 columns x 128 k-bytes per step; 4 wave columns, each owning two 32-wide
// MFMA column tiles.  For kSwiglu the 256 columns are 128 "activated" columns j and their 128 partners j + N/2 and a
// wave owns matching 32-column blocks of both, so the SwiGLU product is formed in registers.
// Operands are staged global -> registers -> LDS with two LDS buffers; LDS rows are 128 bytes with the 16-byte chunk
// index XOR-ed with (row & 7), which makes both the 16-byte stores and the MFMA operand loads bank-conflict free.
// Weights are consumed K-contiguous ([N, K] per expert, the "transposed" view of the reference API); the row-major
// [K, N] form and shapes whose K is not a multiple of 16 go through a byte-wise loader that is correct but slow.
#include "grouped_gemm_i8.h"

#include "opapi_common.h"

#include <hip/hip_fp16.h>

#include <algorithm>

namespace gemm {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kStepBytes = 128;  // k extent of one pipeline step (int8 elements == bytes)
constexpr int kTileN = 256;
constexpr int kWavesN = 4;
constexpr int kChunk = 16;
constexpr int kChunksPerRow = kStepBytes / kChunk;
constexpr int kXcds = 8;
constexpr int kGroupM = 4;  // m-tiles walked together per n-tile for L2 reuse of weight columns
constexpr int kMaxGroups = 1024;

// ---------------------------------------------------------------------------------------------- scheduling table
// int32 layout: [0] total rows covered by groups, [1] total m-tiles, [2..2+G) row start, [..+G) rows, [..+G+1) m-tile prefix
__host__ __device__ inline int SchedInts(int groups) { return 2 + 3 * groups + 1; }

struct SchedArgs {
    const void* groupList;
    int32_t* sched;
    uint32_t* rowMax;  // zeroed for [0, M) when not null
    int32_t groups;
    int32_t groupListIsInt64;
    int32_t isCount;
    int32_t tileM;
    int64_t M;
};

__global__ __launch_bounds__(1024) void ScheduleKernel(SchedArgs a) {
    __shared__ int32_t scan[1024];
    const int t = threadIdx.x;
    auto at = [&](int i) -> int64_t {
        return a.groupListIsInt64 ? static_cast<const int64_t*>(a.groupList)[i]
                                  : static_cast<int64_t>(static_cast<const int32_t*>(a.groupList)[i]);
    };
    auto inclusiveScan = [&](int32_t v) -> int32_t {
        scan[t] = v;
        __syncthreads();
        for (int d = 1; d < 1024; d <<= 1) {
            const int32_t add = t >= d ? scan[t - d] : 0;
            __syncthreads();
            scan[t] += add;
            __syncthreads();
        }
        const int32_t r = scan[t];
        __syncthreads();
        return r;
    };
    // group boundaries, clamped into [0, M] and made monotonic so that a malformed list cannot push rows out of range
    int64_t begin = 0, end = 0;
    if (t < a.groups) {
        if (a.isCount) {
            int64_t c = at(t);
            c = c < 0 ? 0 : (c > a.M ? a.M : c);
            end = c;  // turned into a cumsum below
        } else {
            end = at(t);
            begin = t > 0 ? at(t - 1) : 0;
        }
    }
    if (a.isCount) {
        const int32_t inc = inclusiveScan(static_cast<int32_t>(end));
        begin = static_cast<int64_t>(inc) - end;
        end = inc;
    }
    begin = begin < 0 ? 0 : (begin > a.M ? a.M : begin);
    end = end < begin ? begin : (end > a.M ? a.M : end);
    const int32_t rows = t < a.groups ? static_cast<int32_t>(end - begin) : 0;
    const int32_t tiles = (rows + a.tileM - 1) / a.tileM;
    const int32_t tileInc = inclusiveScan(tiles);
    int32_t* rowStart = a.sched + 2;
    int32_t* rowCount = rowStart + a.groups;
    int32_t* tilePrefix = rowCount + a.groups;
    if (t < a.groups) {
        rowStart[t] = static_cast<int32_t>(begin);
        rowCount[t] = rows;
        tilePrefix[t] = tileInc - tiles;
        if (t == a.groups - 1) {
            tilePrefix[a.groups] = tileInc;
            a.sched[0] = static_cast<int32_t>(end);
            a.sched[1] = tileInc;
        }
    }
    if (a.rowMax != nullptr) {
        for (int64_t i = t; i < a.M; i += 1024) a.rowMax[i] = 0u;
    }
}

// ---------------------------------------------------------------------------------------------- GEMM kernel
struct KernelArgs {
    const int8_t* x;
    const int8_t* w;
    int64_t wGroupStride;  // bytes between experts
    int64_t wStrideN;      // bytes between consecutive output channels
    int64_t wStrideK;      // bytes between consecutive k
    int32_t M, K, N;
    int32_t groups;
    int32_t tilesN;
    int32_t halfN;  // N / 2 (kSwiglu)
    const int32_t* sched;
    void* out;
    int32_t outDtype;
    const void* scale;
    int32_t scaleDtype;
    const float* rowScale;
    float* sOut;
    uint32_t* rowMax;
};

__device__ __forceinline__ int LdsOffset(int row, int chunk) { return row * kStepBytes + ((chunk ^ (row & 7)) << 4); }

__device__ __forceinline__ float LoadScale(const void* p, int64_t i, int dtype) {
    if (dtype == 0) return static_cast<const float*>(p)[i];
    const uint16_t raw = static_cast<const uint16_t*>(p)[i];
    if (dtype == 1) return __half2float(__ushort_as_half(raw));
    return __uint_as_float(static_cast<uint32_t>(raw) << 16);
}

__device__ __forceinline__ uint16_t ToBf16(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return static_cast<uint16_t>((u >> 16) | 0x40);
    u += 0x7fffu + ((u >> 16) & 1u);
    return static_cast<uint16_t>(u >> 16);
}

// kFastLoad: 16-byte global loads (K-contiguous weights, K % 16 == 0, 16-byte aligned bases).  Otherwise byte-wise.
template <int kSubM, int kWavesM, Epilogue kEpi, bool kFastLoad>
__global__ __launch_bounds__(256 * kWavesM) void GroupedGemmKernel(KernelArgs a) {
    constexpr int kThreads = 256 * kWavesM;
    constexpr int kTileM = 32 * kSubM * kWavesM;
    constexpr int kRowsPerPass = kThreads / kChunksPerRow;  // tile rows covered by one load per thread
    constexpr int kALoads = kTileM / kRowsPerPass;           // == kSubM
    constexpr int kBLoads = kTileN / kRowsPerPass;
    constexpr bool kSwiglu = kEpi == Epilogue::kSwiglu;
    extern __shared__ __attribute__((aligned(16))) char lds[];
    char* const ldsA = lds;
    char* const ldsB = lds + 2 * kTileM * kStepBytes;

    // ---- which tile ----
    const int32_t totalMTiles = a.sched[1];
    const int64_t totalTiles = static_cast<int64_t>(totalMTiles) * a.tilesN;
    const int64_t perXcd = (totalTiles + kXcds - 1) / kXcds;
    const int64_t local = blockIdx.x / kXcds;
    const int64_t logical = static_cast<int64_t>(blockIdx.x % kXcds) * perXcd + local;
    if (local >= perXcd || logical >= totalTiles) return;
    const int32_t* rowStartTbl = a.sched + 2;
    const int32_t* rowCountTbl = rowStartTbl + a.groups;
    const int32_t* tilePrefix = rowCountTbl + a.groups;
    const int32_t q = static_cast<int32_t>(logical / a.tilesN);
    int lo = 0, hi = a.groups;
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (tilePrefix[mid] <= q) lo = mid; else hi = mid;
    }
    const int group = lo;
    const int32_t inGroup = static_cast<int32_t>(logical - static_cast<int64_t>(tilePrefix[group]) * a.tilesN);
    const int32_t tilesM = tilePrefix[group + 1] - tilePrefix[group];
    const int32_t band = inGroup / (kGroupM * a.tilesN);
    const int32_t rem = inGroup % (kGroupM * a.tilesN);
    const int32_t bandTiles = min(kGroupM, tilesM - kGroupM * band);
    const int32_t tileN = rem / bandTiles;
    const int32_t tileMIdx = kGroupM * band + rem % bandTiles;
    const int32_t rowBase = rowStartTbl[group] + tileMIdx * kTileM;
    const int32_t rows = min(kTileM, rowCountTbl[group] - tileMIdx * kTileM);  // >= 1

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int waveN = wave % kWavesN;
    const int waveM = wave / kWavesN;
    const int l32 = lane & 31;
    const int lhi = lane >> 5;

    // Output channel held in LDS row r of the weight tile.
    const int32_t colBase = kSwiglu ? tileN * (kTileN / 2) : tileN * kTileN;
    auto channelOfRow = [&](int r) -> int32_t {
        int32_t n;
        if (kSwiglu) n = r < kTileN / 2 ? colBase + r : a.halfN + colBase + (r - kTileN / 2);
        else n = colBase + r;
        return n < a.N ? n : a.N - 1;  // clamped loads; such columns are never stored
    };

    const int8_t* const wGroup = a.w + static_cast<int64_t>(group) * a.wGroupStride;
    const int kSteps = (a.K + kStepBytes - 1) / kStepBytes;

    v4i regA[kALoads];
    v4i regB[kBLoads];

    auto loadGlobal = [&](int step) {
        const int k0 = step * kStepBytes;
        if (kFastLoad) {
            const int chunk = tid % kChunksPerRow;
            const int rowInPass = tid / kChunksPerRow;
            const int k = k0 + chunk * kChunk;
            const bool kValid = k < a.K;
#pragma unroll
            for (int i = 0; i < kALoads; ++i) {
                const int r = i * kRowsPerPass + rowInPass;
                v4i v = {0, 0, 0, 0};
                if (i * kRowsPerPass < rows && kValid) {
                    const int rr = r < rows ? r : rows - 1;
                    v = *reinterpret_cast<const v4i*>(a.x + static_cast<int64_t>(rowBase + rr) * a.K + k);
                }
                regA[i] = v;
            }
#pragma unroll
            for (int i = 0; i < kBLoads; ++i) {
                const int r = i * kRowsPerPass + rowInPass;
                v4i v = {0, 0, 0, 0};
                if (kValid) v = *reinterpret_cast<const v4i*>(wGroup + static_cast<int64_t>(channelOfRow(r)) * a.wStrideN + k);
                regB[i] = v;
            }
        } else {
            // byte-wise: consecutive threads take consecutive tile rows so that N-contiguous weights still coalesce
#pragma unroll
            for (int i = 0; i < kALoads; ++i) {
                const int p = i * kThreads + tid;
                const int r = p % kTileM;
                const int chunk = p / kTileM;
                const int rr = r < rows ? r : rows - 1;
                const int8_t* src = a.x + static_cast<int64_t>(rowBase + rr) * a.K;
                union { v4i v; int8_t b[16]; } u;
                for (int j = 0; j < kChunk; ++j) {
                    const int k = k0 + chunk * kChunk + j;
                    u.b[j] = k < a.K ? src[k] : static_cast<int8_t>(0);
                }
                regA[i] = u.v;
            }
#pragma unroll
            for (int i = 0; i < kBLoads; ++i) {
                const int p = i * kThreads + tid;
                const int r = p % kTileN;
                const int chunk = p / kTileN;
                const int8_t* src = wGroup + static_cast<int64_t>(channelOfRow(r)) * a.wStrideN;
                union { v4i v; int8_t b[16]; } u;
                for (int j = 0; j < kChunk; ++j) {
                    const int k = k0 + chunk * kChunk + j;
                    u.b[j] = k < a.K ? src[static_cast<int64_t>(k) * a.wStrideK] : static_cast<int8_t>(0);
                }
                regB[i] = u.v;
            }
        }
    };

    auto storeLds = [&](int buf) {
        char* A = ldsA + buf * kTileM * kStepBytes;
        char* B = ldsB + buf * kTileN * kStepBytes;
        if (kFastLoad) {
            const int chunk = tid % kChunksPerRow;
            const int rowInPass = tid / kChunksPerRow;
#pragma unroll
            for (int i = 0; i < kALoads; ++i) {
                const int r = i * kRowsPerPass + rowInPass;
                *reinterpret_cast<v4i*>(A + LdsOffset(r, chunk)) = regA[i];
            }
#pragma unroll
            for (int i = 0; i < kBLoads; ++i) {
                const int r = i * kRowsPerPass + rowInPass;
                *reinterpret_cast<v4i*>(B + LdsOffset(r, chunk)) = regB[i];
            }
        } else {
#pragma unroll
            for (int i = 0; i < kALoads; ++i) {
                const int p = i * kThreads + tid;
                *reinterpret_cast<v4i*>(A + LdsOffset(p % kTileM, p / kTileM)) = regA[i];
            }
#pragma unroll
            for (int i = 0; i < kBLoads; ++i) {
                const int p = i * kThreads + tid;
                *reinterpret_cast<v4i*>(B + LdsOffset(p % kTileN, p / kTileN)) = regB[i];
            }
        }
    };

    // ---- main loop ----
    v16i acc[kSubM][2];
#pragma unroll
    for (int mi = 0; mi < kSubM; ++mi)
#pragma unroll
        for (int ni = 0; ni < 2; ++ni)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[mi][ni][v] = 0;

    const int waveRow0 = waveM * 32 * kSubM;
    int active = (rows - waveRow0 + 31) / 32;  // 32-row MFMA tiles of this wave that hold real rows
    active = active < 0 ? 0 : (active > kSubM ? kSubM : active);
    const int bRow0 = kSwiglu ? 32 * waveN : 64 * waveN;
    const int bRowStep = kSwiglu ? kTileN / 2 : 32;

    loadGlobal(0);
    storeLds(0);
    __syncthreads();
    for (int step = 0; step < kSteps; ++step) {
        const int buf = step & 1;
        if (step + 1 < kSteps) loadGlobal(step + 1);
        const char* A = ldsA + buf * kTileM * kStepBytes;
        const char* B = ldsB + buf * kTileN * kStepBytes;
#pragma unroll
        for (int ks = 0; ks < kStepBytes / 32; ++ks) {
            const int chunk = 2 * ks + lhi;
            const v4i b0 = *reinterpret_cast<const v4i*>(B + LdsOffset(bRow0 + l32, chunk));
            const v4i b1 = *reinterpret_cast<const v4i*>(B + LdsOffset(bRow0 + bRowStep + l32, chunk));
#pragma unroll
            for (int mi = 0; mi < kSubM; ++mi) {
                if (mi < active) {
                    const v4i av = *reinterpret_cast<const v4i*>(A + LdsOffset(waveRow0 + mi * 32 + l32, chunk));
                    acc[mi][0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av, b0, acc[mi][0], 0, 0, 0);
                    acc[mi][1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av, b1, acc[mi][1], 0, 0, 0);
                }
            }
        }
        if (step + 1 < kSteps) storeLds(buf ^ 1);
        __syncthreads();
    }

    // ---- epilogue ----
    // acc[mi][ni][v] is C[row, col] with row = waveRow0 + 32*mi + 8*(v/4) + 4*lhi + (v%4), col = column block ni, lane l32.
    if (kEpi == Epilogue::kInt32 || kEpi == Epilogue::kDequant) {
#pragma unroll
        for (int ni = 0; ni < 2; ++ni) {
            const int32_t n = colBase + 64 * waveN + 32 * ni + l32;
            const bool nValid = n < a.N;
            float sc = 0.0f;
            if (kEpi == Epilogue::kDequant && nValid) sc = LoadScale(a.scale, static_cast<int64_t>(group) * a.N + n, a.scaleDtype);
#pragma unroll
            for (int mi = 0; mi < kSubM; ++mi) {
                if (mi >= active) continue;
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int r = waveRow0 + 32 * mi + 8 * (v / 4) + 4 * lhi + (v % 4);
                    if (r >= rows || !nValid) continue;
                    const int64_t o = static_cast<int64_t>(rowBase + r) * a.N + n;
                    if (kEpi == Epilogue::kInt32) {
                        static_cast<int32_t*>(a.out)[o] = acc[mi][ni][v];
                    } else {
                        float y = __fmul_rn(static_cast<float>(acc[mi][ni][v]), sc);
                        if (a.rowScale != nullptr) y = __fmul_rn(y, a.rowScale[rowBase + r]);
                        if (a.outDtype == 27) static_cast<uint16_t*>(a.out)[o] = ToBf16(y);
                        else if (a.outDtype == 1) static_cast<__half*>(a.out)[o] = __float2half_rn(y);
                        else static_cast<float*>(a.out)[o] = y;
                    }
                }
            }
        }
    } else {
        const int32_t j = colBase + 32 * waveN + l32;  // column of S
        const bool jValid = j < a.halfN;
        float scA = 0.0f, scB = 0.0f;
        if (jValid) {
            scA = LoadScale(a.scale, static_cast<int64_t>(group) * a.N + j, a.scaleDtype);
            scB = LoadScale(a.scale, static_cast<int64_t>(group) * a.N + a.halfN + j, a.scaleDtype);
        }
#pragma unroll
        for (int mi = 0; mi < kSubM; ++mi) {
            if (mi >= active) continue;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int r = waveRow0 + 32 * mi + 8 * (v / 4) + 4 * lhi + (v % 4);
                const bool valid = r < rows && jValid;
                float s = 0.0f;
                if (valid) {
                    const float xs = a.rowScale[rowBase + r];
                    const float ca = __fmul_rn(__fmul_rn(static_cast<float>(acc[mi][0][v]), xs), scA);
                    const float cb = __fmul_rn(__fmul_rn(static_cast<float>(acc[mi][1][v]), xs), scB);
                    s = __fmul_rn(__fdiv_rn(ca, __fadd_rn(1.0f, expf(-ca))), cb);
                    a.sOut[static_cast<int64_t>(rowBase + r) * a.halfN + j] = s;
                }
                float m = fabsf(s);
#pragma unroll
                for (int d = 1; d < 32; d <<= 1) m = fmaxf(m, __shfl_xor(m, d, 64));
                if (l32 == 0 && r < rows) atomicMax(a.rowMax + rowBase + r, __float_as_uint(m));
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------- requantisation
struct RequantArgs {
    const float* s;          // [M, halfN]
    const uint32_t* rowMax;  // [M] bit pattern of max |S|
    const int32_t* sched;
    int8_t* y;               // [M, halfN]
    float* yScale;           // [M]
    int32_t halfN;
};

__device__ __forceinline__ int8_t QuantOne(float s, float inv) {
    const __half h = __float2half_rn(__fmul_rn(s, inv));
    return static_cast<int8_t>(__float2int_rn(__half2float(h)));
}

// One workgroup per row; rows at or beyond the last group boundary are left untouched.
__global__ __launch_bounds__(256) void RequantKernel(RequantArgs a) {
    const int64_t row = blockIdx.x;
    if (row >= a.sched[0]) return;
    const float mx = __uint_as_float(a.rowMax[row]);
    const float ys = __fdiv_rn(mx, 127.0f);
    const float inv = __fdiv_rn(1.0f, ys);
    if (threadIdx.x == 0) a.yScale[row] = ys;
    const float* src = a.s + row * a.halfN;
    int8_t* dst = a.y + row * a.halfN;
    const bool zeroRow = mx == 0.0f;  // reference: 0 * inf; defined here as zeros
    if ((a.halfN & 3) == 0) {
        for (int j = threadIdx.x * 4; j < a.halfN; j += 256 * 4) {
            const float4 v = *reinterpret_cast<const float4*>(src + j);
            char4 q;
            q.x = zeroRow ? 0 : QuantOne(v.x, inv);
            q.y = zeroRow ? 0 : QuantOne(v.y, inv);
            q.z = zeroRow ? 0 : QuantOne(v.z, inv);
            q.w = zeroRow ? 0 : QuantOne(v.w, inv);
            *reinterpret_cast<char4*>(dst + j) = q;
        }
    } else {
        for (int j = threadIdx.x; j < a.halfN; j += 256) dst[j] = zeroRow ? 0 : QuantOne(src[j], inv);
    }
}

// ---------------------------------------------------------------------------------------------- dispatch
template <int kSubM, int kWavesM, Epilogue kEpi, bool kFastLoad>
hipError_t LaunchOne(const KernelArgs& args, int64_t grid, hipStream_t stream) {
    constexpr int kTileM = 32 * kSubM * kWavesM;
    constexpr int kLdsBytes = 2 * (kTileM + kTileN) * kStepBytes;
    auto kernel = GroupedGemmKernel<kSubM, kWavesM, kEpi, kFastLoad>;
    static hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
    if (attr != hipSuccess) return attr;
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(grid)), dim3(256 * kWavesM), kLdsBytes, stream, args);
    return hipGetLastError();
}

template <Epilogue kEpi, bool kFastLoad>
hipError_t LaunchShape(const Plan& plan, const KernelArgs& args, int64_t grid, hipStream_t stream) {
    if constexpr (!kFastLoad) {  // the byte-wise loader exists for two shapes only
        if (plan.tileM <= 32) return LaunchOne<1, 1, kEpi, false>(args, grid, stream);
        return LaunchOne<4, 1, kEpi, false>(args, grid, stream);
    } else {
        switch (plan.tileM) {
            case 32: return LaunchOne<1, 1, kEpi, true>(args, grid, stream);
            case 64: return LaunchOne<2, 1, kEpi, true>(args, grid, stream);
            case 96: return LaunchOne<3, 1, kEpi, true>(args, grid, stream);
            case 128: return LaunchOne<4, 1, kEpi, true>(args, grid, stream);
            case 192: return LaunchOne<3, 2, kEpi, true>(args, grid, stream);
            default: return LaunchOne<4, 2, kEpi, true>(args, grid, stream);
        }
    }
}

bool FastLoadOk(const Problem& p) {
    return p.wKMajor && p.K % kChunk == 0 && reinterpret_cast<uintptr_t>(p.x) % kChunk == 0 &&
           reinterpret_cast<uintptr_t>(p.w) % kChunk == 0;
}

uint64_t Align256(uint64_t v) { return (v + 255) / 256 * 256; }

}  // namespace

Plan MakePlan(const Problem& p) {
    Plan plan;
    const int64_t groups = p.groups > 0 ? p.groups : 1;
    const double want = static_cast<double>(p.M) / static_cast<double>(groups) * 1.3;
    static const int kShapes[] = {32, 64, 96, 128, 192, 256};
    plan.tileM = 256;
    for (int s : kShapes) {
        if (static_cast<double>(s) >= want) { plan.tileM = s; break; }
    }
    if (!FastLoadOk(p)) plan.tileM = plan.tileM <= 32 ? 32 : 128;
    plan.wavesM = plan.tileM > 128 ? 2 : 1;
    plan.subTilesM = plan.tileM / 32 / plan.wavesM;
    const int64_t cols = p.epilogue == Epilogue::kSwiglu ? p.N / 2 : p.N;
    const int64_t colsPerTile = p.epilogue == Epilogue::kSwiglu ? kTileN / 2 : kTileN;
    plan.tilesN = static_cast<int32_t>((cols + colsPerTile - 1) / colsPerTile);
    const int64_t maxMTiles = p.M / plan.tileM + groups;
    // round up so that every XCD's share [xcd * ceil(total/8), ...) is covered by the launch
    plan.maxTiles = (maxMTiles * plan.tilesN + kXcds - 1) / kXcds * kXcds;
    uint64_t off = 0;
    plan.offSched = off;
    off += Align256(static_cast<uint64_t>(SchedInts(static_cast<int>(groups))) * 4);
    if (p.epilogue == Epilogue::kSwiglu) {
        plan.offRowMax = off;
        off += Align256(static_cast<uint64_t>(p.M) * 4);
        plan.offS = off;
        off += Align256(static_cast<uint64_t>(p.M) * static_cast<uint64_t>(p.N / 2) * 4);
    }
    plan.workspaceBytes = off;
    return plan;
}

hipError_t Enqueue(const Problem& p, const Plan& plan, void* workspace, hipStream_t stream) {
    if (p.M == 0 || p.N == 0 || p.groups == 0) return hipSuccess;
    if (p.groups > kMaxGroups) return hipErrorInvalidValue;
    char* ws = static_cast<char*>(workspace);
    int32_t* sched = reinterpret_cast<int32_t*>(ws + plan.offSched);
    const bool swiglu = p.epilogue == Epilogue::kSwiglu;
    uint32_t* rowMax = swiglu ? reinterpret_cast<uint32_t*>(ws + plan.offRowMax) : nullptr;
    float* sBuf = swiglu ? reinterpret_cast<float*>(ws + plan.offS) : nullptr;

    SchedArgs sa{};
    sa.groupList = p.groupList;
    sa.sched = sched;
    sa.rowMax = rowMax;
    sa.groups = p.groups;
    sa.groupListIsInt64 = p.groupListIsInt64 ? 1 : 0;
    sa.isCount = p.groupListKind == GroupListKind::kCount ? 1 : 0;
    sa.tileM = plan.tileM;
    sa.M = p.M;
    {
        opapi::KernelTimer timer("gmm_schedule", stream);
        hipLaunchKernelGGL(ScheduleKernel, dim3(1), dim3(1024), 0, stream, sa);
    }

    KernelArgs ka{};
    ka.x = p.x;
    ka.w = p.w;
    ka.wGroupStride = p.K * p.N;
    ka.wStrideN = p.wKMajor ? p.K : 1;
    ka.wStrideK = p.wKMajor ? 1 : p.N;
    ka.M = static_cast<int32_t>(p.M);
    ka.K = static_cast<int32_t>(p.K);
    ka.N = static_cast<int32_t>(p.N);
    ka.groups = p.groups;
    ka.tilesN = plan.tilesN;
    ka.halfN = static_cast<int32_t>(p.N / 2);
    ka.sched = sched;
    ka.out = p.out;
    ka.outDtype = p.outDtype;
    ka.scale = p.scale;
    ka.scaleDtype = p.scaleDtype;
    ka.rowScale = p.rowScale;
    ka.sOut = sBuf;
    ka.rowMax = rowMax;

    hipError_t e = hipSuccess;
    if (p.K > 0) {
        const bool fast = FastLoadOk(p);
        opapi::KernelTimer timer(p.epilogue == Epilogue::kSwiglu ? "gmm_swiglu"
                                 : p.epilogue == Epilogue::kDequant ? "gmm_dequant" : "gmm_int32", stream);
        switch (p.epilogue) {
            case Epilogue::kInt32:
                e = fast ? LaunchShape<Epilogue::kInt32, true>(plan, ka, plan.maxTiles, stream)
                         : LaunchShape<Epilogue::kInt32, false>(plan, ka, plan.maxTiles, stream);
                break;
            case Epilogue::kDequant:
                e = fast ? LaunchShape<Epilogue::kDequant, true>(plan, ka, plan.maxTiles, stream)
                         : LaunchShape<Epilogue::kDequant, false>(plan, ka, plan.maxTiles, stream);
                break;
            case Epilogue::kSwiglu:
                e = fast ? LaunchShape<Epilogue::kSwiglu, true>(plan, ka, plan.maxTiles, stream)
                         : LaunchShape<Epilogue::kSwiglu, false>(plan, ka, plan.maxTiles, stream);
                break;
        }
        if (e != hipSuccess) return e;
    }
    if (swiglu) {
        RequantArgs ra{sBuf, rowMax, sched, p.quantOut, p.quantScaleOut, static_cast<int32_t>(p.N / 2)};
        opapi::KernelTimer timer("gmm_requant", stream);
        hipLaunchKernelGGL(RequantKernel, dim3(static_cast<unsigned>(p.M)), dim3(256), 0, stream, ra);
        e = hipGetLastError();
    }
    return e;
}

}  // namespace gemm
