// Host interface of the expert-grouped int8 GEMM engine shared by aclnnGroupedMatmulSwigluQuant and aclnnGroupedMatmulV4.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

namespace gemm {

enum class Epilogue : int {
    kInt32 = 0,    // out[int32] = acc
    kDequant = 1,  // out = cast((float(acc) * scale[e,c]) * rowScale[r])
    kSwiglu = 2,   // S = swish(C[:, j]) * C[:, j + N/2] with C = (float(acc) * rowScale[r]) * scale[e,c]; S and row max |S| out
};

// kSparse: [groups, 2] pairs (expert id, rows) in row order, ended by the first pair without rows.
enum class GroupListKind : int { kCumsum = 0, kCount = 1, kSparse = 2 };

// Element type codes follow aclDataType: 0 fp32, 1 fp16, 27 bf16, 3 int32.
struct Problem {
    // operands
    const int8_t* x = nullptr;       // [M, K] row-major
    const int8_t* w = nullptr;       // per group: [N, K] K-contiguous when wKMajor, else [K, N] N-contiguous
    bool wKMajor = true;
    // Blocked weight layout (the reference's FRACTAL_NZ for int8): per group [N/32][K/16][16][32], i.e. element (k, n)
    // at ((n / 32) * (K / 16) + k / 16) * 512 + (k % 16) * 32 + n % 32.  Needs K % 16 == 0 and N % 32 == 0; wKMajor is
    // then ignored.
    bool wNz = false;
    int64_t M = 0, K = 0, N = 0;
    int32_t groups = 0;
    const void* groupList = nullptr; // device, int64 or int32: cumsum or counts [groups], or sparse pairs [groups, 2]
    bool groupListIsInt64 = true;
    GroupListKind groupListKind = GroupListKind::kCumsum;
    int64_t expectedRowsPerGroup = 0; // > 0: caller's hint for the tile height; 0: use M / groups
    // epilogue
    Epilogue epilogue = Epilogue::kInt32;
    void* out = nullptr;             // kInt32 / kDequant: [M, N]
    int outDtype = 3;
    const void* scale = nullptr;     // [groups, N] per output channel
    int scaleDtype = 0;
    const float* rowScale = nullptr; // [M] per token, may be null for kDequant
    // kDequant with fp32 output only: scatter-add instead of store.  Row r of the result is added (atomically, fp32) to
    // out[combineIndex[r], :] when the index lies in [0, combineRows); with a bias, combineWeight[r] * bias[e, c] is
    // added to the value first.  `out` is then [combineRows, N] and must hold its initial value before the launch.
    const void* combineIndex = nullptr;  // [M] int64 or int32
    bool combineIndexIsInt64 = true;
    int64_t combineRows = 0;
    const float* combineWeight = nullptr;  // [M], used with bias only
    const void* bias = nullptr;            // [groups, N]
    int biasDtype = 0;
    // kSwiglu only
    int8_t* quantOut = nullptr;      // [M, N/2]
    float* quantScaleOut = nullptr;  // [M]
};

// Tile shape chosen from the static shape (M, groups); fixed for the lifetime of a plan.
struct Plan {
    int tileM = 0;          // rows per workgroup tile (multiple of 32)
    int wavesM = 1;         // 1 or 2 wave rows
    int subTilesM = 1;      // 32-row MFMA tiles per wave
    int64_t maxTiles = 0;   // launch bound on workgroups
    int32_t maxMTiles = 0;  // upper bound on m-tiles over all groups (M / tileM + groups)
    int32_t tilesN = 0;
    bool pullTiles = false; // LDS-ring kernels: workgroups draw their tiles from counters instead of walking fixed shares
    int64_t bandRows = 0;   // kSwiglu: rows of S held in the workspace at a time (M when the launch runs as one band)
    uint64_t offSched = 0, offRowMax = 0, offS = 0;
    uint64_t workspaceBytes = 0;
};

Plan MakePlan(const Problem& p);

// Enqueues scheduling, GEMM and (kSwiglu) requantisation kernels on `stream`.  Returns hipSuccess or the launch error.
hipError_t Enqueue(const Problem& p, const Plan& plan, void* workspace, hipStream_t stream);

}  // namespace gemm
