// Device side of the expert-grouped int8 GEMM (see grouped_gemm_i8.hip for the overview): the LDS-ring kernels, the
// byte-wise kernel, their epilogues and launchers.  Included by grouped_gemm_i8.hip (scheduling, requantisation, planning)
// and by one translation unit per epilogue (grouped_gemm_i8_int32.hip, _dequant.hip, _swiglu.hip), each of which
// instantiates the kernels of its epilogue only, so that the three compile side by side.
#pragma once
#include "grouped_gemm_i8.h"

#include <hip/hip_fp16.h>

#include <algorithm>
#include <atomic>
#include <cstdlib>
#include <type_traits>

#include "opapi_common.h"

#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Wunused-function"

namespace gemm {

// Arguments of the GEMM kernels (one type for every translation unit of the engine).
struct KernelArgs {
    const int8_t* x;
    const int8_t* w;
    int64_t wGroupStride;  // bytes between experts
    int64_t wStrideN;      // bytes between consecutive output channels
    int64_t wStrideK;      // bytes between consecutive k
    int32_t wNz;           // weights in 32-channel x 16-k blocks ([N/32][K/16][16][32] per expert), see Problem::wNz
    int32_t M, K, N;
    int32_t groups;
    int32_t tilesN;
    int32_t halfN;  // N / 2 (kSwiglu)
    void* out;
    int32_t outDtype;
    const void* scale;
    int32_t scaleDtype;
    const float* rowScale;
    float* sOut;
    float* rowMax;  // [tilesN][M] partial max |S| per n-tile
    // scatter-add mode of the fp32 kDequant epilogue (Problem::combineIndex)
    const void* combineIndex;
    int32_t combineIndexIsInt64;
    int32_t combineRows;
    const float* combineWeight;
    const void* bias;
    int32_t biasDtype;
    // workgroup spans (include/opapi_profile.h): per workgroup {start, end} of the 100 MHz real-time counter and the
    // number of tiles it computed; null unless span recording is on
    uint64_t* wgSpans;
    // LDS-ring kernels: the tile counters of the scheduling table as a pointer the kernel may write through (the table
    // itself is a read-only kernel parameter), and whether workgroups pull their tiles from the counters (1) or walk a
    // fixed share (0)
    int32_t* queueCounters;
    int32_t pullTiles;
};

// Defined in grouped_gemm_i8.hip.
int DeviceCuCount();
uint64_t* SpanBufferFor(Epilogue epi, int grid, int tileM);

// One launcher pair per epilogue, each defined in its own translation unit: the LDS-ring kernels (K a multiple of 128,
// one of the three weight layouts) and the byte-wise kernel.
hipError_t LaunchRingInt32(const Plan& plan, const KernelArgs& args, const int32_t* sched, hipStream_t stream);
hipError_t LaunchRingDequant(const Plan& plan, const KernelArgs& args, const int32_t* sched, hipStream_t stream);
hipError_t LaunchRingSwiglu(const Plan& plan, const KernelArgs& args, const int32_t* sched, hipStream_t stream);
hipError_t LaunchGenericInt32(const Plan& plan, const KernelArgs& args, const int32_t* sched, hipStream_t stream);
hipError_t LaunchGenericDequant(const Plan& plan, const KernelArgs& args, const int32_t* sched, hipStream_t stream);
hipError_t LaunchGenericSwiglu(const Plan& plan, const KernelArgs& args, const int32_t* sched, hipStream_t stream);

namespace {

typedef int v2i __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) v2i* LdsV2iPtr;
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float Float2 __attribute__((ext_vector_type(2)));
typedef __bf16 Bf16x2 __attribute__((ext_vector_type(2)));

constexpr int kTileN = 256;
constexpr int kWavesN = 4;
constexpr int kChunk = 16;
constexpr int kXcds = 8;
constexpr int kGroupM = 4;  // m-tiles walked together per n-tile for L2 reuse of weight columns
constexpr int kMaxGroups = 1024;
constexpr int kLdsBudget = 160 * 1024;

// ---------------------------------------------------------------------------------------------- scheduling table
// int32 layout, all written by the scheduling kernel:
//   header, 32 ints: [0] big m-tiles, [1] small m-tiles, [2] cost of the small ones, [3] cost of the big ones (see below),
//                    [4] / [5] band width of the big / small run, [6] total rows covered by the groups;
//   16 tile counters in one 128-byte line (32 ints): counter [2 * xcd + list], zeroed;
//   the m-tile table, 4 ints per m-tile {group, first row, rows, 0} (at most maxMTiles of them): the big m-tiles in group
//   order, then the small ones.  A GEMM kernel finds everything about a tile with one 16-byte load.
// An m-tile is small when it holds at most kSmallRows rows: its time is the weight stream's (the whole K x 256 weight
// block for a handful of rows), not the matrix pipe's.  The two kinds are kept apart so that a launch which holds both
// (a skewed routing: a few experts with thousands of rows, many with a few) can run them side by side -- some
// workgroups streaming small tiles while the others multiply big ones -- instead of a compute-bound phase followed by
// a bandwidth-bound one.  Costs are in units of one 32-row MFMA tile over the whole K: a big m-tile costs its count of
// occupied 32-row tiles (at least kSmallCost), a small one kSmallCost (what the weight stream of a tile takes when
// only a part of the workgroups stream).
constexpr int kSmallRows = 64;
constexpr int kSmallCost = 3;
constexpr int kQueueHeaderInts = 32;
constexpr int kQueueCounterInts = 32;
constexpr int kHdrCoveredRows = 6;
__host__ __device__ inline int SchedTotalInts(int maxMTiles) { return kQueueHeaderInts + kQueueCounterInts + 4 * maxMTiles; }


// One output tile of one group, decoded from the scheduling table (all fields are wave-uniform).
struct TileInfo {
    int32_t valid;
    int32_t group;
    int32_t rowBase;  // first row of the tile in x / out
    int32_t rows;     // 1..tileM real rows
    int32_t tileN;
    int32_t colBase;  // first output channel (kSwiglu: first column of S)
};

// Tile `logical` of one run of the m-tile table (`count` m-tiles from entry `first` on).  Bands of bandWidth m-tiles walk
// the n-tiles together: consecutive tiles are the band's m-tiles at one n-tile, then the next n-tile.
template <int kTileM, bool kSwiglu>
__device__ __forceinline__ TileInfo DecodeListTile(const KernelArgs& a, const int4* __restrict__ table, int32_t first,
                                                   int32_t count, int32_t bandWidth, int64_t logical) {
    TileInfo t{};
    const int32_t perBand = bandWidth * a.tilesN;
    const int32_t band = static_cast<int32_t>(logical / perBand);
    const int32_t rem = static_cast<int32_t>(logical % perBand);
    const int32_t bandTiles = min(bandWidth, count - bandWidth * band);
    const int4 e = table[first + bandWidth * band + rem % bandTiles];
    t.valid = 1;
    t.group = e.x;
    t.rowBase = e.y;
    t.rows = e.z;  // 1..kTileM
    t.tileN = rem / bandTiles;
    t.colBase = kSwiglu ? t.tileN * (kTileN / 2) : t.tileN * kTileN;
    return t;
}

// ---- tile counters: workgroups pull their tiles instead of walking a fixed share ----
// Each of the two runs of the m-tile table (big, small) is cut into eight contiguous shares of tiles, one per XCD, so
// that the workgroups of an XCD sit on neighbouring tiles and share operands through that XCD's L2.  Counter
// [2 * xcd + list] hands out the tiles of a share in order.  A workgroup draws from its own XCD first -- the list it
// prefers, then the other -- and, when both are used up, from the other XCDs' shares in ring order, so nobody idles
// while tiles are left anywhere.  The counters are only ever added to (values past a share's size mean "used up").
// (The lists' sizes travel as plain values: a structure handed round by reference, or an array indexed at run time,
// ends up in scratch memory.)
__device__ __forceinline__ void QueueShare(int64_t tilesBig, int64_t tilesSmall, int counter, int64_t* first, int64_t* size) {
    const int64_t total = (counter & 1) ? tilesSmall : tilesBig;
    const int64_t per = (total + kXcds - 1) / kXcds;
    const int64_t begin = (counter >> 1) * per;
    *first = begin;
    *size = total - begin < 0 ? 0 : (total - begin < per ? total - begin : per);
}
// Counter i-th in the preference order of a workgroup on XCD `home` that prefers list `prefer`.
__device__ __forceinline__ int QueueCandidate(int i, int home, int prefer) {
    return 2 * ((home + (i >> 1)) & (kXcds - 1)) + ((i & 1) ? 1 - prefer : prefer);
}
// onlyPreferred: the other run's counters are not candidates at all (a workgroup that serves one run at a time).
__device__ __forceinline__ int QueueFirstOpen(uint32_t usedUp, int home, int prefer, bool onlyPreferred = false) {
#pragma unroll
    for (int i = 0; i < 2 * kXcds; ++i) {
        if (onlyPreferred && (i & 1)) continue;
        const int c = QueueCandidate(i, home, prefer);
        if (((usedUp >> c) & 1u) == 0) return c;
    }
    return -1;
}
__device__ __forceinline__ int32_t QueueTake(int32_t* counters, int c) {
    return __hip_atomic_fetch_add(counters + c, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// Completes a draw that began with QueueTake on counter c (value v; c < 0: nothing was open): returns the list (0 big,
// 1 small) and the tile inside that list's run, or list -1 when every share is used up.  One thread of the workgroup.
struct QueueDraw {
    int32_t list;     // 0 big, 1 small, -1 none
    int32_t logical;  // tile inside that list's run
    uint32_t usedUp;  // the caller's mask of used-up counters, updated
};
__device__ __forceinline__ QueueDraw QueueResolve(int64_t tilesBig, int64_t tilesSmall, int32_t* counters, int home, int prefer,
                                                  uint32_t usedUp, int c, int32_t v, bool onlyPreferred = false) {
    while (c >= 0) {
        int64_t first, size;
        QueueShare(tilesBig, tilesSmall, c, &first, &size);
        if (v < size) return QueueDraw{c & 1, static_cast<int32_t>(first + v), usedUp};
        usedUp |= 1u << c;
        // a look at all sixteen counters at once (one round trip) spares a failed draw, i.e. a round trip, per used-up share
        int32_t now[2 * kXcds];  // fully unrolled below: stays in registers
#pragma unroll
        for (int i = 0; i < 2 * kXcds; ++i) now[i] = __hip_atomic_load(counters + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
        for (int i = 0; i < 2 * kXcds; ++i) {
            QueueShare(tilesBig, tilesSmall, i, &first, &size);
            if (now[i] >= size) usedUp |= 1u << i;
        }
        c = QueueFirstOpen(usedUp, home, prefer, onlyPreferred);
        if (c >= 0) v = QueueTake(counters, c);
    }
    return QueueDraw{-1, 0, usedUp};
}

// Output channel held in row r of the weight tile (clamped: channels past N are loaded but never stored).
template <bool kSwiglu>
__device__ __forceinline__ int32_t ChannelOfRow(const KernelArgs& a, const TileInfo& t, int r) {
    int32_t n;
    if (kSwiglu) n = r < kTileN / 2 ? t.colBase + r : a.halfN + t.colBase + (r - kTileN / 2);
    else n = t.colBase + r;
    return n < a.N ? n : a.N - 1;
}

__device__ __forceinline__ float LoadScale(const void* p, int64_t i, int dtype) {
    if (dtype == 0) return static_cast<const float*>(p)[i];
    const uint16_t raw = static_cast<const uint16_t*>(p)[i];
    if (dtype == 1) return __half2float(__ushort_as_half(raw));
    return __uint_as_float(static_cast<uint32_t>(raw) << 16);
}

// fp32 -> fp16, round to nearest even, of a value that is itself an fp32 result.  The reference rounds its products to
// fp32 and then casts; left in sight of each other, a multiply and this conversion are merged by the compiler into one
// v_fma_mixlo_f16, which rounds the exact product once -- a different value in the rare double-rounding cases.  The
// empty statement hides the value's origin.
__device__ __forceinline__ uint16_t HalfBitsOfRounded(float f) {
    asm("" : "+v"(f));
    return __half_as_ushort(__float2half_rn(f));
}

// Byte offset of (channel n, k = 0) inside one expert's weights; consecutive k are a.wStrideK bytes apart (32 in the
// blocked layout: a 32-channel block holds its K rows of 32 channel bytes back to back).
__device__ __forceinline__ int64_t WeightRowBase(const KernelArgs& a, int32_t n) {
    return a.wNz ? static_cast<int64_t>(n >> 5) * a.K * 32 + (n & 31) : static_cast<int64_t>(n) * a.wStrideN;
}

// Epilogue of one tile.  acc[mi][ni][v] is C[row, col] with row = waveRow0 + 32*mi + 8*(v/4) + 4*lhi + (v%4); the wave
// owns column blocks ni = 0, 1, lane l32 inside each (plain: 64*waveN + 32*ni; kSwiglu: S column 32*waveN and its partner).
// Only the first mySub accumulator tiles of the wave are real.  ldsRowScale holds the tile's per-row scales.
// afterScaleLoads() is called once the channel scales of the tile have been requested and before anything is stored: a
// memory request made there queues behind loads whose answers the epilogue needs first, not in front of them.
struct NoHook {
    __device__ __forceinline__ void operator()() const {}
};
//
// A wave that holds kNi = 4 column blocks (four waves per tile, 128 x 128 each) calls the per-wave part once per pair
// of blocks: kPair picks acc[mi][2 * kPair] and acc[mi][2 * kPair + 1], and waveN is then the column position
// 0..3 that this pair has in the tile (what the wave index is when eight waves hold one pair each).
template <int kSubM, int kNi, int kPair, int kTileM, Epilogue kEpi, typename Hook = NoHook>
__device__ __forceinline__ void TileEpilogueWave(const KernelArgs& a, const TileInfo& t, v16i (&accAll)[kSubM][kNi], int mySub,
                                                 int waveRow0, int waveN, int l32, int lhi,
                                                 const float* ldsRowScale, float* ldsRowMax, Hook afterScaleLoads = NoHook{}) {
    // the pair's two accumulator columns under the name the code below uses: acc(mi, 0 / 1)
    auto acc = [&](int mi, int j) __attribute__((always_inline)) -> v16i& { return accAll[mi][2 * kPair + j]; };
    const int32_t rows = t.rows, rowBase = t.rowBase, group = t.group;
    // The row / address arithmetic below depends only on the lane; hoisted out of the persistent tile loop it would
    // stay alive across the whole kernel and spill, and a reload in here waits for every store issued so far.  An
    // opaque per-call zero folded into the lane index keeps the arithmetic inside the epilogue.
    int opaqueZero;
    asm volatile("v_mov_b32 %0, 0" : "=v"(opaqueZero));
    lhi += opaqueZero;
    l32 += opaqueZero;
    if (kEpi == Epilogue::kInt32 || kEpi == Epilogue::kDequant) {
        const bool hasRowScale = a.rowScale != nullptr;
        const int32_t n0 = t.colBase + 64 * waveN + l32;  // column block 0; block 1 is 32 columns further
        const bool valid0 = n0 < a.N, valid1 = n0 + 32 < a.N;
        float sc0 = 0.0f, sc1 = 0.0f;
        if (kEpi == Epilogue::kDequant) {
            if (valid0) sc0 = LoadScale(a.scale, static_cast<int64_t>(group) * a.N + n0, a.scaleDtype);
            if (valid1) sc1 = LoadScale(a.scale, static_cast<int64_t>(group) * a.N + n0 + 32, a.scaleDtype);
        }
        float bias0 = 0.0f, bias1 = 0.0f;
        if (kEpi == Epilogue::kDequant && a.bias != nullptr) {
            if (valid0) bias0 = LoadScale(a.bias, static_cast<int64_t>(group) * a.N + n0, a.biasDtype);
            if (valid1) bias1 = LoadScale(a.bias, static_cast<int64_t>(group) * a.N + n0 + 32, a.biasDtype);
        }
        afterScaleLoads();
        // 16-bit outputs: a lane holds one column of each block, i.e. 2-byte pieces 64 bytes apart.  Neighbouring lanes
        // swap one value so that an even lane owns columns (c, c+1) of block 0 and the odd lane next to it the same pair
        // of block 1; every lane then stores one aligned 32-bit word and a half-wave covers a whole 128-byte row segment.
        const bool pairStores = kEpi == Epilogue::kDequant && a.outDtype != 0 && (a.N & 1) == 0 &&
                                t.colBase + 64 * waveN + 64 <= a.N;  // wave-uniform
        const bool oddLane = (l32 & 1) != 0;
        if (kEpi == Epilogue::kDequant && (a.outDtype == 27 || a.outDtype == 1) && pairStores) {
            const bool toBf16 = a.outDtype == 27;  // wave-uniform: bf16, else fp16
            // The common case (16-bit output, whole column pairs) without per-element dtype dispatch: row scales come
            // from LDS four at a time, every lane stores one 32-bit word per accumulator pair through a
            // (uniform row pointer + 32-bit lane offset) address.
            uint16_t* const outTile = static_cast<uint16_t*>(a.out) + static_cast<int64_t>(rowBase + waveRow0) * a.N;
            const int32_t laneOff = 4 * lhi * a.N + (oddLane ? n0 + 31 : n0);
#pragma unroll
            for (int mi = 0; mi < kSubM; ++mi) {
                const int rTop = waveRow0 + 32 * mi;
                if (mi >= mySub || rTop >= rows) continue;
                // The row checks are made per group of eight rows (accumulator entries 4q .. 4q + 3 of the two lane
                // halves), wave-uniformly: a group wholly inside the expert's rows takes a copy of the code without
                // checks, a group wholly outside is skipped, and only the one group that straddles the last row tests
                // every lane.  A per-lane test makes every element a predicated basic block of its own, and the
                // independent chains of a tile no longer interleave.
                // the tile's 32 row scales, read in one go (one wave-uniform test instead of one per row group)
                float4 rsTile[4];
#pragma unroll
                for (int q = 0; q < 4; ++q) rsTile[q] = make_float4(1.0f, 1.0f, 1.0f, 1.0f);  // multiplying by 1 is exact
                if (hasRowScale) {
#pragma unroll
                    for (int q = 0; q < 4; ++q) rsTile[q] = *reinterpret_cast<const float4*>(ldsRowScale + rTop + 8 * q + 4 * lhi);
                }
                auto rowGroup = [&](int q, auto fullTag, auto bf16Tag) __attribute__((always_inline)) {
                    constexpr bool kFull = decltype(fullTag)::value;
                    constexpr bool kToBf16 = decltype(bf16Tag)::value;  // compile-time: a run-time choice per element splits the block
                    const float4 rs = rsTile[q];
                    const float rsv[4] = {rs.x, rs.y, rs.z, rs.w};
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int v = 4 * q + i;
                        const Float2 f = {__fmul_rn(__fmul_rn(static_cast<float>(acc(mi, 0)[v]), sc0), rsv[i]),
                                          __fmul_rn(__fmul_rn(static_cast<float>(acc(mi, 1)[v]), sc1), rsv[i])};
                        uint32_t pk;
                        if constexpr (kToBf16) {
                            pk = __builtin_bit_cast(uint32_t, __builtin_convertvector(f, Bf16x2));
                        } else {
                            pk = static_cast<uint32_t>(HalfBitsOfRounded(f[0])) | (static_cast<uint32_t>(HalfBitsOfRounded(f[1])) << 16);
                        }
                        const uint32_t got = static_cast<uint32_t>(__builtin_amdgcn_mov_dpp(static_cast<int>(pk), 0xB1, 0xF, 0xF, true));
                        const uint32_t word = __builtin_amdgcn_perm(got, pk, oddLane ? 0x03020706u : 0x05040100u);
                        uint16_t* const rowPtr = outTile + static_cast<int64_t>(32 * mi + 8 * q + i) * a.N;
                        if (kFull || rTop + 8 * q + 4 * lhi + i < rows) __builtin_nontemporal_store(word, reinterpret_cast<uint32_t*>(rowPtr + laneOff));
                    }
                };
                auto rowsOfTile = [&](auto bf16Tag) __attribute__((always_inline)) {
                    if (rTop + 32 <= rows) {
#pragma unroll
                        for (int q = 0; q < 4; ++q) rowGroup(q, std::true_type{}, bf16Tag);
                    } else {
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            if (rTop + 8 * q >= rows) break;
                            if (rTop + 8 * q + 8 <= rows) rowGroup(q, std::true_type{}, bf16Tag);
                            else rowGroup(q, std::false_type{}, bf16Tag);
                        }
                    }
                };
                if (toBf16) rowsOfTile(std::true_type{});
                else rowsOfTile(std::false_type{});
            }
            return;
        }
#pragma unroll
        for (int mi = 0; mi < kSubM; ++mi) {
            if (mi >= mySub || waveRow0 + 32 * mi >= rows) continue;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int r = waveRow0 + 32 * mi + 8 * (v / 4) + 4 * lhi + (v % 4);
                const int64_t rowOff = static_cast<int64_t>(rowBase + r) * a.N;
                if (kEpi == Epilogue::kInt32) {
                    if (r < rows && valid0) static_cast<int32_t*>(a.out)[rowOff + n0] = acc(mi, 0)[v];
                    if (r < rows && valid1) static_cast<int32_t*>(a.out)[rowOff + n0 + 32] = acc(mi, 1)[v];
                    continue;
                }
                float y0 = __fmul_rn(static_cast<float>(acc(mi, 0)[v]), sc0);
                float y1 = __fmul_rn(static_cast<float>(acc(mi, 1)[v]), sc1);
                if (hasRowScale) {
                    const float rs = ldsRowScale[r < rows ? r : 0];
                    y0 = __fmul_rn(y0, rs);
                    y1 = __fmul_rn(y1, rs);
                }
                if (a.outDtype == 0) {
                    if (a.combineIndex != nullptr) {
                        if (r >= rows) continue;
                        const int64_t src = rowBase + r;
                        const int64_t dst = a.combineIndexIsInt64 ? static_cast<const int64_t*>(a.combineIndex)[src]
                                                                  : static_cast<const int32_t*>(a.combineIndex)[src];
                        if (dst < 0 || dst >= a.combineRows) continue;
                        if (a.bias != nullptr) {
                            const float wgt = a.combineWeight != nullptr ? a.combineWeight[src] : 1.0f;
                            y0 = __fadd_rn(y0, __fmul_rn(wgt, bias0));
                            y1 = __fadd_rn(y1, __fmul_rn(wgt, bias1));
                        }
                        float* const dstRow = static_cast<float*>(a.out) + dst * a.N;
                        if (valid0) unsafeAtomicAdd(dstRow + n0, y0);
                        if (valid1) unsafeAtomicAdd(dstRow + n0 + 32, y1);
                        continue;
                    }
                    if (r < rows && valid0) static_cast<float*>(a.out)[rowOff + n0] = y0;
                    if (r < rows && valid1) static_cast<float*>(a.out)[rowOff + n0 + 32] = y1;
                    continue;
                }
                // both values rounded to nearest even and packed (low half = block 0)
                uint32_t pk;
                if (a.outDtype == 27) {
                    const Float2 f = {y0, y1};
                    pk = __builtin_bit_cast(uint32_t, __builtin_convertvector(f, Bf16x2));  // v_cvt_pk_bf16_f32
                } else {
                    pk = static_cast<uint32_t>(HalfBitsOfRounded(y0)) | (static_cast<uint32_t>(HalfBitsOfRounded(y1)) << 16);
                }
                if (pairStores) {
                    // quad_perm [1,0,3,2]: exchange with the lane whose index differs in bit 0, then keep
                    // (own block-0 value, neighbour's block-0 value) on even lanes and
                    // (neighbour's block-1 value, own block-1 value) on odd lanes
                    const uint32_t got = static_cast<uint32_t>(__builtin_amdgcn_mov_dpp(static_cast<int>(pk), 0xB1, 0xF, 0xF, true));
                    const uint32_t word = __builtin_amdgcn_perm(got, pk, oddLane ? 0x03020706u : 0x05040100u);
                    const int32_t col = oddLane ? n0 + 31 : n0;  // odd lane l: block 1, columns 32 + (l - 1), 32 + l
                    if (r < rows) *reinterpret_cast<uint32_t*>(static_cast<uint16_t*>(a.out) + rowOff + col) = word;
                } else {
                    if (r < rows && valid0) static_cast<uint16_t*>(a.out)[rowOff + n0] = static_cast<uint16_t>(pk & 0xffffu);
                    if (r < rows && valid1) static_cast<uint16_t*>(a.out)[rowOff + n0 + 32] = static_cast<uint16_t>(pk >> 16);
                }
            }
        }
    } else {
        const int32_t j = t.colBase + 32 * waveN + l32;  // column of S
        const bool jValid = j < a.halfN;
        float scA = 0.0f, scB = 0.0f;
        if (jValid) {
            scA = LoadScale(a.scale, static_cast<int64_t>(group) * a.N + j, a.scaleDtype);
            scB = LoadScale(a.scale, static_cast<int64_t>(group) * a.N + a.halfN + j, a.scaleDtype);
        }
        afterScaleLoads();
        const bool wholeColumns = t.colBase + 32 * waveN + 32 <= a.halfN;  // wave-uniform
#pragma unroll
        for (int mi = 0; mi < kSubM; ++mi) {
            if (mi >= mySub) continue;  // wave-uniform
            const int rTop = waveRow0 + 32 * mi;
            if (wholeColumns && rTop < rows) {
                // Fast form for whole column blocks: row scales four at a time, no column checks, and the 16 row
                // maxima of the MFMA tile reduced across the 32 lanes by a halving butterfly (16 exchanges, not 80).
                float* const sTile = a.sOut + static_cast<int64_t>(rowBase + rTop) * a.halfN;
                const int32_t laneOff = 4 * lhi * a.halfN + j;
                float m[16];
                // Row checks per group of eight rows, wave-uniformly, as in the 16-bit stores above.
                auto rowGroup = [&](int q, auto fullTag) __attribute__((always_inline)) {
                    constexpr bool kFull = decltype(fullTag)::value;
                    const float4 xs4 = *reinterpret_cast<const float4*>(ldsRowScale + rTop + 8 * q + 4 * lhi);
                    const float xsv[4] = {xs4.x, xs4.y, xs4.z, xs4.w};
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int v = 4 * q + i;
                        const float ca = __fmul_rn(__fmul_rn(static_cast<float>(acc(mi, 0)[v]), xsv[i]), scA);
                        const float cb = __fmul_rn(__fmul_rn(static_cast<float>(acc(mi, 1)[v]), xsv[i]), scB);
                        float sv = __fmul_rn(__fmul_rn(ca, __builtin_amdgcn_rcpf(__fadd_rn(1.0f, __expf(-ca)))), cb);
                        const bool ok = kFull || rTop + 8 * q + 4 * lhi + i < rows;
                        if (ok) __builtin_nontemporal_store(sv, &sTile[static_cast<int64_t>(8 * q + i) * a.halfN + laneOff]);
                        m[v] = ok ? fabsf(sv) : 0.0f;
                    }
                };
                if (rTop + 32 <= rows) {
#pragma unroll
                    for (int q = 0; q < 4; ++q) rowGroup(q, std::true_type{});
                } else {
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        if (rTop + 8 * q >= rows) {
#pragma unroll
                            for (int i = 0; i < 4; ++i) m[4 * q + i] = 0.0f;
                        } else if (rTop + 8 * q + 8 <= rows) {
                            rowGroup(q, std::true_type{});
                        } else {
                            rowGroup(q, std::false_type{});
                        }
                    }
                }
                // lanes l and l ^ 16: one instruction trades the upper-row half of m[i] for the lower-row half of
                // m[i + 8]; afterwards lanes 0..15 of each half-wave own v = i and lanes 16..31 own v = i + 8
                typedef unsigned int Uint2 __attribute__((ext_vector_type(2)));
                float k8[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const Uint2 sw = __builtin_amdgcn_permlane16_swap(__float_as_uint(m[i]), __float_as_uint(m[i + 8]), false, false);
                    k8[i] = fmaxf(__uint_as_float(sw[0]), __uint_as_float(sw[1]));
                }
                const bool b3 = (l32 & 8) != 0, b2 = (l32 & 4) != 0, b1 = (l32 & 2) != 0;
                float k4[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {  // partner l ^ 8: lanes with bit 3 clear keep i, the others i + 4
                    const float send = b3 ? k8[i] : k8[i + 4];
                    k4[i] = fmaxf(b3 ? k8[i + 4] : k8[i], __shfl_xor(send, 8, 64));
                }
                float k2[2];
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    const float send = b2 ? k4[i] : k4[i + 2];
                    k2[i] = fmaxf(b2 ? k4[i + 2] : k4[i], __shfl_xor(send, 4, 64));
                }
                const float send1 = b1 ? k2[0] : k2[1];
                float k1 = fmaxf(b1 ? k2[1] : k2[0], __shfl_xor(send1, 2, 64));
                k1 = fmaxf(k1, __shfl_xor(k1, 1, 64));
                // the lane pair (2p, 2p + 1) of a half-wave now holds the maximum of accumulator index v = p:
                // bit 4 of the lane chose bit 3 of v, bit 3 -> bit 2, bit 2 -> bit 1, bit 1 -> bit 0
                const int v = l32 >> 1;
                if ((l32 & 1) == 0) ldsRowMax[waveN * kTileM + rTop + 8 * (v / 4) + 4 * lhi + (v % 4)] = k1;
                continue;
            }
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int r = waveRow0 + 32 * mi + 8 * (v / 4) + 4 * lhi + (v % 4);
                const bool valid = r < rows && jValid;
                float s = 0.0f;
                if (valid) {
                    const float xs = ldsRowScale[r];
                    const float ca = __fmul_rn(__fmul_rn(static_cast<float>(acc(mi, 0)[v]), xs), scA);
                    const float cb = __fmul_rn(__fmul_rn(static_cast<float>(acc(mi, 1)[v]), xs), scB);
                    // swish(ca) * cb with the hardware exp2 / reciprocal: a few ulp from the correctly rounded value,
                    // far inside the +-1 LSB the int8 requantisation is held to
                    s = __fmul_rn(__fmul_rn(ca, __builtin_amdgcn_rcpf(__fadd_rn(1.0f, __expf(-ca)))), cb);
                    a.sOut[static_cast<int64_t>(rowBase + r) * a.halfN + j] = s;
                }
                // max |S| of this row over the wave's 32 columns, kept by the first lane of each half-wave
                float m = fabsf(s);
#pragma unroll
                for (int d = 1; d < 32; d <<= 1) m = fmaxf(m, __shfl_xor(m, d, 64));
                if (l32 == 0) ldsRowMax[waveN * kTileM + r] = m;
            }
        }
    }
}

// The part of the kSwiglu epilogue that follows the waves' own work: folds the four column positions' partial row maxima
// into one per (n-tile, row).  Contains a workgroup barrier: every wave must call it (the workgroup has at least
// kTileM threads).
template <int kTileM>
__device__ __forceinline__ void TileEpilogueFoldMax(const KernelArgs& a, const TileInfo& t, int tid, const float* ldsRowMax) {
    __syncthreads();
    // one partial maximum per (n-tile, row): no atomics and nothing to pre-zero; the requantisation folds them
    if (tid < t.rows) {
        float m = ldsRowMax[tid];
#pragma unroll
        for (int w = 1; w < kWavesN; ++w) m = fmaxf(m, ldsRowMax[w * kTileM + tid]);
        a.rowMax[static_cast<int64_t>(t.tileN) * a.M + t.rowBase + tid] = m;
    }
}

// Eight-wave form (one pair of column blocks per wave): the per-wave part, then the fold.
template <int kSubM, int kTileM, Epilogue kEpi, typename Hook = NoHook>
__device__ __forceinline__ void TileEpilogue(const KernelArgs& a, const TileInfo& t, v16i (&acc)[kSubM][2], int mySub,
                                             int waveRow0, int waveN, int l32, int lhi, int tid,
                                             const float* ldsRowScale, float* ldsRowMax, Hook afterScaleLoads = NoHook{}) {
    TileEpilogueWave<kSubM, 2, 0, kTileM, kEpi>(a, t, acc, mySub, waveRow0, waveN, l32, lhi, ldsRowScale, ldsRowMax, afterScaleLoads);
    if (kEpi == Epilogue::kSwiglu) TileEpilogueFoldMax<kTileM>(a, t, tid, ldsRowMax);
}

// Calls f(std::integral_constant<int, n>) for n = count clamped into 0..kMax.
template <int kMax, typename F>
__device__ __forceinline__ void ForCount(int count, F& f) {
    if constexpr (kMax == 0) {
        f(std::integral_constant<int, 0>{});
    } else {
        if (count >= kMax) f(std::integral_constant<int, kMax>{});
        else ForCount<kMax - 1>(count, f);
    }
}

// ---------------------------------------------------------------------------------------------- fast path: LDS-DMA ring
// kStep = k-bytes per ring stage: 128 streams weights in whole 128-byte lines (best HBM efficiency).
// The tile's rows are split over one or two wave rows: wave row 0 owns kSub0 MFMA tiles (32 rows each), wave row 1 the
// next kSub1 (kSub1 <= kSub0; kSub1 == 0 means four waves only).
//
// A stage is kTileM activation rows and kTileN weight channels of kStep k-bytes each.  Every wave fetches, per stage,
// instructions wave, wave + kWaves, ... of the stage's list (activation part first, then weight part).
//
// Common depth (every height but 192 rows): a ring of whole stages.
//
// Staggered depths (192 rows).  Whole stages fit twice there, but three weight stages and two activation stages fit as
// well -- and the depth matters for the weights, which come out of HBM, not for the activation rows, which the n-tiles
// of an expert re-read from L2.  So the two parts live in rings of their own depth (the activation ring first), and
// each has its own issue cursor: at k-step s a wave issues its activation share of step s + 2 and then its weight share
// of step s + 3.  A wave's loads return in issue order; with the activation share going out first, "at most one weight
// share outstanding" certifies both the activation stage issued one step ago and the weight stage issued two steps ago.
//
// kWn = waves side by side along the channels: four (a wave owns 64 channels, two MFMA column blocks) or two (128
// channels, four column blocks: with two wave rows that is four waves per workgroup, one per SIMD, each holding a
// 128 x 128 block of the tile -- a third fewer fragment bytes out of LDS per MFMA, the accumulators in AccVGPRs).
// Only kWn = 4 is launched.  The four-wave form of the 256-row tile gives the same bits and measured 16 % slower on the
// matrix-bound shape (4.14 against 3.58 ms): with one wave per SIMD nothing runs under a wave's sixteen operand
// requests per k-step or under its epilogue, and what it saves in LDS reads is not what bounds the step.
template <int kSub0, int kSub1, int kStep, int kWn = kWavesN>
struct StreamCfg {
    static_assert(kSub1 <= kSub0, "wave row 0 is the taller one");
    static_assert(kWn == 4 || kWn == 2, "a wave owns two or four column blocks");
    static constexpr int kWavesM = kSub1 > 0 ? 2 : 1;
    static constexpr int kWaves = kWn * kWavesM;
    static constexpr int kNi = kTileN / 32 / kWn;  // MFMA column blocks per wave
    static constexpr int kThreads = 64 * kWaves;
    static constexpr int kTileM = 32 * (kSub0 + kSub1);
    static constexpr int kStageBytesA = kTileM * kStep;
    static constexpr int kStageBytesB = kTileN * kStep;
    static constexpr int kQueueLdsInts = 16;  // the workgroup's tile sequence (four {list, tile} pairs) and its draw state
    static constexpr int kScratchBytes = (1 + kWavesN) * kTileM * 4 + kQueueLdsInts * 4;
    static constexpr bool kStaggered = kTileM == 192;
    static constexpr int kFitWhole = (kLdsBudget - kScratchBytes) / (kStageBytesA + kStageBytesB);
    static constexpr int kStagesB = kStaggered ? (kLdsBudget - kScratchBytes - 2 * kStageBytesA) / kStageBytesB
                                               : (kFitWhole > 8 ? 8 : kFitWhole);
    static constexpr int kStagesA = kStaggered ? 2 : kStagesB;
    static constexpr int kLdsBytes = kStagesA * kStageBytesA + kStagesB * kStageBytesB + kScratchBytes;
    // one DMA instruction moves 64 lanes x 16 bytes = kRowsPerInstr tile rows of kStep k-bytes
    static constexpr int kChunksPerRow = kStep / kChunk;
    static constexpr int kRowsPerInstr = 64 / kChunksPerRow;
    static constexpr int kInstrA = kTileM / kRowsPerInstr;
    static constexpr int kInstrB = kTileN / kRowsPerInstr;
    static constexpr int kInstr = kInstrA + kInstrB;
    static_assert(kTileM % kRowsPerInstr == 0, "tile rows must fill whole DMA instructions");
    static_assert(kThreads >= kTileM, "one thread per tile row stages the row scales and folds the row maxima");
    // Every wave issues exactly kMaxPerWave DMA instructions per stage: slots past the last instruction repeat it (same
    // bytes to the same place), which keeps the issue code free of branches and the vmcnt arithmetic uniform.
    static constexpr int kMaxPerWave = (kInstr + kWaves - 1) / kWaves;
    // staggered depths: the first kSlotsA slots of every wave are activation instructions, the others weight instructions
    static constexpr int kSlotsA = kInstrA / kWaves;
    static constexpr int kSlotsB = kMaxPerWave - kSlotsA;
    static_assert(!kStaggered || (kInstrA % kWaves == 0 && kInstrB % kWaves == 0), "the same split of slots in every wave");
    static_assert(kStagesA >= 2 && kStagesB >= kStagesA, "each ring needs at least two stages");
    static_assert(kStagesB * kMaxPerWave <= 63, "vmcnt is a 6-bit counter");
};

// Byte offset of 16-byte chunk `chunk` of row `row` in a stage whose rows are kStep bytes.  The LDS serves 16 lanes per
// clock out of 64 banks (256 bytes): the chunk index is XOR-ed with row bits such that 16 consecutive rows reading the
// same logical chunk land in 16 different 16-byte bank groups.
template <int kStep>
__device__ __forceinline__ int LdsOffset(int row, int chunk) {
    if (kStep == 64) return row * 64 + ((chunk ^ ((row >> 2) & 3)) << 4);
    return row * 128 + ((chunk ^ ((row >> 1) & 7)) << 4);
}

// A wave-uniform pointer, forced into scalar registers.
__device__ __forceinline__ const char* UniformPtr(const char* p) {
    const uint64_t b = reinterpret_cast<uint64_t>(p);
    const uint32_t lo = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(static_cast<uint32_t>(b))));
    const uint32_t hi = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(static_cast<uint32_t>(b >> 32))));
    return reinterpret_cast<const char*>(static_cast<uint64_t>(lo) | (static_cast<uint64_t>(hi) << 32));
}

// The 32-bit LDS address of a generic pointer into LDS (wave-uniform).
__device__ __forceinline__ uint32_t LdsAddress(const char* p) {
    typedef __attribute__((address_space(3))) const char* LdsPtr;
    return static_cast<uint32_t>(
        __builtin_amdgcn_readfirstlane(static_cast<int>(static_cast<uint32_t>(reinterpret_cast<size_t>((LdsPtr)p)))));
}

// 16 bytes per lane from (uniform base + 32-bit lane offset) straight into LDS at ldsAddr + lane * 16 (ldsAddr is the
// 32-bit LDS address, see LdsAddress).  The compiler does not see this as a memory instruction: completion is awaited
// with WaitVmcnt below.
// kStreaming marks the load non-temporal: the bytes are used once (weights), so they should not push the operands
// that are re-read from L2 (activation rows) out of the caches.
// The instruction takes its LDS base from m0, which the statement sets itself.  m0 is a reserved register that cannot
// be named as a clobber; nothing else in these kernels uses it (no LDS-direct or register-indexed code is generated
// for them), and the compiler sets m0 afresh before any use of its own.
template <bool kStreaming>
__device__ __forceinline__ void DmaToLdsAddr16(const char* base, uint32_t laneOffset, uint32_t ldsAddr) {
    const uint32_t m0 = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(ldsAddr)));
    const char* const sbase = UniformPtr(base);
    if (kStreaming) {
        asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2 nt" ::"s"(m0), "v"(laneOffset), "s"(sbase) : "memory");
    } else {
        asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(m0), "v"(laneOffset), "s"(sbase) : "memory");
    }
}

// The value itself, through a statement the optimiser cannot see through: what is computed from the copy stays where it
// is written.  Used on lane indices at the head of per-tile code, so that the per-lane offsets and addresses of that code
// are recomputed once per tile instead of being hoisted out of the tile loop and held in registers (or spilled) across the
// k loop, where the accumulators and fragments of the tallest tiles leave no room for them.
__device__ __forceinline__ int Opaque(int v) {
    asm volatile("" : "+v"(v));
    return v;
}

template <int kCount>
__device__ __forceinline__ void WaitVmcnt() {  // s_waitcnt vmcnt(kCount), leaving expcnt / lgkmcnt untouched
    __builtin_amdgcn_s_waitcnt(0x0f70 | (kCount & 15) | ((kCount >> 4) << 14));
}

// Persistent: the grid is one workgroup per CU (a multiple of 8); workgroup b serves XCD b % 8 and walks that XCD's
// share of the tile list with stride gridDim / 8.
//
// kNz: the weights come in the 32-channel x 16-k blocked layout.  A 32-channel block is then one contiguous stream of
// K x 32 bytes, so a stage's weight part is eight 4 KB pieces that land in LDS as [block][k][32 channels]; the MFMA
// operand (16 consecutive k of one channel per lane) is read back with the transposing LDS load ds_read_b64_tr_b8:
// per 16 lanes, lanes 2r and 2r + 1 supply the two 8-byte halves of row r (r = 0..7) and lane i receives column i,
// i.e. with rows = 8 consecutive k and columns = 16 channels each lane gets 8 consecutive k of its channel.
//
// kNMajor: the weights are row-major [K, N] per expert (N contiguous), the reference's plain ND layout of the grouped
// matmul.  A stage's weight part is then 128 k-rows of the tile's 256 channel bytes (one 256-byte run per k-row, two of
// 128 bytes for the gate and up halves of a SwiGLU tile); it lies in LDS as [k][256] with the 16-byte chunk index of row
// k XOR-ed by 2 * (k & 7), and the operands come out through the same transposing load as for the blocked layout: the
// 32 lanes the LDS serves together read one pair of neighbouring chunks from each of 8 consecutive k-rows, and the
// swizzle puts those 8 pairs into 8 different bank groups (a row of 256 bytes spans all 64 banks once).
//
// kRun: which runs of the m-tile table the body serves.  kBothRuns: all of it (pulled or in fixed shares).  kBigRun /
// kSmallRun: that run only, pulled, until its counters are used up on every XCD -- the form in which MixedGemmKernel
// calls the body twice, once per run with a stage geometry of that run's own.
constexpr int kBigRun = 0, kSmallRun = 1, kBothRuns = 2;
template <int kSub0, int kSub1, int kStep, Epilogue kEpi, bool kNz, bool kNMajor, int kWn, int kRun>
__device__ __forceinline__ void StreamGemmBody(const KernelArgs& a, const int32_t* __restrict__ sched, char* const lds,
                                               uint64_t& spanTiles) {
    static_assert(!(kNz || kNMajor) || kStep == 128, "the blocked and row-major weight layouts are built for 128-byte k-steps");
    static_assert(!(kNz && kNMajor), "one weight layout at a time");
    using Cfg = StreamCfg<kSub0, kSub1, kStep, kWn>;
    constexpr int kSubM = kSub0;  // accumulator tiles per wave (wave row 1 uses the first kSub1 of them)
    constexpr int kNi = Cfg::kNi;
    constexpr int kTileM = Cfg::kTileM;
    constexpr int kStagesA = Cfg::kStagesA, kStagesB = Cfg::kStagesB;
    constexpr int kStageBytesA = Cfg::kStageBytesA, kStageBytesB = Cfg::kStageBytesB;
    // LDS layout.  Common depth: stage after stage, each its activation part followed by its weight part.  Staggered
    // depths: the ring of activation stages, behind it the ring of weight stages.
    constexpr bool kStaggered = Cfg::kStaggered;
    constexpr int kStrideA = kStaggered ? kStageBytesA : kStageBytesA + kStageBytesB;  // from one activation stage to the next
    constexpr int kStrideB = kStaggered ? kStageBytesB : kStageBytesA + kStageBytesB;
    constexpr int kFirstB = kStaggered ? kStagesA * kStageBytesA : kStageBytesA;       // weight part of stage 0
    constexpr bool kSwiglu = kEpi == Epilogue::kSwiglu;
    float* const ldsRowScale = reinterpret_cast<float*>(lds + kStagesA * kStageBytesA + kStagesB * kStageBytesB);  // [kTileM]
    float* const ldsRowMax = ldsRowScale + kTileM;                                      // [kWavesN][kTileM]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int waveN = wave % kWn;
    const int waveM = wave / kWn;
    const int l32 = lane & 31;
    const int lhi = lane >> 5;

    // ---- this workgroup's sequence of tiles ----
    // Workgroup b serves XCD b % 8 as its slot b / 8.  With a.pullTiles the sequence comes out of the tile counters (see
    // QueueShare): thread 0 draws, the result reaches the other waves through a four-entry ring in LDS, and tile n + 2
    // is drawn while tile n's epilogue runs (the draw goes out at its head, the answer is looked at behind it),
    // because the issue side already reads tile n + 1's operands during tile n.  Otherwise the two runs of
    // the m-tile table are one list cut into eight fixed shares, which the workgroups of an XCD walk with stride
    // gridDim / 8.
    const int32_t* const queueHdr = sched;
    const int32_t countBig = queueHdr[0], countSmall = queueHdr[1];  // m-tiles per list
    const int32_t bandBig = queueHdr[4], bandSmall = queueHdr[5];
    const int4* const mTileTable = reinterpret_cast<const int4*>(queueHdr + kQueueHeaderInts + kQueueCounterInts);
    const int xcd = blockIdx.x % kXcds;
    const int32_t slots = gridDim.x / kXcds;
    const int32_t slot = blockIdx.x / kXcds;
    constexpr bool kOneRun = kRun != kBothRuns;
    const bool pull = kOneRun || a.pullTiles != 0;
    const int64_t bigTiles = static_cast<int64_t>(countBig) * a.tilesN;
    const int64_t totalTiles = bigTiles + static_cast<int64_t>(countSmall) * a.tilesN;
    const int64_t perXcd = (totalTiles + kXcds - 1) / kXcds;
    const int64_t xcdFirst = static_cast<int64_t>(xcd) * perXcd;
    int32_t* const ldsSeq = reinterpret_cast<int32_t*>(ldsRowMax + kWavesN * kTileM);
    constexpr int kSeqUsedUp = 8, kSeqDrawCounter = 9;  // thread 0's draw state, behind the ring
    // Which list this workgroup draws from first: the small m-tiles get the share of each XCD's workgroups that their
    // cost is of the whole, so that both lists run dry at about the same time; until then a part of the machine
    // streams weights for a handful of rows each while the rest multiplies.
    int prefer = 0;
    {
        const int64_t costSmall = queueHdr[2], costAll = costSmall + queueHdr[3];
        int64_t forSmall = costAll > 0 ? (slots * costSmall + costAll / 2) / costAll : 0;
        if (forSmall == 0 && countSmall > 0 && slots > 1) forSmall = 1;
        if (countBig == 0) forSmall = slots;
        prefer = kOneRun ? kRun : (slot < forSmall ? 1 : 0);
    }
    auto listTile = [&](int32_t list, int64_t logical) __attribute__((always_inline)) {
        return DecodeListTile<kTileM, kSwiglu>(a, mTileTable, list ? countBig : 0, list ? countSmall : countBig,
                                               list ? bandSmall : bandBig, logical);
    };
    // the n-th tile of this workgroup (n at most two ahead of the tile being computed)
    auto tileAt = [&](int32_t n) __attribute__((always_inline)) -> TileInfo {
        if (pull) {
            const int32_t list = __builtin_amdgcn_readfirstlane(ldsSeq[2 * (n & 3)]);
            const int32_t logical = __builtin_amdgcn_readfirstlane(ldsSeq[2 * (n & 3) + 1]);
            if (list < 0) return TileInfo{};
            return listTile(list, logical);
        }
        const int64_t local = slot + static_cast<int64_t>(n) * slots;
        const int64_t logical = xcdFirst + local;
        if (local >= perXcd || logical >= totalTiles) return TileInfo{};
        return logical < bigTiles ? listTile(0, logical) : listTile(1, logical - bigTiles);
    };
    if (pull) {
        if (tid == 0) {
            // the first two tiles: both draws go out together
            uint32_t usedUp = 0;
            const int c = QueueFirstOpen(usedUp, xcd, prefer, kOneRun);
            const int32_t v0 = QueueTake(a.queueCounters, c);
            const int32_t v1 = QueueTake(a.queueCounters, c);
            QueueDraw d = QueueResolve(bigTiles, totalTiles - bigTiles, a.queueCounters, xcd, prefer, usedUp, c, v0, kOneRun);
            ldsSeq[0] = d.list;
            ldsSeq[1] = d.logical;
            if (d.list >= 0) d = QueueResolve(bigTiles, totalTiles - bigTiles, a.queueCounters, xcd, prefer, d.usedUp, c, v1, kOneRun);
            ldsSeq[2] = d.list;
            ldsSeq[3] = d.logical;
            ldsSeq[kSeqUsedUp] = static_cast<int32_t>(d.usedUp);
        }
        __syncthreads();
    }

    int32_t curNo = 0;  // position of the tile being computed in this workgroup's sequence
    TileInfo cur = tileAt(0);
    if (!cur.valid) return;
    const int kSteps = a.K / kStep;
    // Small tiles are the decode shapes: a handful of rows per expert, every weight byte used once, pure streaming.
    constexpr bool kSmallTile = kTileM <= 64;
    const int kRotate = kSmallTile ? static_cast<int>((blockIdx.x * 7u + blockIdx.x / kXcds) % static_cast<unsigned>(kSteps)) : 0;

    // ---- issue side: runs ahead of the compute side by the depth of the ring(s), across tile boundaries ----
    // A cursor walks this workgroup's tiles k-step by k-step.  Cursor B drives the weight part -- and the activation
    // part too where the depths are the same; with staggered depths the activation part has cursor A, one k-step behind.
    // (Plain variables, picked by if constexpr: a cursor struct handed round by reference ends up in vector registers.)
    const uint32_t ldsBase = LdsAddress(lds);
    TileInfo issTileA = cur, issTileB = cur;
    int32_t issNoA = 0, issNoB = 0;            // position of each cursor's tile in the sequence
    int issStepA = 0, issStepB = 0;            // k-step of the tile that goes out next
    int issSlotA = 0, issSlotB = 0;            // ring buffer it goes into
    bool issDrainedA = false, issDrainedB = false;  // no further tile: the issue slots re-read one hot kilobyte (see advance)
    const char* issBaseA = nullptr;  // the tile's activation rows
    const char* issBaseB = nullptr;  // its expert's weights
    uint32_t laneOff[Cfg::kMaxPerWave];
    constexpr int kPartA = 1, kPartB = 2, kBothParts = 3;
    using PartATag = std::integral_constant<int, kPartA>;
    using PartBTag = std::integral_constant<int, kPartB>;
    using BothPartsTag = std::integral_constant<int, kBothParts>;
    // instruction of slot q in the stage's list (activation part, then weight part)
    auto slotInstr = [&](int q) __attribute__((always_inline)) { return min(wave + q * Cfg::kWaves, Cfg::kInstr - 1); };

    // 256-row tiles (the matrix-bound shapes): the tile's two base pointers are moved into scalar registers once per tile,
    // and every slot of a stage is of the same part (activation / weight) in every wave.  A DMA then costs three
    // instructions (LDS address, m0, the load) instead of nine (a select, a 64-bit vector add and two v_readfirstlane
    // on top): the burst of refill requests behind a step's barrier, under which the matrix pipe has little to run, is a
    // third as long.  Same-box A/B: Mixtral prefill gate/up 3.66 -> 3.56 ms, down 1.70 -> 1.67; the 192-row tiles of
    // the HBM-bound shape measured 1.2 % slower with it and keep the vector form.
    constexpr bool kScalarIssue = kTileM >= 256;
    auto scalarBase = [&](const char* p) __attribute__((always_inline)) { return kScalarIssue ? UniformPtr(p) : p; };

    // The lambdas below are forced inline: left to the inliner's size heuristics, one of them staying a real call puts
    // the whole issue state (captured by reference) into scratch memory and the kernel runs three times slower.
    // Bases and lane offsets of the given part(s) for tile t.
    auto setupIssue = [&](const TileInfo& t, auto partsTag) __attribute__((always_inline)) {
        constexpr int kParts = decltype(partsTag)::value;
        if (kParts & kPartA) issBaseA = scalarBase(reinterpret_cast<const char*>(a.x) + static_cast<int64_t>(t.rowBase) * a.K);
        if (kParts & kPartB) issBaseB = scalarBase(reinterpret_cast<const char*>(a.w) + static_cast<int64_t>(t.group) * a.wGroupStride);
        // lane -> (row inside the instruction, LDS chunk slot); the global chunk it fetches is the one LdsOffset puts there
        const int lane = Opaque(tid & 63);
        const int rowIn = lane / Cfg::kChunksPerRow;
        const int slot = lane % Cfg::kChunksPerRow;
#pragma unroll
        for (int q = 0; q < Cfg::kMaxPerWave; ++q) {
            if (kParts != kBothParts && (q < Cfg::kSlotsA) != (kParts == kPartA)) continue;
            const int g = slotInstr(q);
            const int j = g < Cfg::kInstrA ? g : g - Cfg::kInstrA;  // instruction of its part
            if (g < Cfg::kInstrA) {
                // rows past the tile's last row are never used: such lanes re-read the last real row (same cache
                // lines as its own lanes), and an instruction wholly past it reads one chunk, so the number of DMAs
                // per stage stays constant while the activation traffic follows the real row count
                const int r = Cfg::kRowsPerInstr * j + rowIn;
                const int c = (LdsOffset<kStep>(r, slot) >> 4) % Cfg::kChunksPerRow;
                const bool wholeInstrPast = Cfg::kRowsPerInstr * j >= t.rows;
                laneOff[q] = wholeInstrPast ? 0u : static_cast<uint32_t>(min(r, t.rows - 1) * a.K + c * kChunk);
            } else if (kNMajor) {
                // weight instruction j moves k-rows 4 * j .. + 3 of the stage, 256 channel bytes each; lane ->
                // (k-row lane / 16, LDS chunk slot lane % 16), fetching the logical chunk that the swizzle puts there.
                // Chunks past the last channel are never stored: such lanes re-read the last real chunk.
                const int k = 4 * j + lane / 16;
                const int c = (lane % 16) ^ ((k & 7) << 1);
                int32_t col;
                if (kSwiglu) {
                    col = c < 8 ? min(t.colBase + 16 * c, a.halfN - 16) : min(a.halfN + t.colBase + 16 * (c - 8), a.N - 16);
                } else {
                    col = min(t.colBase + 16 * c, a.N - 16);
                }
                laneOff[q] = static_cast<uint32_t>(k * a.N + col);
            } else if (kNz) {
                // weight instruction j moves 32 k-rows (x 32 channel bytes) of channel block j / 4: 1 KB, contiguous
                // in memory and in LDS; lane -> (k-row lane / 2, 16-byte half lane % 2)
                const int32_t block = ChannelOfRow<kSwiglu>(a, t, 32 * (j / 4)) >> 5;
                laneOff[q] = static_cast<uint32_t>(block * a.K * 32 + ((j % 4) * 32 + lane / 2) * 32 + (lane % 2) * kChunk);
            } else {
                const int r = Cfg::kRowsPerInstr * j + rowIn;
                const int c = (LdsOffset<kStep>(r, slot) >> 4) % Cfg::kChunksPerRow;
                laneOff[q] = static_cast<uint32_t>(ChannelOfRow<kSwiglu>(a, t, r) * a.K + c * kChunk);
            }
        }
    };
    // Moves the cursor of the given part(s) to the next k-step (after the last instruction of a stage has gone out).
    auto advance = [&](auto partsTag) __attribute__((always_inline)) {
        constexpr int kParts = decltype(partsTag)::value;
        constexpr bool kCursorA = kParts == kPartA;
        TileInfo& tile = kCursorA ? issTileA : issTileB;
        int32_t& tileNo = kCursorA ? issNoA : issNoB;
        int& step = kCursorA ? issStepA : issStepB;
        int& slot = kCursorA ? issSlotA : issSlotB;
        bool& drained = kCursorA ? issDrainedA : issDrainedB;
        constexpr int kDepth = kCursorA ? kStagesA : kStagesB;
        slot = slot + 1 == kDepth ? 0 : slot + 1;
        if (++step == kSteps) {
            // move to this workgroup's next tile.  Past the last one the issue slots still go out (that keeps the number
            // of outstanding DMAs per stage, hence the vmcnt arithmetic, constant) into ring slots nobody reads -- but
            // every one of them then re-reads the same first kilobyte of the last tile's weights, which stays in L2,
            // instead of pulling more stages of weights from HBM per workgroup.
            step = 0;
            const TileInfo next = tileAt(tileNo + 1);
            if (next.valid) {
                tile = next;
                ++tileNo;
                setupIssue(tile, partsTag);
            } else if (!drained) {
                drained = true;
                // any mapped, 16-byte aligned kilobyte will do: the start of the last tile's expert's weights
                const char* const hot = scalarBase(reinterpret_cast<const char*>(a.w) + static_cast<int64_t>(tile.group) * a.wGroupStride);
                if (kParts & kPartA) issBaseA = hot;
                if (kParts & kPartB) issBaseB = hot;
#pragma unroll
                for (int q = 0; q < Cfg::kMaxPerWave; ++q) {
                    if (kParts != kBothParts && (q < Cfg::kSlotsA) != (kParts == kPartA)) continue;
                    laneOff[q] = static_cast<uint32_t>(lane) * kChunk;
                }
            }
        }
    };
    // This wave's DMA instructions of the given part(s) of the stage at the part's cursor.
    auto emitParts = [&](auto partsTag) __attribute__((always_inline)) {
        constexpr int kParts = decltype(partsTag)::value;
        constexpr bool kOwnA = kParts == kPartA;  // else the activation part, if any, follows cursor B
        // On small tiles the k-steps of a tile are walked from a start that differs between workgroups (integer
        // accumulation does not care about the order).  When rows lie a power-of-two stride apart (K = 4096 with
        // K-contiguous weights), the low address bits of every row of every expert depend on the k offset alone:
        // workgroups that all sit at the same k-step all queue on the same memory channels.  Only for small tiles, where
        // every weight byte is used once: on the large-tile shapes neighbouring workgroups share operands through L2,
        // and walking k in step is what makes those hits.
        auto kOffset = [&](int step, bool drained) __attribute__((always_inline)) {
            const int kIdx = step + kRotate;
            return drained ? 0 : (kIdx >= kSteps ? kIdx - kSteps : kIdx) * kStep;
        };
        const int kOffB = kOffset(issStepB, issDrainedB);
        const int kOffA = kOwnA ? kOffset(issStepA, issDrainedA) : kOffB;
        // weights -- blocked layout: one k is 32 bytes further; row-major: N bytes
        const int kOffW = kNz ? kOffB * 32 : (kNMajor ? kOffB * a.N : kOffB);
        // instruction g lands g KB behind dstA (activation part) or dstB (weight part, whose first instruction is kInstrA)
        const uint32_t dstA = ldsBase + (kOwnA ? issSlotA : issSlotB) * kStrideA;
        const uint32_t dstB = ldsBase + kFirstB + issSlotB * kStrideB - Cfg::kInstrA * 1024;
#pragma unroll
        for (int q = 0; q < Cfg::kMaxPerWave; ++q) {
            if (kParts != kBothParts && (q < Cfg::kSlotsA) != (kParts == kPartA)) continue;
            const int g = slotInstr(q);
            // where the activation instructions divide evenly among the waves, slot q is of the same part in every wave
            constexpr bool kStaticSplit = kScalarIssue && Cfg::kInstrA % Cfg::kWaves == 0;
            const bool isA = kStaticSplit ? q < Cfg::kInstrA / Cfg::kWaves : g < Cfg::kInstrA;
            // wave-uniform choice: activation rows always stay cacheable (the n-tiles of a group re-read them from L2);
            // on small tiles (every weight byte is used exactly once) the weights stream past the caches.  On large
            // tiles the m-tiles of a group share their weight columns through L2 and must not.
            if constexpr (kSmallTile) {
                if (isA) DmaToLdsAddr16<false>(issBaseA + kOffA, laneOff[q], dstA + g * 1024);
                else DmaToLdsAddr16<true>(issBaseB + kOffW, laneOff[q], dstB + g * 1024);
            } else {  // selects, no branch: the k-step stays one basic block
                DmaToLdsAddr16<false>(isA ? issBaseA + kOffA : issBaseB + kOffW, laneOff[q], (isA ? dstA : dstB) + g * 1024);
            }
        }
    };
    // One k-step's worth of issue: a whole stage, or (staggered depths) the activation share and then the weight share,
    // each of the stage its own cursor has reached.
    // The cursors move when all of it has gone out, so that the DMAs of a k-step stay in one basic block.
    auto issueStage = [&]() __attribute__((always_inline)) {
        if constexpr (kStaggered) {
            emitParts(PartATag{});
            emitParts(PartBTag{});
            advance(PartATag{});
            advance(PartBTag{});
        } else {
            emitParts(BothPartsTag{});
            advance(BothPartsTag{});
        }
    };
    // vmcnt that certifies the stage the compute side needs next with `younger` whole k-steps' worth of issue behind it
    // (staggered depths: and that stage's own weight share, which went out after its activation share)
    auto waitStage = [&](auto tag) __attribute__((always_inline)) {
        constexpr int kYounger = decltype(tag)::value;
        WaitVmcnt<kYounger * Cfg::kMaxPerWave + (kStaggered ? Cfg::kSlotsB : 0)>();
    };

    // Shifted barrier (tall tiles).  The plain k-step opens with its barrier -- the stage has landed, the previous one is
    // no longer read -- after which every wave waits for its first fragments before it has any MFMA to issue.  Here the
    // step's one barrier sits in front of its LAST block of MFMAs instead: by then every k-slice of the stage has been
    // read, so the buffers take their refill a quarter of a step earlier, the same barrier certifies the next stage as
    // landed, and the next step's first fragments are read while the matrix pipe still has a block of MFMAs to run.  All
    // buffers of both rings are in use.
    constexpr bool kEarly = kTileM >= 96;
    static_assert(!kStaggered || kEarly, "staggered depths are built on the shifted barrier");
    setupIssue(cur, BothPartsTag{});
    if constexpr (kStaggered) {
        // the order the steady state would have left behind: weight stages 0 .. kStagesB - kStagesA - 1 alone, then
        // (activation stage i, weight stage kStagesB - kStagesA + i) for i = 0 .. kStagesA - 1
#pragma unroll 1
        for (int s = 0; s < kStagesB - kStagesA; ++s) {
            emitParts(PartBTag{});
            advance(PartBTag{});
        }
#pragma unroll 1
        for (int s = 0; s < kStagesA; ++s) issueStage();
    } else {
#pragma unroll 1
        for (int s = 0; s < (kEarly ? kStagesB : kStagesB - 1); ++s) issueStage();
    }
    int ringA = 0, ringB = 0;  // buffers the compute side reads next (one index where the depths are the same)
    if constexpr (kEarly) {
        waitStage(std::integral_constant<int, kStagesA - 1>{});
        __syncthreads();  // stage 0 has landed for every wave
    }

    if (kEpi != Epilogue::kInt32 && a.rowScale != nullptr && tid < kTileM) {
        ldsRowScale[tid] = a.rowScale[cur.rowBase + (tid < cur.rows ? tid : cur.rows - 1)];
    }

    // The tile's real rows (rounded up to whole 32-row MFMA tiles) are split between the two wave rows tile by tile:
    // wave row 0 takes the first half (rounded up), wave row 1 the rest, and MFMA tiles that hold no real row are never
    // computed -- on the memory-bound shapes the matrix pipe's power is what is worth saving.  The k loop is
    // instantiated once per MFMA-tile count (0..kSub0) so that its body stays straight-line code.
    int waveRow0 = 0;  // first tile row of this wave
    int mySub = 0;     // MFMA tiles of this wave in the current tile
    // Row of the weight tile where the wave's column block ni begins.  Blocks come in pairs (2p, 2p + 1) that sit at
    // column position kNi / 2 * waveN + p of the tile: plain epilogues, the two halves of 64 neighbouring channels;
    // kSwiglu, 32 activated channels (rows 0..127 of the tile) and their 32 linear partners (rows 128..255).
    auto bRow = [&](int ni) __attribute__((always_inline)) {
        const int position = kNi / 2 * waveN + ni / 2;
        return kSwiglu ? 32 * position + (ni & 1) * (kTileN / 2) : 64 * position + 32 * (ni & 1);
    };
    v16i acc[kSubM][kNi];

    while (true) {
        const TileInfo following = tileAt(curNo + 1);
        // the next tile's per-row scale travels in a register until this tile's epilogue has read the LDS copy
        float followingRowScale = 0.0f;
        if (following.valid && kEpi != Epilogue::kInt32 && a.rowScale != nullptr && tid < kTileM) {
            followingRowScale = a.rowScale[following.rowBase + (tid < following.rows ? tid : following.rows - 1)];
        }
#pragma unroll
        for (int mi = 0; mi < kSubM; ++mi)
#pragma unroll
            for (int ni = 0; ni < kNi; ++ni)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[mi][ni][v] = 0;

        // The k loop of a wave with kMy MFMA tiles.  A k-step is straight-line code: the operands of k-slice ks + 1 are
        // read from LDS before the MFMAs of k-slice ks are issued (fragment double buffer af / bf).
        // Plain form: one barrier at the start of a step (the stage has landed, the previous one is no longer read),
        // and the refill of the buffer it frees goes out behind the first block of MFMAs.
        // kEarly form: see above; the fragments of a step's first k-slice are read at the end of the step before.
        auto runTile = [&](auto myTag) __attribute__((always_inline)) {
            constexpr int kMy = decltype(myTag)::value;
            constexpr int kSlices = kStep / 32;
            static_assert(kSlices % 2 == 0, "the fragment double buffer is handed over between steps at slot 0");
            v4i bf[2][kNi];
            v4i af[2][kMy > 0 ? kMy : 1];
            auto loadSlice = [&](int stageA, int stageB, int ks, int buf) __attribute__((always_inline)) {
                if (kMy == 0) return;
                const char* const A = lds + (kStaggered ? stageA : stageB) * kStrideA;  // common depth: one ring index
                const char* const B = lds + kFirstB + stageB * kStrideB;
                const int chunk = 2 * ks + lhi;
                if constexpr (kNMajor) {
                    // 16-lane group g: channels 16 * (g % 2) .. + 15 of the 32-channel block, k-half g / 2 (= lhi) of the
                    // slice; lane j of the group supplies bytes (k = kBase + j / 2, channels 8 * (j % 2) .. + 7)
                    const int j = lane & 15;
                    const int k = 32 * ks + 16 * lhi + (j >> 1);
                    const uint32_t bBase = ldsBase + kFirstB + stageB * kStrideB + 8 * (j & 1);
#pragma unroll
                    for (int ni = 0; ni < kNi; ++ni) {
                        const int c = (bRow(ni) + 16 * ((lane >> 4) & 1)) >> 4;  // logical 16-byte chunk of the row
                        // k and k + 8 share their low three bits, hence their swizzle
                        const uint32_t lo = bBase + k * 256 + ((c ^ ((k & 7) << 1)) << 4);
                        const uint32_t hi = lo + 8 * 256;
                        const v2i vlo = __builtin_amdgcn_ds_read_tr8_b64_v2i32(reinterpret_cast<LdsV2iPtr>(lo));
                        const v2i vhi = __builtin_amdgcn_ds_read_tr8_b64_v2i32(reinterpret_cast<LdsV2iPtr>(hi));
                        bf[buf][ni] = v4i{vlo[0], vlo[1], vhi[0], vhi[1]};
                    }
                } else if constexpr (kNz) {
                    // 16-lane group g: channels 16 * (g % 2) .. + 15 of the block, k-half g / 2 (= lhi) of the slice;
                    // lane j of the group supplies bytes (k = kBase + j / 2, channels 8 * (j % 2) .. + 7)
                    const int j = lane & 15;
                    const int inBlock = (32 * ks + 16 * lhi + (j >> 1)) * 32 + 16 * ((lane >> 4) & 1) + 8 * (j & 1);
#pragma unroll
                    for (int ni = 0; ni < kNi; ++ni) {
                        // addressed through the 32-bit LDS address: no generic-to-LDS pointer conversion in the loop
                        const uint32_t blk = ldsBase + kFirstB + stageB * kStrideB + (bRow(ni) >> 5) * 4096 + inBlock;
                        const v2i lo = __builtin_amdgcn_ds_read_tr8_b64_v2i32(reinterpret_cast<LdsV2iPtr>(blk));
                        const v2i hi = __builtin_amdgcn_ds_read_tr8_b64_v2i32(reinterpret_cast<LdsV2iPtr>(blk + 8 * 32));
                        bf[buf][ni] = v4i{lo[0], lo[1], hi[0], hi[1]};
                    }
                } else {
#pragma unroll
                    for (int ni = 0; ni < kNi; ++ni) {
                        bf[buf][ni] = *reinterpret_cast<const v4i*>(B + LdsOffset<kStep>(bRow(ni) + l32, chunk));
                    }
                }
#pragma unroll
                for (int mi = 0; mi < kMy; ++mi) {
                    af[buf][mi] = *reinterpret_cast<const v4i*>(A + LdsOffset<kStep>(waveRow0 + mi * 32 + l32, chunk));
                }
            };
            if constexpr (kEarly) loadSlice(ringA, ringB, 0, 0);  // the tile's first stage was certified at the end of the tile before
#pragma unroll 1
            for (int step = 0; step < kSteps; ++step) {
                if constexpr (!kEarly) {
                    // the oldest stage in flight has landed once at most (stages - 2) stages' worth of this wave's DMAs remain
                    waitStage(std::integral_constant<int, kStagesA - 2>{});
                    __syncthreads();  // every wave's share of the stage is in LDS, and the previous stage is no longer read
                    loadSlice(ringA, ringB, 0, 0);
                }
                const int nextA = !kStaggered ? 0 : ringA + 1 == kStagesA ? 0 : ringA + 1;  // unused with a common depth
                const int nextB = ringB + 1 == kStagesB ? 0 : ringB + 1;
#pragma unroll
                for (int ks = 0; ks < kSlices; ++ks) {
                    if (!kEarly || ks + 1 < kSlices) {
                        if (ks + 1 < kSlices) loadSlice(ringA, ringB, ks + 1, (ks + 1) & 1);
                    } else {
                        // Before the step's last block of MFMAs: every k-slice of this stage has been read (the reads
                        // of the last one returned in the shadow of the block before), and the next stage, issued one
                        // step ago, should have landed.  One barrier certifies both; inside a tile, the next step's
                        // first fragments are read behind the MFMAs.
                        __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): this wave's LDS reads have returned
                        waitStage(std::integral_constant<int, kStagesA - 2>{});
                        __syncthreads();
                        issueStage();  // into the buffer(s) that this step read
                        if (step + 1 < kSteps) loadSlice(nextA, nextB, 0, 0);
                    }
#pragma unroll
                    for (int mi = 0; mi < kMy; ++mi) {
#pragma unroll
                        for (int ni = 0; ni < kNi; ++ni) {
                            acc[mi][ni] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[ks & 1][mi], bf[ks & 1][ni], acc[mi][ni], 0, 0, 0);
                        }
                    }
                    if constexpr (kEarly && kMy > 0) {
                        if (ks + 1 < kSlices) {
                            // The k-slice's pipeline, pinned: the reads of the next slice go out behind the first MFMA
                            // and return under the others.  Left alone, the scheduler makes this order on some builds
                            // and, at the register limit of the tallest tiles, on others a late-read order that stalls
                            // the matrix pipe.  (Reading each fragment only when the one before it has retired saves
                            // registers and measures slower.)
                            constexpr int kReads = kMy + ((kNz || kNMajor) ? 2 * kNi : kNi);
                            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);              // one MFMA
                            __builtin_amdgcn_sched_group_barrier(0x100, kReads, 0);         // the LDS reads
                            __builtin_amdgcn_sched_group_barrier(0x008, kNi * kMy - 1, 0);  // the other MFMAs
                        }
                    }
                    if (!kEarly && ks == 0) issueStage();  // into the buffer that the step before read
                }
                ringA = nextA;
                ringB = nextB;
            }
        };
        {
            const int active = (cur.rows + 31) >> 5;                       // MFMA tiles with real rows, 1..kSub0+kSub1
            const int share0 = Cfg::kWavesM == 2 ? (active + 1) >> 1 : active;  // wave row 0's share
            waveRow0 = waveM == 0 ? 0 : 32 * share0;
            mySub = waveM == 0 ? share0 : active - share0;
        }
        ForCount<kSub0>(mySub, runTile);

        // The draw for the tile after the next goes out inside the epilogue and is looked at behind it.  A wave's memory
        // requests are counted back in issue order and the draw, an atomic that is settled at the memory side, takes
        // microseconds on a loaded machine: in front of the k loop it would hold up the count of every operand stage
        // issued after it.  During the epilogue the ring is full and nothing is issued.
        int32_t drawValue = 0;
        auto draw = [&]() __attribute__((always_inline)) {
            if (pull && following.valid && tid == 0) {
                const int c = QueueFirstOpen(static_cast<uint32_t>(ldsSeq[kSeqUsedUp]), xcd, prefer, kOneRun);
                ldsSeq[kSeqDrawCounter] = c;
                if (c >= 0) drawValue = QueueTake(a.queueCounters, c);
            }
        };
        TileEpilogueWave<kSubM, kNi, 0, kTileM, kEpi>(a, cur, acc, mySub, waveRow0, kNi / 2 * waveN, Opaque(l32), Opaque(lhi),
                                                      ldsRowScale, ldsRowMax, draw);
        if constexpr (kNi == 4) {
            TileEpilogueWave<kSubM, kNi, 1, kTileM, kEpi>(a, cur, acc, mySub, waveRow0, kNi / 2 * waveN + 1, Opaque(l32), Opaque(lhi),
                                                          ldsRowScale, ldsRowMax);
        }
        if constexpr (kSwiglu) TileEpilogueFoldMax<kTileM>(a, cur, Opaque(tid), ldsRowMax);
        // Loads and stores may retire out of order with respect to each other, so drain everything (the epilogue's
        // stores and the DMAs in flight, which had the whole epilogue to land) before counting DMAs again.
        WaitVmcnt<0>();
        ++spanTiles;
        if (!following.valid) break;
        if (pull && tid == 0) {
            const QueueDraw d = QueueResolve(bigTiles, totalTiles - bigTiles, a.queueCounters, xcd, prefer,
                                             static_cast<uint32_t>(ldsSeq[kSeqUsedUp]), ldsSeq[kSeqDrawCounter], drawValue, kOneRun);
            ldsSeq[2 * ((curNo + 2) & 3)] = d.list;
            ldsSeq[2 * ((curNo + 2) & 3) + 1] = d.logical;
            ldsSeq[kSeqUsedUp] = static_cast<int32_t>(d.usedUp);
        }
        __syncthreads();  // the epilogue's reads of ldsRowScale / ldsRowMax are done; the drawn tile is in the ring
        if (kEpi != Epilogue::kInt32 && a.rowScale != nullptr && tid < kTileM) ldsRowScale[tid] = followingRowScale;
        cur = following;
        ++curNo;
    }
}

// Workgroup span record (include/opapi_profile.h): start, end, tiles computed.
__device__ __forceinline__ void WriteSpan(const KernelArgs& a, uint64_t start, uint64_t tiles) {
    if (a.wgSpans != nullptr && threadIdx.x == 0) {
        a.wgSpans[3 * blockIdx.x] = start;
        a.wgSpans[3 * blockIdx.x + 1] = __builtin_amdgcn_s_memrealtime();
        a.wgSpans[3 * blockIdx.x + 2] = tiles;
    }
}

template <int kSub0, int kSub1, int kStep, Epilogue kEpi, bool kNz, bool kNMajor = false, int kWn = kWavesN>
__global__ __launch_bounds__(64 * kWn * (kSub1 > 0 ? 2 : 1)) void StreamGemmKernel(
    KernelArgs a, const int32_t* __restrict__ sched) {
    extern __shared__ __attribute__((aligned(16))) char lds[];
    const uint64_t spanStart = a.wgSpans != nullptr ? __builtin_amdgcn_s_memrealtime() : 0;
    uint64_t spanTiles = 0;
    StreamGemmBody<kSub0, kSub1, kStep, kEpi, kNz, kNMajor, kWn, kBothRuns>(a, sched, lds, spanTiles);
    WriteSpan(a, spanStart, spanTiles);
}

// Tall tiles (192 and 256 rows) with pulled tiles: the two runs of the m-tile table, each with a stage geometry of its
// own.  A big m-tile of 256 rows needs 256 activation rows per stage and leaves LDS room for two stages; a small one (at
// most 64 rows: the whole K x 256 weight block for a handful of rows) needs 64 and runs as a pure weight stream, for
// which two stages in flight per CU are too few -- with the geometry of the 64-row tiles it has three, the rotated k
// walk and the non-temporal weight loads of the decode shapes.  A workgroup serves the run it prefers (the small run gets the share
// of each XCD's workgroups that its cost is of the whole) until that run's counters are used up on every XCD, lets its
// ring drain, and serves the other; a launch without small m-tiles costs the workgroups that looked for them one draw.
template <int kSub0, int kSub1, Epilogue kEpi, bool kNz, bool kNMajor>
__global__ __launch_bounds__(512) void MixedGemmKernel(KernelArgs a, const int32_t* __restrict__ sched) {
    static_assert(StreamCfg<1, 1, 128>::kTileM == kSmallRows, "the small run's geometry is that of the 64-row tiles");
    static_assert(StreamCfg<1, 1, 128>::kThreads == 512 && StreamCfg<kSub0, kSub1, 128>::kThreads == 512, "one workgroup size for both");
    extern __shared__ __attribute__((aligned(16))) char lds[];
    const uint64_t spanStart = a.wgSpans != nullptr ? __builtin_amdgcn_s_memrealtime() : 0;
    uint64_t spanTiles = 0;
    const int64_t costSmall = sched[2], costAll = costSmall + sched[3];
    const int32_t slots = gridDim.x / kXcds, slot = blockIdx.x / kXcds;
    int64_t forSmall = costAll > 0 ? (slots * costSmall + costAll / 2) / costAll : 0;
    if (forSmall == 0 && sched[1] > 0 && slots > 1) forSmall = 1;
    if (slot < forSmall) {
        StreamGemmBody<1, 1, 128, kEpi, kNz, kNMajor, kWavesN, kSmallRun>(a, sched, lds, spanTiles);
        __syncthreads();  // the other geometry lays LDS out anew
        StreamGemmBody<kSub0, kSub1, 128, kEpi, kNz, kNMajor, kWavesN, kBigRun>(a, sched, lds, spanTiles);
    } else {
        StreamGemmBody<kSub0, kSub1, 128, kEpi, kNz, kNMajor, kWavesN, kBigRun>(a, sched, lds, spanTiles);
        __syncthreads();
        StreamGemmBody<1, 1, 128, kEpi, kNz, kNMajor, kWavesN, kSmallRun>(a, sched, lds, spanTiles);
    }
    WriteSpan(a, spanStart, spanTiles);
}

// ---------------------------------------------------------------------------------------------- generic path
constexpr int kGenStep = 128;  // k-bytes per step

__device__ __forceinline__ int Lds128Offset(int row, int chunk) { return row * kGenStep + ((chunk ^ ((row >> 1) & 7)) << 4); }

// One tile per workgroup (grid = static upper bound of tiles), 4 waves, operands gathered byte by byte through
// registers into a single LDS buffer.  Handles any K and both weight layouts.
template <int kSubM, Epilogue kEpi>
__global__ __launch_bounds__(256) void GenericGemmKernel(KernelArgs a, const int32_t* __restrict__ sched) {
    constexpr int kThreads = 256;
    constexpr int kTileM = 32 * kSubM;
    constexpr int kChunksPerRow = kGenStep / kChunk;
    constexpr int kALoads = kTileM * kChunksPerRow / kThreads;
    constexpr int kBLoads = kTileN * kChunksPerRow / kThreads;
    constexpr bool kSwiglu = kEpi == Epilogue::kSwiglu;
    __shared__ __attribute__((aligned(16))) char ldsA[kTileM * kGenStep];
    __shared__ __attribute__((aligned(16))) char ldsB[kTileN * kGenStep];
    __shared__ __attribute__((aligned(16))) float ldsRowScale[kTileM];
    __shared__ float ldsRowMax[kWavesN * kTileM];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int waveN = tid >> 6;
    const int l32 = lane & 31;
    const int lhi = lane >> 5;

    // one tile per workgroup: the two runs of the m-tile table as one list, cut into eight contiguous shares
    const int32_t* const queueHdr = sched;
    const int4* const mTileTable = reinterpret_cast<const int4*>(queueHdr + kQueueHeaderInts + kQueueCounterInts);
    const int32_t countBig = queueHdr[0], countSmall = queueHdr[1];
    const int64_t bigTiles = static_cast<int64_t>(countBig) * a.tilesN;
    const int64_t totalTiles = bigTiles + static_cast<int64_t>(countSmall) * a.tilesN;
    const int64_t perXcd = (totalTiles + kXcds - 1) / kXcds;
    const int64_t local = blockIdx.x / kXcds;
    const int64_t logical = static_cast<int64_t>(blockIdx.x % kXcds) * perXcd + local;
    if (local >= perXcd || logical >= totalTiles) return;
    const TileInfo t = logical < bigTiles
        ? DecodeListTile<kTileM, kSwiglu>(a, mTileTable, 0, countBig, queueHdr[4], logical)
        : DecodeListTile<kTileM, kSwiglu>(a, mTileTable, countBig, countSmall, queueHdr[5], logical - bigTiles);
    if (kEpi != Epilogue::kInt32 && a.rowScale != nullptr && tid < kTileM) {
        ldsRowScale[tid] = a.rowScale[t.rowBase + (tid < t.rows ? tid : t.rows - 1)];
    }
    const int8_t* const wGroup = a.w + static_cast<int64_t>(t.group) * a.wGroupStride;
    const int bRow0 = kSwiglu ? 32 * waveN : 64 * waveN;
    const int bRowStep = kSwiglu ? kTileN / 2 : 32;

    v16i acc[kSubM][2];
#pragma unroll
    for (int mi = 0; mi < kSubM; ++mi)
#pragma unroll
        for (int ni = 0; ni < 2; ++ni)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[mi][ni][v] = 0;

    for (int k0 = 0; k0 < a.K; k0 += kGenStep) {
        // consecutive threads take consecutive tile rows so that N-contiguous weights still coalesce
#pragma unroll
        for (int i = 0; i < kALoads; ++i) {
            const int p = i * kThreads + tid;
            const int r = p % kTileM;
            const int chunk = p / kTileM;
            const int8_t* src = a.x + static_cast<int64_t>(t.rowBase + (r < t.rows ? r : t.rows - 1)) * a.K;
            union { v4i v; int8_t b[16]; } u;
            for (int j = 0; j < kChunk; ++j) {
                const int k = k0 + chunk * kChunk + j;
                u.b[j] = k < a.K ? src[k] : static_cast<int8_t>(0);
            }
            *reinterpret_cast<v4i*>(ldsA + Lds128Offset(r, chunk)) = u.v;
        }
#pragma unroll
        for (int i = 0; i < kBLoads; ++i) {
            const int p = i * kThreads + tid;
            const int r = p % kTileN;
            const int chunk = p / kTileN;
            const int8_t* src = wGroup + WeightRowBase(a, ChannelOfRow<kSwiglu>(a, t, r));
            union { v4i v; int8_t b[16]; } u;
            for (int j = 0; j < kChunk; ++j) {
                const int k = k0 + chunk * kChunk + j;
                u.b[j] = k < a.K ? src[static_cast<int64_t>(k) * a.wStrideK] : static_cast<int8_t>(0);
            }
            *reinterpret_cast<v4i*>(ldsB + Lds128Offset(r, chunk)) = u.v;
        }
        __syncthreads();
#pragma unroll
        for (int ks = 0; ks < kGenStep / 32; ++ks) {
            const int chunk = 2 * ks + lhi;
            const v4i b0 = *reinterpret_cast<const v4i*>(ldsB + Lds128Offset(bRow0 + l32, chunk));
            const v4i b1 = *reinterpret_cast<const v4i*>(ldsB + Lds128Offset(bRow0 + bRowStep + l32, chunk));
#pragma unroll
            for (int mi = 0; mi < kSubM; ++mi) {
                const v4i av = *reinterpret_cast<const v4i*>(ldsA + Lds128Offset(mi * 32 + l32, chunk));
                acc[mi][0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av, b0, acc[mi][0], 0, 0, 0);
                acc[mi][1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av, b1, acc[mi][1], 0, 0, 0);
            }
        }
        __syncthreads();
    }
    TileEpilogue<kSubM, kTileM, kEpi>(a, t, acc, kSubM, 0, waveN, l32, lhi, tid, ldsRowScale, ldsRowMax);
}

// ---------------------------------------------------------------------------------------------- launchers
template <int kSub0, int kSub1, int kStep, Epilogue kEpi, bool kNz, bool kNMajor, int kWn = kWavesN>
hipError_t LaunchStream(const KernelArgs& args, const int32_t* sched, int64_t maxTiles, hipStream_t stream) {
    using Cfg = StreamCfg<kSub0, kSub1, kStep, kWn>;
    auto kernel = StreamGemmKernel<kSub0, kSub1, kStep, kEpi, kNz, kNMajor, kWn>;
    static std::atomic<uint64_t> optedIn{0};
    const hipError_t attr = opapi::EnsureDynamicLds(reinterpret_cast<const void*>(kernel), Cfg::kLdsBytes, optedIn);
    if (attr != hipSuccess) return attr;
    // persistent grid: one workgroup per CU (the LDS ring fills the CU), a multiple of the XCD count
    int64_t grid = DeviceCuCount();
    if (grid > maxTiles) grid = maxTiles;
    grid = grid / kXcds * kXcds;
    if (grid < kXcds) grid = kXcds;
    KernelArgs launchArgs = args;
    launchArgs.wgSpans = SpanBufferFor(kEpi, static_cast<int>(grid), Cfg::kTileM);
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(grid)), dim3(Cfg::kThreads), Cfg::kLdsBytes, stream, launchArgs, sched);
    return hipGetLastError();
}

template <int kSub0, int kSub1, Epilogue kEpi, bool kNz, bool kNMajor>
hipError_t LaunchMixed(const KernelArgs& args, const int32_t* sched, int64_t maxTiles, hipStream_t stream) {
    using Big = StreamCfg<kSub0, kSub1, 128>;
    using Small = StreamCfg<1, 1, 128>;
    constexpr int kLdsBytes = Big::kLdsBytes > Small::kLdsBytes ? Big::kLdsBytes : Small::kLdsBytes;
    auto kernel = MixedGemmKernel<kSub0, kSub1, kEpi, kNz, kNMajor>;
    static std::atomic<uint64_t> optedIn{0};
    const hipError_t attr = opapi::EnsureDynamicLds(reinterpret_cast<const void*>(kernel), kLdsBytes, optedIn);
    if (attr != hipSuccess) return attr;
    int64_t grid = DeviceCuCount();
    if (grid > maxTiles) grid = maxTiles;
    grid = grid / kXcds * kXcds;
    if (grid < kXcds) grid = kXcds;
    KernelArgs launchArgs = args;
    launchArgs.wgSpans = SpanBufferFor(kEpi, static_cast<int>(grid), Big::kTileM);
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(grid)), dim3(512), kLdsBytes, stream, launchArgs, sched);
    return hipGetLastError();
}

// Tile heights and their (wave row 0, wave row 1, k-step) shapes.  Up to 192 rows the weight ring holds three or more
// 128-byte stages; from 192 rows on the activation ring holds two.
template <Epilogue kEpi, bool kNz, bool kNMajor>
hipError_t LaunchStreamShapeOf(const Plan& plan, const KernelArgs& args, const int32_t* sched, hipStream_t stream) {
    switch (plan.tileM) {
        case 32: return LaunchStream<1, 0, 128, kEpi, kNz, kNMajor>(args, sched, plan.maxTiles, stream);
        case 64: return LaunchStream<1, 1, 128, kEpi, kNz, kNMajor>(args, sched, plan.maxTiles, stream);
        case 96: return LaunchStream<2, 1, 128, kEpi, kNz, kNMajor>(args, sched, plan.maxTiles, stream);
        case 128: return LaunchStream<2, 2, 128, kEpi, kNz, kNMajor>(args, sched, plan.maxTiles, stream);
        // (160-row tiles were measured in the two-geometry form as well: the down projection of the DeepSeek-V3 prefill
        // shape, whose few overflowing experts leave small second m-tiles, 0.834 against 0.820 ms -- sixteen k-steps
        // per tile do not repay a change of geometry)
        case 160: return LaunchStream<3, 2, 128, kEpi, kNz, kNMajor>(args, sched, plan.maxTiles, stream);
        // pulled tiles of 192 and 256 rows: the two runs of the table with a stage geometry each
        case 192:
            if (plan.pullTiles) return LaunchMixed<3, 3, kEpi, kNz, kNMajor>(args, sched, plan.maxTiles, stream);
            return LaunchStream<3, 3, 128, kEpi, kNz, kNMajor>(args, sched, plan.maxTiles, stream);
        default:
            if (plan.pullTiles) return LaunchMixed<4, 4, kEpi, kNz, kNMajor>(args, sched, plan.maxTiles, stream);
            return LaunchStream<4, 4, 128, kEpi, kNz, kNMajor>(args, sched, plan.maxTiles, stream);
    }
}

template <Epilogue kEpi>
hipError_t LaunchStreamShape(const Plan& plan, const KernelArgs& args, const int32_t* sched, hipStream_t stream) {
    if (args.wNz) return LaunchStreamShapeOf<kEpi, true, false>(plan, args, sched, stream);
    if (args.wStrideN == 1) return LaunchStreamShapeOf<kEpi, false, true>(plan, args, sched, stream);  // row-major [K, N]
    return LaunchStreamShapeOf<kEpi, false, false>(plan, args, sched, stream);
}

template <Epilogue kEpi>
hipError_t LaunchGenericShape(const Plan& plan, const KernelArgs& args, const int32_t* sched, hipStream_t stream) {
    const dim3 grid(static_cast<unsigned>(plan.maxTiles));
    if (plan.tileM <= 32) hipLaunchKernelGGL((GenericGemmKernel<1, kEpi>), grid, dim3(256), 0, stream, args, sched);
    else hipLaunchKernelGGL((GenericGemmKernel<4, kEpi>), grid, dim3(256), 0, stream, args, sched);
    return hipGetLastError();
}

}  // namespace
}  // namespace gemm

#pragma clang diagnostic pop
