// Expert-grouped int8 x int8 -> int32 GEMM for gfx950 (CDNA4) with fused epilogues.
//
// Computes, for every group e and every row r of that group, acc[r, c] = sum_k x[r, k] * w[e, k, c] on
// v_mfma_i32_32x32x32_i8 and applies one of three epilogues in registers:
//   kInt32   raw accumulators                                   (aclnnGroupedMatmulV4, int32 output)
//   kDequant (float(acc) * scale[e, c]) * rowScale[r] -> bf16 / fp16 / fp32
//            (reference order: gmm/grouped_matmul/op_kernel/grouped_matmul_quant_mixcore.h:248-291,293-310)
//   kSwiglu  C = (float(acc) * rowScale[r]) * scale[e, c];  S = swish(C[:, j]) * C[:, j + N/2]
//            (reference order: gmm/grouped_matmul_swiglu_quant/op_kernel/grouped_matmul_swiglu_quant.h:368-399,446-474),
//            S is written as fp32 together with one partial max |S| per (n-tile, row); a second, bandwidth-trivial
//            kernel folds the partials and turns S into int8 with the row scale max/127 (same file :477-513).
//
// Scheduling.  Group sizes live in device memory, so a one-workgroup kernel (here) turns groupList into one table entry
// per m-tile -- big m-tiles first, then those of at most 64 rows -- plus tile counters.  Each run of the table is cut
// into eight contiguous shares, one per XCD, so that the workgroups of an XCD sit on neighbouring tiles (shared
// activation rows and weight columns stay in that XCD's L2); workgroups pull their tiles from the counters, or walk
// fixed shares where tiles are too short to hide a draw.
//
// This file: the scheduling kernel, the requantisation kernel, planning and the launch sequence.  The GEMM kernels
// themselves are in grouped_gemm_i8_kernels.h and are instantiated by one translation unit per epilogue:
//   StreamGemmKernel  the fast path (K a multiple of 128; K-contiguous, blocked or row-major [K, N] weights).  Persistent
//                     workgroups; operands go global -> LDS with global_load_lds_dwordx4 into a ring of 2..4 stages of
//                     128 k-bytes (192-row tiles: two activation and three weight stages), so several stages of weights
//                     are in flight per CU with no staging registers, and the ring already holds the next tile's first
//                     steps while the current tile's epilogue runs.
//   MixedGemmKernel   the same body twice, once per run of the table with a stage geometry of its own (pulled tiles of
//                     192 and 256 rows).
//   GenericGemmKernel byte-wise loader for K not a multiple of 128 and channel counts off the 16-byte grid: correct, slow.
// LDS rows are XOR-swizzled in 16-byte chunks so that the 16 lanes the LDS serves per clock (64 banks) never collide,
// for the DMA writes as well as for the MFMA operand reads.
#include "grouped_gemm_i8.h"

#include <mutex>
#include <vector>

#include "grouped_gemm_i8_kernels.h"

namespace gemm {
namespace {

// ---------------------------------------------------------------------------------------------- scheduling kernel
struct SchedArgs {
    const void* groupList;
    int32_t* sched;
    int32_t groups;
    int32_t groupListIsInt64;
    int32_t isCount;  // 0 cumsum, 1 counts, 2 sparse (expert id, count) pairs
    int32_t tileM;
    int32_t maxMTiles;
    int64_t M;
    int64_t rowBegin, rowEnd;  // only rows in [rowBegin, rowEnd) get tiles (one band of a launch that runs in row bands)
};

__global__ __launch_bounds__(1024) void ScheduleKernel(SchedArgs a) {
    __shared__ int32_t scan[1024];
    const int t = threadIdx.x;
    auto at = [&](int i) -> int64_t {
        return a.groupListIsInt64 ? static_cast<const int64_t*>(a.groupList)[i]
                                  : static_cast<int64_t>(static_cast<const int32_t*>(a.groupList)[i]);
    };
    // inclusive prefix sum over the 1024 threads: shuffles inside each wave, then the sixteen wave totals through LDS
    __shared__ int32_t waveTotal[16];
    auto inclusiveScan = [&](int32_t v) -> int32_t {
        const int lane = t & 63, wave = t >> 6;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const int32_t below = __shfl_up(v, d, 64);
            if (lane >= d) v += below;
        }
        __syncthreads();  // the totals of an earlier call have been read
        if (lane == 63) waveTotal[wave] = v;
        __syncthreads();
        int32_t base = 0;
        for (int i = 0; i < wave; ++i) base += waveTotal[i];
        return v + base;
    };
    // the same over two 32-bit counts packed into one 64-bit value (neither half may overflow into the other)
    __shared__ uint64_t waveTotal64[16];
    auto inclusiveScan64 = [&](uint64_t v) -> uint64_t {
        const int lane = t & 63, wave = t >> 6;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const uint64_t below = __shfl_up(v, d, 64);
            if (lane >= d) v += below;
        }
        __syncthreads();
        if (lane == 63) waveTotal64[wave] = v;
        __syncthreads();
        uint64_t base = 0;
        for (int i = 0; i < wave; ++i) base += waveTotal64[i];
        return v + base;
    };
    // group boundaries, clamped into [0, M] and made monotonic so that a malformed list cannot push rows out of range
    int64_t begin = 0, end = 0;
    if (a.isCount == 2) {
        // Sparse list [groups, 2]: pair p = (expert id, rows); pairs take consecutive row ranges in list order and the
        // list ends at the first pair without rows.  The table stays indexed by expert: an expert named by a pair gets
        // that pair's row range, every other expert none (an expert named twice keeps the later range only).
        __shared__ int32_t firstEmpty;
        __shared__ int32_t expertBegin[kMaxGroups], expertEnd[kMaxGroups];
        if (t == 0) firstEmpty = a.groups;
        expertBegin[t] = 0;
        expertEnd[t] = 0;
        __syncthreads();
        int64_t key = -1, val = 0;
        if (t < a.groups) {
            key = at(2 * t);
            val = at(2 * t + 1);
            if (val <= 0) atomicMin(&firstEmpty, t);
        }
        __syncthreads();
        if (t >= firstEmpty) val = 0;
        val = val > a.M ? a.M : val;
        const int32_t inc = inclusiveScan(static_cast<int32_t>(val));
        int64_t pairEnd = inc, pairBegin = inc - val;
        pairBegin = pairBegin > a.M ? a.M : pairBegin;
        pairEnd = pairEnd > a.M ? a.M : pairEnd;
        if (val > 0 && key >= 0 && key < a.groups) {
            expertBegin[key] = static_cast<int32_t>(pairBegin);
            expertEnd[key] = static_cast<int32_t>(pairEnd);
        }
        __syncthreads();
        begin = expertBegin[t];
        end = expertEnd[t];
    } else if (t < a.groups) {
        if (a.isCount) {
            int64_t c = at(t);
            c = c < 0 ? 0 : (c > a.M ? a.M : c);
            end = c;  // turned into a cumsum below
        } else {
            end = at(t);
            begin = t > 0 ? at(t - 1) : 0;
        }
    }
    if (a.isCount == 1) {
        const int32_t inc = inclusiveScan(static_cast<int32_t>(end));
        begin = static_cast<int64_t>(inc) - end;
        end = inc;
    }
    begin = begin < 0 ? 0 : (begin > a.M ? a.M : begin);
    end = end < begin ? begin : (end > a.M ? a.M : end);
    // the band of rows this launch covers: a group keeps the part of its rows that lies inside
    begin = begin < a.rowBegin ? a.rowBegin : (begin > a.rowEnd ? a.rowEnd : begin);
    end = end < a.rowBegin ? a.rowBegin : (end > a.rowEnd ? a.rowEnd : end);
    const int32_t rows = t < a.groups ? static_cast<int32_t>(end - begin) : 0;
    const int32_t tiles = (rows + a.tileM - 1) / a.tileM;
    // big and small m-tiles of this group (with tiles of at most kSmallRows rows every m-tile is small; otherwise only
    // a group's last, partly filled m-tile can be) and the cost of the big ones; two packed prefix sums give every
    // group the positions of its m-tiles in the two runs of the table, and the launch the totals
    const bool allSmall = a.tileM <= kSmallRows;
    const int32_t lastRows = tiles > 0 ? rows - (tiles - 1) * a.tileM : 0;
    const int32_t smallCount = allSmall ? tiles : (tiles > 0 && lastRows <= kSmallRows ? 1 : 0);
    const int32_t bigCount = tiles - smallCount;
    int32_t bigCost = 0;
    if (bigCount > 0) {
        const bool lastIsBig = smallCount == 0;
        const int32_t lastSub = (lastRows + 31) >> 5;
        bigCost = (bigCount - (lastIsBig ? 1 : 0)) * max(a.tileM >> 5, kSmallCost) + (lastIsBig ? max(lastSub, kSmallCost) : 0);
    }
    const uint64_t countsInc = inclusiveScan64(static_cast<uint64_t>(tiles) | (static_cast<uint64_t>(bigCount) << 32));
    const uint64_t costInc = inclusiveScan64(static_cast<uint64_t>(bigCost) | (static_cast<uint64_t>(tiles > 0 ? 1 : 0) << 32));
    const int32_t tileInc = static_cast<int32_t>(countsInc & 0xffffffffu), bigInc = static_cast<int32_t>(countsInc >> 32);
    // rows covered by the list: the end of the last group, or with a sparse list the furthest end of any expert
    int32_t covered = static_cast<int32_t>(end);
    if (a.isCount == 2) {
        scan[t] = t < a.groups ? static_cast<int32_t>(end) : 0;
        __syncthreads();
        for (int d = 512; d > 0; d >>= 1) {
            if (t < d) scan[t] = max(scan[t], scan[t + d]);
            __syncthreads();
        }
        covered = scan[0];
        __syncthreads();
    }
    __shared__ int32_t sRowStart[kMaxGroups], sRows[kMaxGroups], sBigBefore[kMaxGroups], sSmallBefore[kMaxGroups];
    __shared__ int32_t totals[4];
    sRowStart[t] = static_cast<int32_t>(begin);
    sRows[t] = rows;
    sBigBefore[t] = bigInc - bigCount;
    sSmallBefore[t] = (tileInc - bigInc) - smallCount;
    __shared__ int32_t sCovered;
    if (t == a.groups - 1) sCovered = covered;
    if (t == 1023) {
        totals[0] = bigInc;
        totals[1] = tileInc - bigInc;
        totals[2] = static_cast<int32_t>(costInc & 0xffffffffu);
        totals[3] = static_cast<int32_t>(costInc >> 32);  // groups with rows
    }
    // group of every m-tile: scan[] takes the inclusive m-tile prefix (zero-tile groups repeat their
    // predecessor's value); m-tile m belongs to the first group whose inclusive prefix exceeds m
    scan[t] = t < a.groups ? tileInc : 0x7fffffff;
    __syncthreads();
    const int32_t totalMTiles = scan[a.groups - 1];
    // A well-formed list never needs more than maxMTiles m-tiles (M / tileM + groups).  A malformed one whose groups
    // overlap could: the m-tiles beyond the table are dropped, so no kernel indexes past it.
    const int32_t nBig = min(totals[0], a.maxMTiles);
    const int32_t nSmall = min(totals[1], a.maxMTiles - nBig);
    if (t < kQueueCounterInts) a.sched[kQueueHeaderInts + t] = 0;
    // Band width: with two or more m-tiles per group on average, four neighbouring m-tiles (mostly of one group) walk
    // the n-tiles together and share each weight column block through L2; with one m-tile per group the n-tiles of a
    // group follow each other, so that its activation rows are what stays in L2.  A small m-tile is its group's only
    // one of its kind unless every tile is small.
    const int32_t wideBands = totalMTiles >= 2 * totals[3] ? kGroupM : 1;
    if (t < kQueueHeaderInts) {
        a.sched[t] = t == 0 ? nBig : t == 1 ? nSmall : t == 2 ? nSmall * kSmallCost : t == 3 ? totals[2] : t == 4 ? wideBands
                   : t == 5 ? (allSmall ? wideBands : 1) : t == kHdrCoveredRows ? sCovered : 0;
    }
    int4* const mTileTable = reinterpret_cast<int4*>(a.sched + kQueueHeaderInts + kQueueCounterInts);
    for (int32_t m = t; m < totalMTiles; m += 1024) {
        int lo = -1, hi = a.groups - 1;  // scan[hi] > m always holds, scan[lo] <= m (lo = -1: nothing before)
        while (hi - lo > 1) {
            const int mid = (lo + hi) >> 1;
            if (scan[mid] > m) hi = mid; else lo = mid;
        }
        const int32_t inGroup = m - (hi > 0 ? scan[hi - 1] : 0);
        const int32_t tileRows = min(a.tileM, sRows[hi] - inGroup * a.tileM);
        const bool small = allSmall || tileRows <= kSmallRows;
        const int32_t pos = small ? nBig + sSmallBefore[hi] + (allSmall ? inGroup : 0) : sBigBefore[hi] + inGroup;
        const int32_t limit = small ? nBig + nSmall : nBig;
        if (pos < limit) mTileTable[pos] = make_int4(hi, sRowStart[hi] + inGroup * a.tileM, tileRows, 0);
    }
}

// ---------------------------------------------------------------------------------------------- requantisation
struct RequantArgs {
    const float* s;          // [rows of the band, halfN]: row r of the problem at index r - rowBegin
    const float* rowMax;     // [tilesN][M] partial max |S|
    int32_t tilesN;
    int64_t M;
    const int32_t* sched;
    int8_t* y;               // [M, halfN]
    float* yScale;           // [M]
    int32_t halfN;
    int64_t rowBegin;        // first row of the band; the grid covers the band's rows
};

__device__ __forceinline__ int8_t QuantOne(float s, float inv) {
    const __half h = __ushort_as_half(HalfBitsOfRounded(__fmul_rn(s, inv)));
    return static_cast<int8_t>(__float2int_rn(__half2float(h)));
}

// One workgroup per row; rows at or beyond the last group boundary are left untouched.
// Every thread requests its first two packets of S before the row maximum is known, and every wave folds the partial
// maxima for itself (a handful of L2 hits): the row's two dependent memory round trips overlap and there is no barrier.
__global__ __launch_bounds__(256) void RequantKernel(RequantArgs a) {
    const int64_t row = a.rowBegin + blockIdx.x;
    if (row >= a.sched[kHdrCoveredRows]) return;
    typedef float Float4 __attribute__((ext_vector_type(4)));
    const float* src = a.s + static_cast<int64_t>(blockIdx.x) * a.halfN;
    int8_t* dst = a.y + row * a.halfN;
    const bool packets = (a.halfN & 3) == 0;
    constexpr int kAhead = 2;
    Float4 ahead[kAhead];
    if (packets) {
#pragma unroll
        for (int i = 0; i < kAhead; ++i) {
            const int j = (static_cast<int>(threadIdx.x) + 256 * i) * 4;
            // S is read exactly once: a non-temporal load keeps it from displacing anything in the caches
            ahead[i] = j < a.halfN ? __builtin_nontemporal_load(reinterpret_cast<const Float4*>(src + j)) : Float4{0.0f, 0.0f, 0.0f, 0.0f};
        }
    }
    float mx = 0.0f;
    for (int t = threadIdx.x & 63; t < a.tilesN; t += 64) mx = fmaxf(mx, a.rowMax[static_cast<int64_t>(t) * a.M + row]);
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) mx = fmaxf(mx, __shfl_xor(mx, d, 64));
    const float ys = __fdiv_rn(mx, 127.0f);
    const float inv = __fdiv_rn(1.0f, ys);
    if (threadIdx.x == 0) a.yScale[row] = ys;
    const bool zeroRow = mx == 0.0f;  // reference: 0 * inf; defined here as zeros
    if (packets) {
        auto quantPacket = [&](const Float4 v, int j) __attribute__((always_inline)) {
            char4 q;
            q.x = zeroRow ? 0 : QuantOne(v.x, inv);
            q.y = zeroRow ? 0 : QuantOne(v.y, inv);
            q.z = zeroRow ? 0 : QuantOne(v.z, inv);
            q.w = zeroRow ? 0 : QuantOne(v.w, inv);
            *reinterpret_cast<char4*>(dst + j) = q;  // read again soon, by the down projection: stays cacheable
        };
#pragma unroll
        for (int i = 0; i < kAhead; ++i) {
            const int j = (static_cast<int>(threadIdx.x) + 256 * i) * 4;
            if (j < a.halfN) quantPacket(ahead[i], j);
        }
        // rows longer than 2048 columns: one packet per trip (batching four loads per trip measured 5 % slower on
        // 14336-column rows)
        for (int j = (static_cast<int>(threadIdx.x) + 256 * kAhead) * 4; j < a.halfN; j += 256 * 4) {
            quantPacket(__builtin_nontemporal_load(reinterpret_cast<const Float4*>(src + j)), j);
        }
    } else {
        for (int j = threadIdx.x; j < a.halfN; j += 256) dst[j] = zeroRow ? 0 : QuantOne(src[j], inv);
    }
}

}  // namespace

// ---------------------------------------------------------------------------------------------- dispatch
int DeviceCuCount() {
    static const int count = [] {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess) return 256;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) return 256;
        return n;
    }();
    return count;
}

namespace {
// ---- workgroup spans (opapiGemmWorkgroupSpans*, include/opapi_profile.h): a measurement aid, off by default ----
// The buffers are allocated by opapiGemmWorkgroupSpansEnable(1) on the device that is current then, never on a launch
// path; recording is for one device and one launching thread at a time (the mutex only keeps the bookkeeping whole).
constexpr int kSpanKinds = 3;        // indexed by Epilogue
constexpr int kSpanMaxGrid = 1024;
std::mutex gSpanMutex;
bool gSpansOn = false;
int gSpanDevice = -1;
uint64_t* gSpanBuf[kSpanKinds] = {nullptr, nullptr, nullptr};
int gSpanGrid[kSpanKinds] = {0, 0, 0};   // workgroups of the last recorded launch of the kind; 0: nothing recorded
int gSpanTileM[kSpanKinds] = {0, 0, 0};
}  // namespace

// Device buffer for the next ring-kernel launch of this epilogue kind (every workgroup of the launch writes its own
// entry), or null when recording is off, the launch runs on another device or its grid exceeds the buffer -- the kind's
// earlier record is dropped then, so that a report never shows another launch's figures as the last one's.
uint64_t* SpanBufferFor(Epilogue epi, int grid, int tileM) {
    std::lock_guard<std::mutex> lock(gSpanMutex);
    if (!gSpansOn) return nullptr;
    const int k = static_cast<int>(epi);
    int dev = -1;
    if (gSpanBuf[k] == nullptr || grid > kSpanMaxGrid || hipGetDevice(&dev) != hipSuccess || dev != gSpanDevice) {
        gSpanGrid[k] = 0;
        return nullptr;
    }
    gSpanGrid[k] = grid;
    gSpanTileM[k] = tileM;
    return gSpanBuf[k];
}

namespace {
// The DMA ring needs whole 128-byte k steps, 16-byte aligned bases, 32-bit offsets inside one expert's weights and one of
// the three weight layouts it knows: K-contiguous rows per channel, the blocked layout, or row-major [K, N].
bool StreamOk(const Problem& p) {
    // blocked: whole 32-channel blocks; row-major: whole 16-byte chunks (per half of a SwiGLU tile)
    const int64_t grain = p.wNz ? 32 : 16;
    const bool layoutOk = p.wKMajor && !p.wNz ? true
                          : (p.N % grain == 0 && (p.epilogue != Epilogue::kSwiglu || (p.N / 2) % grain == 0));
    // One expert's weights must hold at least the kilobyte (64 lanes x 16 bytes) that a drained workgroup's idle issue
    // slots keep re-reading from the start of its last tile's expert: smaller experts go to the byte-wise kernel.
    return layoutOk && p.K % 128 == 0 && reinterpret_cast<uintptr_t>(p.x) % kChunk == 0 &&
           reinterpret_cast<uintptr_t>(p.w) % kChunk == 0 && p.N * p.K < (1ll << 31) && p.N * p.K >= 64 * kChunk;
}

uint64_t Align256(uint64_t v) { return (v + 255) / 256 * 256; }

}  // namespace

Plan MakePlan(const Problem& p) {
    Plan plan;
    const int64_t groups = p.groups > 0 ? p.groups : 1;
    const int64_t cols = p.epilogue == Epilogue::kSwiglu ? p.N / 2 : p.N;
    const int64_t colsPerTile = p.epilogue == Epilogue::kSwiglu ? kTileN / 2 : kTileN;
    plan.tilesN = static_cast<int32_t>((cols + colsPerTile - 1) / colsPerTile);
    // tile height: the mean group size plus a quarter, so that almost every group is covered by one m-tile and its
    // weights are streamed exactly once.  A group that still overflows its tile adds a second m-tile, i.e. tilesN more
    // tiles, all in one XCD's share: its workgroups walk one round more than the others.  Where a workgroup walks few
    // rounds (one is more than 4 % of the launch) the headroom is half the mean instead: the taller shapes pay for
    // their extra rows with a shallower activation ring, which costs less than that round.
    const double meanRows = p.expectedRowsPerGroup > 0 ? static_cast<double>(p.expectedRowsPerGroup)
                                                       : static_cast<double>(p.M) / static_cast<double>(groups);
    const double rounds = static_cast<double>(groups) * plan.tilesN / DeviceCuCount();
    const double want = meanRows * (rounds <= 24.0 ? 1.5 : 1.25);
    if (StreamOk(p)) {
        static const int kShapes[] = {32, 64, 96, 128, 160, 192, 256};
        plan.tileM = 256;
        for (int s : kShapes) {
            if (static_cast<double>(s) >= want) { plan.tileM = s; break; }
        }
        // A handful of rows per group (decode): the 64-row shape, whose eight waves keep more of the weight stream in
        // flight than the four of the 32-row shape (measured 0.3 - 0.7 % faster on both GEMMs of a 64-token step).
        if (plan.tileM < 64) plan.tileM = 64;
        // tuning override: OPAPI_GEMM_TILE_M=<one of the shapes above>
        if (const char* env = std::getenv("OPAPI_GEMM_TILE_M")) {
            const int forced = std::atoi(env);
            for (int s : kShapes) {
                if (s == forced) plan.tileM = s;
            }
        }
    } else {
        plan.tileM = want <= 32.0 ? 32 : 128;
    }
    // Workgroups pull their tiles from counters where a tile is long enough to hide the draw: at least eight k-steps
    // (the issue side then never runs more than one tile ahead, which is what the two-tile look-ahead of the draw
    // covers) and more than 64 rows; the handful-of-rows tiles of a decode step keep their fixed shares.
    // OPAPI_GEMM_PULL=0 / 1 switches it off / on for every shape with eight k-steps.
    plan.pullTiles = StreamOk(p) && p.K / 128 >= 8 && plan.tileM > 64 && plan.maxTiles < (1ll << 31);
    if (const char* env = std::getenv("OPAPI_GEMM_PULL")) {
        plan.pullTiles = StreamOk(p) && p.K / 128 >= 8 && plan.maxTiles < (1ll << 31) && std::atoi(env) != 0;
    }
    plan.wavesM = plan.tileM >= 64 && StreamOk(p) ? 2 : 1;
    plan.subTilesM = (plan.tileM / 32 + plan.wavesM - 1) / plan.wavesM;
    const int64_t maxMTiles = p.M / plan.tileM + groups;
    plan.maxMTiles = static_cast<int32_t>(maxMTiles);
    // round up so that every XCD's share [xcd * ceil(total/8), ...) is covered by the launch
    plan.maxTiles = (maxMTiles * plan.tilesN + kXcds - 1) / kXcds * kXcds;
    uint64_t off = 0;
    plan.offSched = off;
    off += Align256(static_cast<uint64_t>(SchedTotalInts(plan.maxMTiles)) * 4);
    if (p.epilogue == Epilogue::kSwiglu) {
        plan.offRowMax = off;
        off += Align256(static_cast<uint64_t>(p.M) * 4 * static_cast<uint64_t>(plan.tilesN));
        // S, the fp32 SwiGLU result that the requantisation reads back, is held for one band of rows at a time: at most
        // 512 MiB of it (OPAPI_SWIGLU_WORKSPACE_MB=<n> sets another limit), in whole m-tiles, at least one.  A launch
        // whose S fits runs as one band; a taller one runs schedule, GEMM and requantisation once per band.  A band of
        // 512 MiB is at least 4096 tiles, sixteen rounds of the machine, whatever the shape: measured against a single
        // band on 1.9 GB of S it costs nothing (halving the limit twice costs 2 % and 7 % of the pass).
        uint64_t capBytes = 512ull << 20;
        if (const char* env = std::getenv("OPAPI_SWIGLU_WORKSPACE_MB")) {
            const long long mb = std::atoll(env);
            if (mb > 0) capBytes = static_cast<uint64_t>(mb) << 20;
        }
        const uint64_t rowBytes = static_cast<uint64_t>(p.N / 2) * 4;
        int64_t bandRows = rowBytes > 0 ? static_cast<int64_t>(capBytes / rowBytes) / plan.tileM * plan.tileM : p.M;
        if (bandRows < plan.tileM) bandRows = plan.tileM;
        plan.bandRows = bandRows < p.M ? bandRows : p.M;
        plan.offS = off;
        off += Align256(static_cast<uint64_t>(plan.bandRows) * rowBytes);
    }
    plan.workspaceBytes = off;
    return plan;
}

hipError_t Enqueue(const Problem& p, const Plan& plan, void* workspace, hipStream_t stream) {
    if (p.M == 0 || p.N == 0 || p.groups == 0) return hipSuccess;
    if (p.groups > kMaxGroups) return hipErrorInvalidValue;
    // K = 0 leaves the other epilogues nothing to do; with kSwiglu it would leave the requantisation an unwritten S
    // (the operator's first phase refuses K = 0, so this is a guard, not a path)
    if (p.K <= 0 && p.epilogue == Epilogue::kSwiglu) return hipErrorInvalidValue;
    char* ws = static_cast<char*>(workspace);
    int32_t* sched = reinterpret_cast<int32_t*>(ws + plan.offSched);
    const bool swiglu = p.epilogue == Epilogue::kSwiglu;
    float* rowMax = swiglu ? reinterpret_cast<float*>(ws + plan.offRowMax) : nullptr;
    float* sBuf = swiglu ? reinterpret_cast<float*>(ws + plan.offS) : nullptr;

    SchedArgs sa{};
    sa.groupList = p.groupList;
    sa.sched = sched;
    sa.groups = p.groups;
    sa.groupListIsInt64 = p.groupListIsInt64 ? 1 : 0;
    sa.isCount = static_cast<int32_t>(p.groupListKind);
    sa.tileM = plan.tileM;
    sa.maxMTiles = plan.maxMTiles;
    sa.M = p.M;

    KernelArgs ka{};
    ka.x = p.x;
    ka.w = p.w;
    ka.wGroupStride = p.K * p.N;
    ka.wStrideN = p.wKMajor ? p.K : 1;
    ka.wStrideK = p.wNz ? 32 : (p.wKMajor ? 1 : p.N);
    ka.wNz = p.wNz ? 1 : 0;
    ka.M = static_cast<int32_t>(p.M);
    ka.K = static_cast<int32_t>(p.K);
    ka.N = static_cast<int32_t>(p.N);
    ka.groups = p.groups;
    ka.tilesN = plan.tilesN;
    ka.halfN = static_cast<int32_t>(p.N / 2);
    ka.out = p.out;
    ka.outDtype = p.outDtype;
    ka.scale = p.scale;
    ka.scaleDtype = p.scaleDtype;
    ka.rowScale = p.rowScale;
    ka.sOut = sBuf;
    ka.rowMax = rowMax;
    ka.combineIndex = p.combineIndex;
    ka.combineIndexIsInt64 = p.combineIndexIsInt64 ? 1 : 0;
    ka.combineRows = static_cast<int32_t>(p.combineRows);
    ka.combineWeight = p.combineWeight;
    ka.bias = p.bias;
    ka.biasDtype = p.biasDtype;
    ka.wgSpans = nullptr;
    ka.queueCounters = sched + kQueueHeaderInts;
    ka.pullTiles = plan.pullTiles ? 1 : 0;

    hipError_t e = hipSuccess;
    // One band covers every row unless S is held for a band of rows at a time (kSwiglu with a capped workspace): then
    // schedule, GEMM and requantisation run once per band, the schedule handing out only the band's rows, and S is
    // addressed as if the band's first row were at sBuf (the kernels index S by the row of the problem).
    const int64_t bandRows = swiglu && plan.bandRows > 0 ? plan.bandRows : p.M;
    for (int64_t rowBegin = 0; rowBegin < p.M; rowBegin += bandRows) {
        const int64_t rowEnd = rowBegin + bandRows < p.M ? rowBegin + bandRows : p.M;
        sa.rowBegin = rowBegin;
        sa.rowEnd = rowEnd;
        {
            opapi::KernelTimer timer("gmm_schedule", stream);
            hipLaunchKernelGGL(ScheduleKernel, dim3(1), dim3(1024), 0, stream, sa);
        }
        if (swiglu) {
            ka.sOut = reinterpret_cast<float*>(reinterpret_cast<uintptr_t>(sBuf) -
                                               static_cast<uintptr_t>(rowBegin) * static_cast<uintptr_t>(p.N / 2) * 4);
        }
        if (p.K > 0) {
            const bool fast = StreamOk(p);
            opapi::KernelTimer timer(p.epilogue == Epilogue::kSwiglu ? "gmm_swiglu"
                                     : p.epilogue != Epilogue::kDequant ? "gmm_int32"
                                     : p.combineIndex != nullptr ? "gmm_combine" : "gmm_dequant", stream);
            switch (p.epilogue) {
                case Epilogue::kInt32:
                    e = fast ? LaunchRingInt32(plan, ka, sched, stream) : LaunchGenericInt32(plan, ka, sched, stream);
                    break;
                case Epilogue::kDequant:
                    e = fast ? LaunchRingDequant(plan, ka, sched, stream) : LaunchGenericDequant(plan, ka, sched, stream);
                    break;
                case Epilogue::kSwiglu:
                    e = fast ? LaunchRingSwiglu(plan, ka, sched, stream) : LaunchGenericSwiglu(plan, ka, sched, stream);
                    break;
            }
            if (e != hipSuccess) return e;
        }
        if (swiglu) {
            RequantArgs ra{sBuf, rowMax, plan.tilesN, p.M, sched, p.quantOut, p.quantScaleOut, static_cast<int32_t>(p.N / 2),
                           rowBegin};
            opapi::KernelTimer timer("gmm_requant", stream);
            hipLaunchKernelGGL(RequantKernel, dim3(static_cast<unsigned>(rowEnd - rowBegin)), dim3(256), 0, stream, ra);
            e = hipGetLastError();
            if (e != hipSuccess) return e;
        }
    }
    return e;
}

}  // namespace gemm

extern "C" __attribute__((visibility("default"))) void opapiGemmWorkgroupSpansEnable(int enable) {
    using namespace gemm;
    std::lock_guard<std::mutex> lock(gSpanMutex);
    gSpansOn = false;
    for (int k = 0; k < kSpanKinds; ++k) gSpanGrid[k] = 0;  // records of an earlier recording period are not reported
    if (!enable) return;
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess) return;
    if (dev != gSpanDevice) {
        // buffers of another device stay allocated until the process ends (a few KB); this device gets its own
        for (int k = 0; k < kSpanKinds; ++k) gSpanBuf[k] = nullptr;
        gSpanDevice = dev;
    }
    for (int k = 0; k < kSpanKinds; ++k) {
        if (gSpanBuf[k] == nullptr && hipMalloc(&gSpanBuf[k], kSpanMaxGrid * 3 * sizeof(uint64_t)) != hipSuccess) {
            gSpanBuf[k] = nullptr;
            return;
        }
    }
    gSpansOn = true;
}

extern "C" __attribute__((visibility("default"))) int opapiGemmWorkgroupSpansReport(char* buf, size_t cap) {
    using namespace gemm;
    if (buf == nullptr || cap == 0) return -1;
    if (hipDeviceSynchronize() != hipSuccess) return -1;
    std::lock_guard<std::mutex> lock(gSpanMutex);
    static const char* const kNames[kSpanKinds] = {"gmm_int32", "gmm_dequant", "gmm_swiglu"};
    size_t used = 0;
    int lines = 0;
    buf[0] = 0;
    std::vector<uint64_t> host(kSpanMaxGrid * 3);
    for (int k = 0; k < kSpanKinds; ++k) {
        const int grid = gSpanGrid[k];
        if (gSpanBuf[k] == nullptr || grid <= 0) continue;
        if (hipMemcpy(host.data(), gSpanBuf[k], static_cast<size_t>(grid) * 3 * sizeof(uint64_t), hipMemcpyDeviceToHost) != hipSuccess) return -1;
        uint64_t first = ~0ull, last = 0;
        for (int b = 0; b < grid; ++b) {
            first = std::min(first, host[3 * b]);
            last = std::max(last, host[3 * b + 1]);
        }
        const double span = static_cast<double>(last - first) / 100.0;  // 100 MHz counter -> microseconds
        int n = snprintf(buf + used, cap - used, "%s workgroups %d tile_rows %d span_us %.1f", kNames[k], grid, gSpanTileM[k], span);
        if (n < 0 || static_cast<size_t>(n) >= cap - used) break;
        used += static_cast<size_t>(n);
        // per XCD (workgroup b runs on XCD b % 8): when its last workgroup ended, relative to the launch's first start,
        // the mean busy fraction of its workgroups over the whole span, and the fewest / most tiles one of them took
        for (int x = 0; x < kXcds; ++x) {
            uint64_t xLast = 0, tMin = ~0ull, tMax = 0;
            double busy = 0.0;
            int count = 0;
            for (int b = x; b < grid; b += kXcds) {
                xLast = std::max(xLast, host[3 * b + 1]);
                busy += static_cast<double>(host[3 * b + 1] - host[3 * b]);
                tMin = std::min(tMin, host[3 * b + 2]);
                tMax = std::max(tMax, host[3 * b + 2]);
                ++count;
            }
            n = snprintf(buf + used, cap - used, " xcd%d end_us %.1f busy %.3f tiles %llu-%llu", x,
                         static_cast<double>(xLast - first) / 100.0,
                         span > 0 && count > 0 ? busy / 100.0 / count / span : 0.0, (unsigned long long)tMin, (unsigned long long)tMax);
            if (n < 0 || static_cast<size_t>(n) >= cap - used) break;
            used += static_cast<size_t>(n);
        }
        if (used + 2 < cap) {
            buf[used++] = '\n';
            buf[used] = 0;
        }
        ++lines;
    }
    return lines;
}
