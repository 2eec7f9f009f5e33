// aclnnMoeInitRoutingV2 and aclnnMoeInitRoutingV3 for gfx950: top-k expansion, stable sort by expert, inverse map,
// per-expert counts, row gather (V3: expert range filter, int64 counts, gather- or scatter-type index, scale gather).
//
// Reference behaviour restated (not its structure): moe/moe_init_routing_v2/op_kernel/
//   moe_v2_sort_one_core.h:64-113, moe_v2_sort_multi_core.h:498-504   stable ascending key/value sort of expert ids
//   moe_v2_src_to_dst_op.h:92-108                                     expandedRowIdx[order[d]] = d
//   moe_v2_src_to_dst_with_capacity.h:113-194                         drop/pad: e*C + rank or -1, unused rows zero
//   moe_v2_expert_token_out.h:125-280                                 per-expert count / cumsum
//   moe_v2_gather_out.h:87-138                                        expandedX[dst] = x[i / K]
// Validation follows op_host/moe_init_routing_v2_tiling.cpp:129-283.
//
// Design.  Expert ids are small integers, so the merge sort of the reference becomes a stable LSD radix sort whose
// digit covers all of log2(E) bits in one pass (E <= 2048); larger or unknown id ranges take further passes of the
// same kernels.  One pass is three launches:
//   digit_histogram : every wavefront owns a contiguous slice of the flat index range and counts digits into its own
//                     LDS table, 64 keys a step: a ballot per digit bit yields the lanes holding the same digit, the
//                     lowest such lane adds popcount(mask) to the table.  No atomics, no inter-wave traffic.
//   digit_scan      : one workgroup turns the [slice][digit] table into exclusive offsets (down the slices, then across
//                     digits) and, on the last pass, emits count / cumsum.
//   digit_scatter   : same traversal; destination = running offset + popcount(mask & lanes below), which keeps equal
//                     keys in index order (stability).  The last pass writes the inverse map directly.
// The gather reads each source row once with 16-byte lanes and writes its K destinations.
#include "opapi_common.h"

#include <hip/hip_fp16.h>

#include <mutex>

#include "aclnnop/aclnn_moe_init_routing_quant_v2.h"
#include "aclnnop/aclnn_moe_init_routing_v2.h"
#include "aclnnop/aclnn_moe_init_routing_v3.h"

namespace {

constexpr int kWaveSize = 64;
constexpr int kWavesPerBlock = 4;
constexpr int kSortThreads = kWaveSize * kWavesPerBlock;
constexpr int kMaxDigitBits = 11;
constexpr int kMaxBins = 1 << kMaxDigitBits;

struct SortPass {
    const int32_t* keysIn;
    const int32_t* payloadIn;  // nullptr on the first pass: payload is the flat index itself
    int32_t* keysOut;          // nullptr when no later pass or consumer needs the sorted keys
    int32_t* payloadOut;       // nullptr on the last pass
    int32_t* table;            // [numSlices][bins]
    int32_t* binBase;          // [bins] exclusive offsets of each digit value
    int32_t* binTotal;         // [bins]
    int64_t total;             // M
    int32_t sliceLen;          // keys per wavefront slice (multiple of 64)
    int32_t numSlices;
    int32_t shift;
    int32_t bits;
    int32_t flipSign;          // 1: the top bit of the digit is the key's sign bit, invert it so negatives sort first
};

__device__ __forceinline__ uint32_t DigitOf(int32_t key, const SortPass& p) {
    uint32_t d = (static_cast<uint32_t>(key) >> p.shift) & ((1u << p.bits) - 1u);
    if (p.flipSign) d ^= 1u << (p.bits - 1);
    return d;
}

// Orders this wavefront's LDS accesses: writes made by one lane before the call are seen by every lane after it.
// The LDS unit executes a wavefront's operations in order, so only the compiler needs constraining.
__device__ __forceinline__ void WaveSync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Lanes of this wavefront (among `valid` ones) whose digit equals mine.
__device__ __forceinline__ uint64_t MatchDigit(uint32_t digit, int bits, bool valid) {
    uint64_t mask = __ballot(valid);
    for (int b = 0; b < bits; ++b) {
        const bool bit = (digit >> b) & 1u;
        const uint64_t bal = __ballot(bit);
        mask &= bit ? bal : ~bal;
    }
    return mask;
}

__global__ __launch_bounds__(kSortThreads) void DigitHistogramKernel(SortPass p) {
    __shared__ int32_t tbl[kWavesPerBlock][kMaxBins];
    const int lane = threadIdx.x % kWaveSize;
    const int wave = threadIdx.x / kWaveSize;
    const int bins = 1 << p.bits;
    const int64_t slice = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + wave;
    if (slice >= p.numSlices) return;
    for (int b = lane; b < bins; b += kWaveSize) tbl[wave][b] = 0;
    WaveSync();
    const int64_t begin = slice * p.sliceLen;
    for (int off = 0; off < p.sliceLen; off += kWaveSize) {
        const int64_t i = begin + off + lane;
        const bool valid = i < p.total;
        const uint32_t digit = valid ? DigitOf(p.keysIn[i], p) : 0u;
        const uint64_t mask = MatchDigit(digit, p.bits, valid);
        if (valid && lane == __ffsll(static_cast<unsigned long long>(mask)) - 1) tbl[wave][digit] += __popcll(mask);
        WaveSync();
    }
    for (int b = lane; b < bins; b += kWaveSize) p.table[slice * bins + b] = tbl[wave][b];
}

struct CountOutputs {
    int32_t* countOrCumsum;   // [expertNum] or nullptr
    int32_t* beforeCapacity;  // [expertNum] or nullptr
    int32_t flag;             // 1 cumsum, 2 count (applies to countOrCumsum)
    int32_t expertNum;
    int64_t* wide;            // [expertNum] or nullptr: the same counts as int64 (V3), cumsum when wideCumsum
    int32_t wideCumsum;
};

// One workgroup of 1024 threads.  With B bins, 1024 / B threads share each digit value (one thread owns two values when
// B = 2048): the slices are cut into that many segments, every thread totals its segment, the segment totals are
// prefixed through LDS, and a second walk turns the table into exclusive offsets.
__global__ __launch_bounds__(1024) void DigitScanKernel(SortPass p, CountOutputs co) {
    __shared__ int32_t segTotal[2048];  // [segment][bin]
    __shared__ int32_t partial[1024];
    const int bins = 1 << p.bits;
    const int binsPerThread = bins > 1024 ? bins / 1024 : 1;
    const int segs = bins >= 1024 ? 1 : 1024 / bins;
    const int seg = bins >= 1024 ? 0 : threadIdx.x / bins;
    const int bin0 = bins >= 1024 ? threadIdx.x * binsPerThread : threadIdx.x % bins;
    const int slicesPerSeg = (p.numSlices + segs - 1) / segs;
    const int sBegin = seg * slicesPerSeg;
    const int sEnd = min(p.numSlices, sBegin + slicesPerSeg);
    for (int j = 0; j < binsPerThread; ++j) {
        const int b = bin0 + j;
        int32_t run = 0;
#pragma unroll 8
        for (int s = sBegin; s < sEnd; ++s) run += p.table[static_cast<int64_t>(s) * bins + b];
        segTotal[seg * bins + b] = run;
    }
    __syncthreads();
    // per digit value: offset of this thread's segment inside the value, and the value's total
    int32_t segBase[2] = {0, 0}, total[2] = {0, 0};
    for (int j = 0; j < binsPerThread; ++j) {
        const int b = bin0 + j;
        for (int g = 0; g < segs; ++g) {
            const int32_t v = segTotal[g * bins + b];
            if (g < seg) segBase[j] += v;
            total[j] += v;
        }
    }
    // exclusive scan of the totals across digit values (threads of segment 0 carry them, the others contribute 0)
    const int32_t mine = seg == 0 ? total[0] + total[1] : 0;
    partial[threadIdx.x] = mine;
    __syncthreads();
    for (int d = 1; d < 1024; d <<= 1) {
        const int32_t add = threadIdx.x >= d ? partial[threadIdx.x - d] : 0;
        __syncthreads();
        partial[threadIdx.x] += add;
        __syncthreads();
    }
    if (seg == 0) {
        int32_t base = partial[threadIdx.x] - mine;
        for (int j = 0; j < binsPerThread; ++j) {
            const int b = bin0 + j;
            p.binBase[b] = base;
            p.binTotal[b] = total[j];
            if (b < co.expertNum) {
                if (co.countOrCumsum != nullptr) co.countOrCumsum[b] = co.flag == 1 ? base + total[j] : total[j];
                if (co.beforeCapacity != nullptr) co.beforeCapacity[b] = total[j];
                if (co.wide != nullptr) co.wide[b] = co.wideCumsum ? base + total[j] : total[j];
            }
            base += total[j];
        }
    }
    // second walk: table[slice][bin] becomes the number of keys with this digit in earlier slices
    for (int j = 0; j < binsPerThread; ++j) {
        const int b = bin0 + j;
        int32_t run = segBase[j];
#pragma unroll 4
        for (int s = sBegin; s < sEnd; ++s) {
            const int32_t v = p.table[static_cast<int64_t>(s) * bins + b];
            p.table[static_cast<int64_t>(s) * bins + b] = run;
            run += v;
        }
    }
}

struct InverseMap {
    int32_t* expandedRowIdx;  // scatter-type map [source] -> destination; nullptr unless this is the last pass
    int32_t dropPad;          // 1: destination is e*capacity + rank or -1
    int32_t capacity;
    int32_t* gatherIdx;       // gather-type map [destination] -> source, or nullptr
    int32_t dropFrom;         // destinations at or beyond binBase[dropFrom] are dropped (-1 in both maps); < 0: none
    // Rows of exactly four bytes (a column of per-token scales, say) are copied by the sort's last scatter itself --
    // narrowOut[destination] = narrowX[source / topK] for destinations below activeRows -- which saves the gather
    // launch.  nullptr: rows are gathered by a kernel of their own.
    const uint32_t* narrowX;
    uint32_t* narrowOut;
    int32_t topK;
    int64_t activeRows;
};

__global__ __launch_bounds__(kSortThreads) void DigitScatterKernel(SortPass p, InverseMap im) {
    __shared__ int32_t tbl[kWavesPerBlock][kMaxBins];
    const int lane = threadIdx.x % kWaveSize;
    const int wave = threadIdx.x / kWaveSize;
    const int bins = 1 << p.bits;
    const int64_t slice = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + wave;
    if (slice >= p.numSlices) return;
    for (int b = lane; b < bins; b += kWaveSize) tbl[wave][b] = p.table[slice * bins + b] + p.binBase[b];
    WaveSync();
    const int64_t begin = slice * p.sliceLen;
    const uint64_t lanesBelow = (1ull << lane) - 1ull;
    for (int off = 0; off < p.sliceLen; off += kWaveSize) {
        const int64_t i = begin + off + lane;
        const bool valid = i < p.total;
        const int32_t key = valid ? p.keysIn[i] : 0;
        const uint32_t digit = valid ? DigitOf(key, p) : 0u;
        const uint64_t mask = MatchDigit(digit, p.bits, valid);
        int32_t dst = 0;
        if (valid) dst = tbl[wave][digit] + __popcll(mask & lanesBelow);
        WaveSync();
        if (valid && lane == __ffsll(static_cast<unsigned long long>(mask)) - 1) tbl[wave][digit] += __popcll(mask);
        WaveSync();
        if (valid) {
            const int32_t payload = p.payloadIn != nullptr ? p.payloadIn[i] : static_cast<int32_t>(i);
            if (p.keysOut != nullptr) p.keysOut[dst] = key;
            if (p.payloadOut != nullptr) p.payloadOut[dst] = payload;
            const bool dropped = im.dropFrom >= 0 && dst >= p.binBase[im.dropFrom];
            if (im.expandedRowIdx != nullptr) {
                int32_t row = dst;
                if (im.dropPad) {
                    const int32_t rank = dst - p.binBase[digit];
                    row = rank < im.capacity ? static_cast<int32_t>(digit) * im.capacity + rank : -1;
                }
                im.expandedRowIdx[payload] = dropped ? -1 : row;
            }
            if (im.gatherIdx != nullptr) im.gatherIdx[dst] = dropped ? -1 : payload;
            // four-byte rows ride along with the last pass (see InverseMap)
            if (im.narrowX != nullptr && !dropped && dst < im.activeRows) im.narrowOut[dst] = im.narrowX[payload / im.topK];
        }
    }
}

// Small inputs (decode steps): histogram, scan and scatter of a single-pass sort in ONE workgroup, so the sort costs one
// launch instead of three.  Sixteen waves take one slice of the keys each; the per-wave tables and the digit offsets
// stay in LDS.  Writes everything the three kernels above write (binBase / binTotal included: later kernels read them).
constexpr int kSmallSortWaves = 16;
constexpr int kSmallSortBins = 512;
constexpr int64_t kSmallSortMaxKeys = 8192;

// writer: this workgroup writes the sort's outputs (one workgroup of a launch does).  ownToken >= 0: the destinations
// of that token's topK ids are also left in ownDst[0 .. topK) (-1: dropped), for the caller to use after a barrier.
__device__ __forceinline__ void SmallSortBody(const SortPass& p, const CountOutputs& co, const InverseMap& im, bool writer,
                                              int32_t ownToken, int32_t* ownDst) {
    __shared__ int32_t tbl[kSmallSortWaves][kSmallSortBins];
    __shared__ int32_t base[kSmallSortBins];   // exclusive offset of each digit value
    __shared__ int32_t scan[kSmallSortBins];
    const int lane = threadIdx.x % kWaveSize;
    const int wave = threadIdx.x / kWaveSize;
    const int bins = 1 << p.bits;              // <= kSmallSortBins
    const int64_t begin = static_cast<int64_t>(wave) * p.sliceLen;

    for (int b = lane; b < bins; b += kWaveSize) tbl[wave][b] = 0;
    WaveSync();
    for (int off = 0; off < p.sliceLen; off += kWaveSize) {
        const int64_t i = begin + off + lane;
        const bool valid = i < p.total;
        const uint32_t digit = valid ? DigitOf(p.keysIn[i], p) : 0u;
        const uint64_t mask = MatchDigit(digit, p.bits, valid);
        if (valid && lane == __ffsll(static_cast<unsigned long long>(mask)) - 1) tbl[wave][digit] += __popcll(mask);
        WaveSync();
    }
    __syncthreads();

    // thread b < bins: the slices' counts of digit value b become exclusive prefixes, their sum the value's total
    const int b = threadIdx.x;
    int32_t total = 0;
    if (b < bins) {
        for (int w = 0; w < kSmallSortWaves; ++w) {
            const int32_t v = tbl[w][b];
            tbl[w][b] = total;
            total += v;
        }
        scan[b] = total;
    }
    __syncthreads();
    for (int d = 1; d < bins; d <<= 1) {
        const int32_t add = (b < bins && b >= d) ? scan[b - d] : 0;
        __syncthreads();
        if (b < bins) scan[b] += add;
        __syncthreads();
    }
    if (b < bins) {
        const int32_t mine = scan[b] - total;
        base[b] = mine;
        if (writer) {
            p.binBase[b] = mine;
            p.binTotal[b] = total;
        }
        if (writer && b < co.expertNum) {
            if (co.countOrCumsum != nullptr) co.countOrCumsum[b] = co.flag == 1 ? mine + total : total;
            if (co.beforeCapacity != nullptr) co.beforeCapacity[b] = total;
            if (co.wide != nullptr) co.wide[b] = co.wideCumsum ? mine + total : total;
        }
    }
    __syncthreads();

    const uint64_t lanesBelow = (1ull << lane) - 1ull;
    const int32_t dropBase = im.dropFrom >= 0 ? base[im.dropFrom] : 0;
    for (int off = 0; off < p.sliceLen; off += kWaveSize) {
        const int64_t i = begin + off + lane;
        const bool valid = i < p.total;
        const int32_t key = valid ? p.keysIn[i] : 0;
        const uint32_t digit = valid ? DigitOf(key, p) : 0u;
        const uint64_t mask = MatchDigit(digit, p.bits, valid);
        int32_t dst = 0;
        if (valid) dst = base[digit] + tbl[wave][digit] + __popcll(mask & lanesBelow);
        WaveSync();
        if (valid && lane == __ffsll(static_cast<unsigned long long>(mask)) - 1) tbl[wave][digit] += __popcll(mask);
        WaveSync();
        if (valid) {
            const int32_t payload = static_cast<int32_t>(i);
            const bool dropped = im.dropFrom >= 0 && dst >= dropBase;
            int32_t row = dst;
            if (im.dropPad) {
                const int32_t rank = dst - base[digit];
                row = rank < im.capacity ? static_cast<int32_t>(digit) * im.capacity + rank : -1;
            }
            if (ownToken >= 0 && payload / im.topK == ownToken) ownDst[payload % im.topK] = dropped ? -1 : row;
            if (writer) {
                if (im.expandedRowIdx != nullptr) im.expandedRowIdx[payload] = dropped ? -1 : row;
                if (im.gatherIdx != nullptr) im.gatherIdx[dst] = dropped ? -1 : payload;
                if (im.narrowX != nullptr && !dropped && dst < im.activeRows) im.narrowOut[dst] = im.narrowX[payload / im.topK];
            }
        }
    }
}

__global__ __launch_bounds__(kSmallSortWaves * kWaveSize) void SmallSortKernel(SortPass p, CountOutputs co, InverseMap im) {
    SmallSortBody(p, co, im, true, -1, nullptr);
}

// Per-expert cumsum / count from fully sorted keys, for id ranges wider than one digit:
// cumsum[e] = number of sorted keys <= e (upper bound).
__global__ void CountFromSortedKernel(const int32_t* sortedKeys, int64_t total, CountOutputs co) {
    const int e = blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= co.expertNum) return;
    auto upper = [&](int32_t v) {
        int64_t lo = 0, hi = total;
        while (lo < hi) {
            const int64_t mid = (lo + hi) >> 1;
            if (sortedKeys[mid] <= v) lo = mid + 1; else hi = mid;
        }
        return static_cast<int32_t>(lo);
    };
    const int32_t hiCount = upper(e);
    const int32_t loCount = upper(e - 1);
    if (co.countOrCumsum != nullptr) co.countOrCumsum[e] = co.flag == 1 ? hiCount : hiCount - loCount;
    if (co.beforeCapacity != nullptr) co.beforeCapacity[e] = hiCount - loCount;
}

struct GatherArgs {
    const char* x;
    char* expandedX;
    const int32_t* expandedRowIdx;
    int64_t rowBytes;
    int64_t tokens;
    int32_t topK;
    int64_t activeRows;  // destinations at or beyond this row are not written
    const float* scale;    // optional per-token scale, routed with the rows: expandedScale[destination] = scale[token]
    float* expandedScale;
};

constexpr int kGatherThreads = 256;
constexpr int kMaxCachedK = 64;

// One workgroup per token: the source row is read once and written to each of its K destinations.
template <typename Vec>
__global__ __launch_bounds__(kGatherThreads) void GatherRowsKernel(GatherArgs a) {
    __shared__ int32_t dsts[kMaxCachedK];
    const int64_t n = blockIdx.x;
    const int kCached = a.topK < kMaxCachedK ? a.topK : kMaxCachedK;
    if (threadIdx.x < kCached) dsts[threadIdx.x] = a.expandedRowIdx[n * a.topK + threadIdx.x];
    __syncthreads();
    if (a.scale != nullptr) {
        const float s = a.scale[n];
        for (int j = threadIdx.x; j < a.topK; j += kGatherThreads) {
            const int64_t d = j < kMaxCachedK ? dsts[j] : a.expandedRowIdx[n * a.topK + j];
            if (d >= 0 && d < a.activeRows) a.expandedScale[d] = s;
        }
    }
    const int64_t vecs = a.rowBytes / static_cast<int64_t>(sizeof(Vec));
    const Vec* src = reinterpret_cast<const Vec*>(a.x + n * a.rowBytes);
    for (int64_t v = threadIdx.x; v < vecs; v += kGatherThreads) {
        const Vec val = src[v];
        for (int j = 0; j < a.topK; ++j) {
            const int64_t d = j < kMaxCachedK ? dsts[j] : a.expandedRowIdx[n * a.topK + j];
            if (d >= 0 && d < a.activeRows) reinterpret_cast<Vec*>(a.expandedX + d * a.rowBytes)[v] = val;
        }
    }
}

// Decode-sized inputs, rows copied as they are: sort and row gather in ONE launch.  One workgroup per token; every
// workgroup sorts all the ids for itself (a few hundred keys out of L2: as long as the one-workgroup sort takes, and the
// workgroups run side by side), workgroup 0 writes the sort's outputs, and each workgroup copies its token's row to the
// destinations it has just computed.  Saves the launch between the two steps, a tenth of a 64-token routing call.
constexpr int64_t kFusedGatherMaxTokens = 256;  // one workgroup each, all resident at once

__global__ __launch_bounds__(kSmallSortWaves * kWaveSize) void SmallSortGatherKernel(SortPass p, CountOutputs co, InverseMap im,
                                                                                     GatherArgs a) {
    __shared__ int32_t dsts[kMaxCachedK];
    const int32_t n = blockIdx.x;
    SmallSortBody(p, co, im, n == 0, n, dsts);
    __syncthreads();
    constexpr int kThreads = kSmallSortWaves * kWaveSize;
    if (a.scale != nullptr && threadIdx.x < a.topK) {
        const int64_t d = dsts[threadIdx.x];
        if (d >= 0 && d < a.activeRows) a.expandedScale[d] = a.scale[n];
    }
    // 16-byte packets; the threads split into groups of one row's packets, each group serving every groups-th destination
    const int vecs = static_cast<int>(a.rowBytes / 16);
    const int lanesPerRow = vecs < kThreads ? vecs : kThreads;
    const int groups = kThreads / lanesPerRow;
    const int group = threadIdx.x / lanesPerRow;
    if (group >= groups) return;
    const uint4* src = reinterpret_cast<const uint4*>(a.x + static_cast<int64_t>(n) * a.rowBytes);
    for (int v = threadIdx.x % lanesPerRow; v < vecs; v += lanesPerRow) {
        const uint4 val = src[v];
        for (int j = group; j < a.topK; j += groups) {
            const int64_t d = dsts[j];
            if (d >= 0 && d < a.activeRows) reinterpret_cast<uint4*>(a.expandedX + d * a.rowBytes)[v] = val;
        }
    }
}

// Drop/pad mode: capacity rows of an expert beyond its (capped) token count hold zeros.
template <typename Vec>
__global__ __launch_bounds__(kGatherThreads) void ZeroUnusedCapacityKernel(char* expandedX, const int32_t* binTotal,
                                                                           int32_t capacity, int64_t rowBytes) {
    const int64_t row = blockIdx.x;
    const int32_t e = static_cast<int32_t>(row / capacity);
    const int32_t c = static_cast<int32_t>(row % capacity);
    if (c < binTotal[e]) return;
    const int64_t vecs = rowBytes / static_cast<int64_t>(sizeof(Vec));
    Vec zero;
    __builtin_memset(&zero, 0, sizeof(Vec));
    Vec* dst = reinterpret_cast<Vec*>(expandedX + row * rowBytes);
    for (int64_t v = threadIdx.x; v < vecs; v += kGatherThreads) dst[v] = zero;
}

// V3: ids inside [start, end) become 0 .. end-start-1, everything else the sentinel end-start, which sorts last.
__global__ void RemapKeysKernel(const int32_t* ids, int32_t* keys, int64_t total, int32_t start, int32_t end) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const int32_t id = ids[i];
    keys[i] = (id >= start && id < end) ? id - start : end - start;
}

// V3 token-count output (int64) from the int32 per-expert counts of the active range.
// mode 0: cumsum, 1: count, 2: key/value pairs (expert id, count) of the non-empty experts, zero-filled behind them.
struct CountV3Args {
    const int32_t* counts;  // [active]; nullptr: every count is zero
    int64_t* out;
    int32_t active;
    int32_t expertStart;
    int32_t mode;
    int32_t kvPairs;        // pairs the key/value buffer holds
};

__global__ __launch_bounds__(1024) void CountV3Kernel(CountV3Args a) {
    __shared__ int32_t scan[1024];
    const int t = threadIdx.x;
    // each thread owns a contiguous run of experts; exclusive prefix of (count, non-empty) over the runs through LDS
    const int per = (a.active + 1023) / 1024;
    const int first = t * per, last = min(first + per, a.active);
    int64_t sum = 0;
    int32_t nonEmpty = 0;
    for (int e = first; e < last; ++e) {
        const int32_t c = a.counts != nullptr ? a.counts[e] : 0;
        sum += c;
        nonEmpty += c != 0 ? 1 : 0;
    }
    auto exclusive = [&](int32_t v) -> int32_t {
        scan[t] = v;
        __syncthreads();
        for (int d = 1; d < 1024; d <<= 1) {
            const int32_t add = t >= d ? scan[t - d] : 0;
            __syncthreads();
            scan[t] += add;
            __syncthreads();
        }
        const int32_t r = scan[t] - v;
        __syncthreads();
        return r;
    };
    int64_t running = exclusive(static_cast<int32_t>(sum));
    int32_t slot = exclusive(nonEmpty);
    if (a.mode == 2) {
        for (int i = t; i < 2 * a.kvPairs; i += 1024) a.out[i] = 0;
        __syncthreads();
    }
    for (int e = first; e < last; ++e) {
        const int32_t c = a.counts != nullptr ? a.counts[e] : 0;
        running += c;
        if (a.mode == 0) a.out[e] = running;
        else if (a.mode == 1) a.out[e] = c;
        else if (c != 0 && slot < a.kvPairs) {
            a.out[2 * slot] = a.expertStart + e;
            a.out[2 * slot + 1] = c;
            ++slot;
        }
    }
}

// V3 dynamic quantisation (quantMode 1), fused with the row gather.  Per destination row:
//   v = float(x[token, :]) * smooth[expert - start, :] (smooth optional);  s = max|v| / 127;  expandedScale[dst] = s;
//   expandedX[dst, :] = int8(round_half_away(fp16_toward_zero(v / s)))      (true divide)
// as moe/moe_init_routing_v3/op_kernel/moe_v3_gather_dynamic_quant.h:103-141 does.  A row of zeros gives s = 0 and
// zeros (the reference divides 0 by 0 there).  One workgroup per token; without a smooth scale the K copies of a token
// are identical, so the row is quantised once and written K times.  The row is read twice (maximum, then quantise):
// the second read comes from cache.
struct QuantGatherArgs {
    const void* x;
    int8_t* expandedX;
    float* expandedScale;
    const int32_t* expandedRowIdx;  // scatter-type map
    const int32_t* expertIdx;
    const float* smooth;            // [active, cols], [1, cols] or nullptr
    int64_t cols;
    int64_t limit;                  // destinations at or beyond it are not written
    int32_t topK;
    int32_t expertStart;
    int32_t dtype;                  // ACL_FLOAT, ACL_FLOAT16, ACL_BF16
    int32_t smoothPerExpert;        // 1: smooth row = expert - expertStart; 0: one row for every expert
    int32_t smoothRows;             // rows of the smooth scale; a copy whose expert falls outside them is not written
    // static quantisation (MoeInitRoutingQuantV2 quantMode 0): both non-null, one float each; no per-row scale then
    const float* staticScale;
    const float* staticOffset;
};

__device__ __forceinline__ float LoadAsFloat(const void* p, int64_t i, int dtype) {
    if (dtype == ACL_FLOAT) return static_cast<const float*>(p)[i];
    const uint16_t raw = static_cast<const uint16_t*>(p)[i];
    if (dtype == ACL_FLOAT16) return __half2float(__ushort_as_half(raw));
    return __uint_as_float(static_cast<uint32_t>(raw) << 16);
}

// kVec consecutive elements starting at element i (kVec 4: i is a multiple of 4 and the buffer is 16-byte aligned).
template <int kVec>
__device__ __forceinline__ void LoadRowChunk(const void* p, int64_t i, int dtype, float (&v)[kVec]) {
    if constexpr (kVec == 4) {
        if (dtype == ACL_FLOAT) {
            const float4 f = *reinterpret_cast<const float4*>(static_cast<const float*>(p) + i);
            v[0] = f.x; v[1] = f.y; v[2] = f.z; v[3] = f.w;
        } else {
            const uint2 u = *reinterpret_cast<const uint2*>(static_cast<const uint16_t*>(p) + i);
            const uint16_t raw[4] = {static_cast<uint16_t>(u.x), static_cast<uint16_t>(u.x >> 16),
                                     static_cast<uint16_t>(u.y), static_cast<uint16_t>(u.y >> 16)};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                v[e] = dtype == ACL_FLOAT16 ? __half2float(__ushort_as_half(raw[e]))
                                            : __uint_as_float(static_cast<uint32_t>(raw[e]) << 16);
            }
        }
    } else {
        v[0] = LoadAsFloat(p, i, dtype);
    }
}

__device__ __forceinline__ int8_t QuantizeOne(float v, float scale) {
    const float h = __half2float(__float2half_rz(v / scale));
    float r = truncf(h + copysignf(0.5f, h));
    r = fminf(fmaxf(r, -128.f), 127.f);
    return static_cast<int8_t>(static_cast<int>(r));
}

// Static quantisation of MoeInitRoutingQuantV2 (moe/moe_init_routing_quant_v2/op_kernel/moe_v2_gather_quant.h:93-133): the
// value is narrowed to half precision, multiplied by half(scale) and increased by half(offset) in half arithmetic (each
// step rounds to nearest even), then rounded to the nearest integer and saturated to int8.
__device__ __forceinline__ int8_t StaticQuantOne(float v, __half hScale, __half hOffset) {
    const __half u = __hadd(__hmul(__float2half_rn(v), hScale), hOffset);
    const float r = fminf(fmaxf(rintf(__half2float(u)), -128.f), 127.f);
    return static_cast<int8_t>(static_cast<int>(r));
}

template <int kVec>
__global__ __launch_bounds__(kGatherThreads) void QuantGatherRowsKernel(QuantGatherArgs a) {
    __shared__ float waveMax[kGatherThreads / kWaveSize];
    const int64_t n = blockIdx.x;
    const bool isStatic = a.staticScale != nullptr;
    const __half hScale = isStatic ? __float2half_rn(a.staticScale[0]) : __float2half_rn(0.f);
    const __half hOffset = isStatic ? __float2half_rn(a.staticOffset[0]) : __float2half_rn(0.f);
    const bool perCopy = a.smooth != nullptr && a.smoothPerExpert != 0;  // every copy of the token is scaled differently
    const int copies = perCopy ? a.topK : 1;
    for (int j = 0; j < copies; ++j) {
        const int32_t dstOne = a.expandedRowIdx[n * a.topK + j];
        if (perCopy && (dstOne < 0 || dstOne >= a.limit)) continue;  // uniform over the workgroup
        // expert ids are caller data: an id outside the smooth scale's rows must not index it
        const int64_t smoothRow = perCopy ? static_cast<int64_t>(a.expertIdx[n * a.topK + j]) - a.expertStart : 0;
        if (perCopy && (smoothRow < 0 || smoothRow >= a.smoothRows)) continue;
        const float* smooth = a.smooth == nullptr ? nullptr : a.smooth + smoothRow * a.cols;
        float mx = 0.f;
        for (int64_t c = static_cast<int64_t>(threadIdx.x) * kVec; c < a.cols && !isStatic; c += kGatherThreads * kVec) {
            float v[kVec];
            LoadRowChunk<kVec>(a.x, n * a.cols + c, a.dtype, v);
#pragma unroll
            for (int i = 0; i < kVec; ++i) {
                if (smooth != nullptr) v[i] = v[i] * smooth[c + i];
                mx = fmaxf(mx, fabsf(v[i]));
            }
        }
        for (int d = 32; d > 0; d >>= 1) mx = fmaxf(mx, __shfl_xor(mx, d));
        __syncthreads();  // the previous copy's readers of waveMax are done
        if (threadIdx.x % kWaveSize == 0) waveMax[threadIdx.x / kWaveSize] = mx;
        __syncthreads();
        mx = waveMax[0];
        for (int w = 1; w < kGatherThreads / kWaveSize; ++w) mx = fmaxf(mx, waveMax[w]);
        const float scale = mx / 127.0f;

        for (int jj = (perCopy ? j : 0); jj < (perCopy ? j + 1 : a.topK) && !isStatic; ++jj) {
            const int32_t dst = a.expandedRowIdx[n * a.topK + jj];
            if (dst >= 0 && dst < a.limit && threadIdx.x == 0) a.expandedScale[dst] = scale;
        }
        for (int64_t c = static_cast<int64_t>(threadIdx.x) * kVec; c < a.cols; c += kGatherThreads * kVec) {
            int8_t q[kVec];
            float v[kVec];
            LoadRowChunk<kVec>(a.x, n * a.cols + c, a.dtype, v);
#pragma unroll
            for (int i = 0; i < kVec; ++i) {
                if (smooth != nullptr) v[i] = v[i] * smooth[c + i];
                q[i] = isStatic ? StaticQuantOne(v[i], hScale, hOffset)
                                : (mx == 0.f ? static_cast<int8_t>(0) : QuantizeOne(v[i], scale));
            }
            for (int jj = (perCopy ? j : 0); jj < (perCopy ? j + 1 : a.topK); ++jj) {
                const int64_t dst = a.expandedRowIdx[n * a.topK + jj];
                if (dst < 0 || dst >= a.limit) continue;
                int8_t* out = a.expandedX + dst * a.cols + c;
                if constexpr (kVec == 4) {
                    *reinterpret_cast<uint32_t*>(out) = static_cast<uint32_t>(static_cast<uint8_t>(q[0])) |
                                                        (static_cast<uint32_t>(static_cast<uint8_t>(q[1])) << 8) |
                                                        (static_cast<uint32_t>(static_cast<uint8_t>(q[2])) << 16) |
                                                        (static_cast<uint32_t>(static_cast<uint8_t>(q[3])) << 24);
                } else {
                    out[0] = q[0];
                }
            }
        }
    }
}

// Drop/pad mode with dynamic quantisation: capacity rows beyond an expert's (capped) count get scale 0.
__global__ void ZeroUnusedScaleKernel(float* expandedScale, const int32_t* binTotal, int32_t capacity, int32_t experts) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= experts * capacity) return;
    if (i % capacity >= binTotal[i / capacity]) expandedScale[i] = 0.0f;
}

// V3: expandedScale[destination] = scale[source / K] through the scatter-type map.
__global__ void ScatterScaleKernel(const float* scale, float* expandedScale, const int32_t* rowIdx, int64_t total,
                                   int32_t topK) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const int32_t d = rowIdx[i];
    if (d >= 0) expandedScale[d] = scale[i / topK];
}

int CeilLog2(int64_t v) {
    int b = 0;
    while ((1ll << b) < v) ++b;
    return b;
}

class InitRoutingExecutor : public aclOpExecutor {
   public:
    // problem
    const char* x = nullptr;
    const int32_t* expertIdx = nullptr;
    char* expandedX = nullptr;
    int32_t* expandedRowIdx = nullptr;
    int32_t* countOrCumsum = nullptr;
    int32_t* beforeCapacity = nullptr;
    int64_t tokens = 0, topK = 0, rowBytes = 0, total = 0, activeRows = 0;
    int64_t expertNum = 0, capacity = 0;
    int dropPad = 0, countFlag = 0;
    // V3 only
    bool v3 = false;
    int32_t expertStart = 0, expertEnd = 0;  // active range; keys are remapped when it is not [0, expertNum)
    bool remap = false;
    int32_t* gatherIdxOut = nullptr;          // rowIdxType 0: the caller's index output is the gather-type map
    int64_t* count64 = nullptr;
    int countMode = 1;
    int32_t kvPairs = 0;
    const float* scale = nullptr;
    float* expandedScale = nullptr;
    bool dynamicQuant = false;                // quantMode 1: `scale` is the optional smooth scale [active, cols]
    bool smoothPerExpert = true;              // false: the smooth scale is one row [1, cols] for every expert
    int64_t smoothRows = 0;                   // rows of the smooth scale
    const float* staticScale = nullptr;       // MoeInitRoutingQuantV2 quantMode 0: scale[1], offset[1] on the device
    const float* staticOffset = nullptr;
    int32_t xDtype = ACL_FLOAT;
    int64_t cols = 0;
    uint64_t offRemapKeys = 0, offCounts = 0, offScatterMap = 0;
    // plan
    int passes = 1;
    int bitsPerPass[4] = {0, 0, 0, 0};
    int keyBits = 0;
    bool signedRange = false;  // id range unknown: sort all 32 bits, sign-aware
    int32_t sliceLen = 0, numSlices = 0;
    bool smallSort = false;
    uint64_t offKeys[2] = {0, 0}, offPayload[2] = {0, 0}, offTable = 0, offBinBase = 0, offBinTotal = 0;

    void Plan() {
        if (expertNum > 0) {
            keyBits = CeilLog2(expertNum);
            if (keyBits < 1) keyBits = 1;
        } else {
            keyBits = 32;
            signedRange = true;
        }
        passes = (keyBits + kMaxDigitBits - 1) / kMaxDigitBits;
        int left = keyBits;
        for (int i = 0; i < passes; ++i) {
            const int remainingPasses = passes - i;
            bitsPerPass[i] = (left + remainingPasses - 1) / remainingPasses;
            left -= bitsPerPass[i];
        }
        // Slices: at most 1024 so the scan's serial walk stays short; at least 256 keys each.
        int64_t len = (total + 1023) / 1024;
        if (len < 256) len = 256;
        len = (len + kWaveSize - 1) / kWaveSize * kWaveSize;
        sliceLen = static_cast<int32_t>(len);
        numSlices = static_cast<int32_t>((total + len - 1) / len);
        if (numSlices < 1) numSlices = 1;
        // decode-sized inputs: the whole single-pass sort in one workgroup, one slice per wave
        smallSort = passes == 1 && bitsPerPass[0] <= CeilLog2(kSmallSortBins) && total <= kSmallSortMaxKeys;
        if (smallSort) {
            len = (total + kSmallSortWaves - 1) / kSmallSortWaves;
            len = (len + kWaveSize - 1) / kWaveSize * kWaveSize;
            if (len < kWaveSize) len = kWaveSize;
            sliceLen = static_cast<int32_t>(len);
            numSlices = kSmallSortWaves;
        }

        uint64_t off = 0;
        auto take = [&](uint64_t bytes) {
            const uint64_t o = off;
            off += opapi::AlignUp(bytes, 256);
            return o;
        };
        const bool needSortedKeys = passes > 1;
        for (int i = 0; i < 2; ++i) {
            offKeys[i] = needSortedKeys ? take(static_cast<uint64_t>(total) * 4) : 0;
            offPayload[i] = passes > 1 ? take(static_cast<uint64_t>(total) * 4) : 0;
        }
        offTable = take(static_cast<uint64_t>(numSlices) * kMaxBins * 4);
        offBinBase = take(kMaxBins * 4);
        offBinTotal = take(kMaxBins * 4);
        if (v3) {
            offRemapKeys = remap ? take(static_cast<uint64_t>(total) * 4) : 0;
            offCounts = take(static_cast<uint64_t>(expertNum) * 4);
            offScatterMap = gatherIdxOut != nullptr ? take(static_cast<uint64_t>(total) * 4) : 0;
        }
        workspaceBytes = total > 0 ? off : 0;
    }

    // V3 counts or cumsum over the whole expert range come straight out of the scan kernel (one launch fewer);
    // key/value pairs and a proper sub-range (whose sentinel bin must not be counted) go through CountV3Kernel.
    bool WideCountsFromScan() const { return v3 && !remap && countMode != 2 && passes == 1; }

    // Four-byte rows with nothing else riding along: the sort's last scatter copies the rows itself.
    bool SortCopiesRows() const {
        return rowBytes == 4 && tokens > 0 && !dropPad && scale == nullptr && !dynamicQuant && staticScale == nullptr &&
               (reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(expandedX)) % 4 == 0;
    }

    // Decode-sized calls whose rows are copied unchanged in 16-byte packets: the one-workgroup sort and the row gather
    // run as one launch (SmallSortGatherKernel).
    bool SortGathersRows() const {
        const uintptr_t align = reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(expandedX) |
                                static_cast<uintptr_t>(rowBytes);
        return smallSort && rowBytes >= 16 && align % 16 == 0 && tokens > 0 && tokens <= kFusedGatherMaxTokens &&
               topK <= kMaxCachedK && tokens * topK == total && !dropPad && !dynamicQuant && staticScale == nullptr &&
               !SortCopiesRows();
    }

    template <typename Vec>
    void LaunchGather(char* ws, hipStream_t stream) const {
        if (dropPad) {
            const int32_t* binTotal = reinterpret_cast<const int32_t*>(ws + offBinTotal);
            hipLaunchKernelGGL(ZeroUnusedCapacityKernel<Vec>, dim3(static_cast<unsigned>(expertNum * capacity)),
                               dim3(kGatherThreads), 0, stream, expandedX, binTotal, static_cast<int32_t>(capacity),
                               rowBytes);
        }
        GatherArgs g{x, expandedX, expandedRowIdx, rowBytes, tokens, static_cast<int32_t>(topK),
                     dropPad ? expertNum * capacity : activeRows, scale, expandedScale};
        hipLaunchKernelGGL(GatherRowsKernel<Vec>, dim3(static_cast<unsigned>(tokens)), dim3(kGatherThreads), 0, stream,
                           g);
    }

    aclnnStatus Run(void* workspace, hipStream_t stream) override {
        if (total == 0) {
            if (v3) {  // nothing routed: the count output is still defined (all zero)
                CountV3Args ca{nullptr, count64, expertEnd - expertStart, expertStart, countMode, kvPairs};
                hipLaunchKernelGGL(CountV3Kernel, dim3(1), dim3(1024), 0, stream, ca);
            }
            return ACLNN_SUCCESS;
        }
        char* ws = static_cast<char*>(workspace);
        const unsigned sortBlocks = static_cast<unsigned>((numSlices + kWavesPerBlock - 1) / kWavesPerBlock);
        int shift = 0;
        const int32_t* keysIn = expertIdx;
        const int32_t* payloadIn = nullptr;
        if (v3) {
            // expertNum counts the sort's key values here: the active experts plus, when remapping, the sentinel
            if (remap) {
                int32_t* keys = reinterpret_cast<int32_t*>(ws + offRemapKeys);
                hipLaunchKernelGGL(RemapKeysKernel, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0, stream,
                                   expertIdx, keys, total, expertStart, expertEnd);
                keysIn = keys;
            }
            countOrCumsum = reinterpret_cast<int32_t*>(ws + offCounts);  // int32 counts of every key value
            if (gatherIdxOut != nullptr) expandedRowIdx = reinterpret_cast<int32_t*>(ws + offScatterMap);
        }
        for (int pass = 0; pass < passes; ++pass) {
            const bool last = pass == passes - 1;
            SortPass p{};
            p.keysIn = keysIn;
            p.payloadIn = payloadIn;
            p.keysOut = passes > 1 ? reinterpret_cast<int32_t*>(ws + offKeys[pass & 1]) : nullptr;
            p.payloadOut = last ? nullptr : reinterpret_cast<int32_t*>(ws + offPayload[pass & 1]);
            p.table = reinterpret_cast<int32_t*>(ws + offTable);
            p.binBase = reinterpret_cast<int32_t*>(ws + offBinBase);
            p.binTotal = reinterpret_cast<int32_t*>(ws + offBinTotal);
            p.total = total;
            p.sliceLen = sliceLen;
            p.numSlices = numSlices;
            p.shift = shift;
            p.bits = bitsPerPass[pass];
            p.flipSign = (signedRange && last) ? 1 : 0;
            CountOutputs co{nullptr, nullptr, countFlag, static_cast<int32_t>(expertNum), nullptr, 0};
            if (last && passes == 1) {
                co.countOrCumsum = countOrCumsum;
                co.beforeCapacity = beforeCapacity;
                if (WideCountsFromScan()) {
                    co.wide = count64;
                    co.wideCumsum = countMode == 0 ? 1 : 0;
                }
            }
            InverseMap im{last ? expandedRowIdx : nullptr, dropPad, static_cast<int32_t>(capacity),
                          last ? gatherIdxOut : nullptr, (remap && passes == 1) ? expertEnd - expertStart : -1,
                          nullptr, nullptr, static_cast<int32_t>(topK), activeRows};
            if (last && SortCopiesRows()) {
                im.narrowX = reinterpret_cast<const uint32_t*>(x);
                im.narrowOut = reinterpret_cast<uint32_t*>(expandedX);
            }
            if (smallSort && SortGathersRows()) {
                GatherArgs g{x, expandedX, expandedRowIdx, rowBytes, tokens, static_cast<int32_t>(topK), activeRows, scale,
                             expandedScale};
                opapi::KernelTimer timer("routing_small_sort_gather", stream);
                hipLaunchKernelGGL(SmallSortGatherKernel, dim3(static_cast<unsigned>(tokens)),
                                   dim3(kSmallSortWaves * kWaveSize), 0, stream, p, co, im, g);
                break;
            }
            if (smallSort) {
                opapi::KernelTimer timer("routing_small_sort", stream);
                hipLaunchKernelGGL(SmallSortKernel, dim3(1), dim3(kSmallSortWaves * kWaveSize), 0, stream, p, co, im);
                break;
            }
            {
                opapi::KernelTimer timer("routing_histogram", stream);
                hipLaunchKernelGGL(DigitHistogramKernel, dim3(sortBlocks), dim3(kSortThreads), 0, stream, p);
            }
            {
                opapi::KernelTimer timer("routing_scan", stream);
                hipLaunchKernelGGL(DigitScanKernel, dim3(1), dim3(1024), 0, stream, p, co);
            }
            {
                opapi::KernelTimer timer("routing_scatter", stream);
                hipLaunchKernelGGL(DigitScatterKernel, dim3(sortBlocks), dim3(kSortThreads), 0, stream, p, im);
            }
            keysIn = p.keysOut;
            payloadIn = p.payloadOut;
            shift += bitsPerPass[pass];
        }
        if (passes > 1 && (countOrCumsum != nullptr || beforeCapacity != nullptr)) {
            CountOutputs co{countOrCumsum, beforeCapacity, countFlag, static_cast<int32_t>(expertNum), nullptr, 0};
            const unsigned blocks = static_cast<unsigned>((expertNum + 255) / 256);
            hipLaunchKernelGGL(CountFromSortedKernel, dim3(blocks), dim3(256), 0, stream, keysIn, total, co);
        }
        if (v3 && !WideCountsFromScan()) {
            CountV3Args ca{countOrCumsum, count64, expertEnd - expertStart, expertStart, countMode, kvPairs};
            hipLaunchKernelGGL(CountV3Kernel, dim3(1), dim3(1024), 0, stream, ca);
        }
        if (v3) {
            if (scale != nullptr && !dynamicQuant && !(rowBytes > 0 && tokens > 0)) {  // otherwise the row gather carries the scales
                hipLaunchKernelGGL(ScatterScaleKernel, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0,
                                   stream, scale, expandedScale, expandedRowIdx, total, static_cast<int32_t>(topK));
            }
        }
        if (dynamicQuant || staticScale != nullptr) {
            if (tokens > 0 && cols > 0) {
                opapi::KernelTimer timer("routing_quant_gather", stream);
                if (dropPad) {
                    const int32_t* binTotal = reinterpret_cast<const int32_t*>(ws + offBinTotal);
                    hipLaunchKernelGGL(ZeroUnusedCapacityKernel<uint8_t>, dim3(static_cast<unsigned>(expertNum * capacity)),
                                       dim3(kGatherThreads), 0, stream, expandedX, binTotal, static_cast<int32_t>(capacity), cols);
                    if (dynamicQuant) {
                        hipLaunchKernelGGL(ZeroUnusedScaleKernel, dim3(static_cast<unsigned>((expertNum * capacity + 255) / 256)),
                                           dim3(256), 0, stream, expandedScale, binTotal, static_cast<int32_t>(capacity),
                                           static_cast<int32_t>(expertNum));
                    }
                }
                QuantGatherArgs q{x, reinterpret_cast<int8_t*>(expandedX), expandedScale, expandedRowIdx, expertIdx,
                                  dynamicQuant ? scale : nullptr, cols, dropPad ? expertNum * capacity : activeRows,
                                  static_cast<int32_t>(topK), expertStart, xDtype, smoothPerExpert ? 1 : 0,
                                  static_cast<int32_t>(smoothRows), staticScale,
                                  staticOffset};
                const bool wide = cols % 4 == 0 && reinterpret_cast<uintptr_t>(expandedX) % 4 == 0 &&
                                  reinterpret_cast<uintptr_t>(x) % 16 == 0;
                if (wide) hipLaunchKernelGGL(QuantGatherRowsKernel<4>, dim3(static_cast<unsigned>(tokens)), dim3(kGatherThreads), 0, stream, q);
                else hipLaunchKernelGGL(QuantGatherRowsKernel<1>, dim3(static_cast<unsigned>(tokens)), dim3(kGatherThreads), 0, stream, q);
            }
            return ACLNN_SUCCESS;
        }
        if (rowBytes > 0 && tokens > 0 && !SortCopiesRows() && !SortGathersRows()) {
            opapi::KernelTimer timer("routing_gather", stream);
            const uintptr_t align = reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(expandedX) |
                                    static_cast<uintptr_t>(rowBytes);
            if (align % 16 == 0) LaunchGather<uint4>(ws, stream);
            else if (align % 4 == 0) LaunchGather<uint32_t>(ws, stream);
            else if (align % 2 == 0) LaunchGather<uint16_t>(ws, stream);
            else LaunchGather<uint8_t>(ws, stream);
        }
        return ACLNN_SUCCESS;
    }
};

// Shared first phase of aclnnMoeInitRoutingV2 (quantMode -1: rows are copied) and aclnnMoeInitRoutingQuantV2
// (quantMode 0: static, 1: dynamic quantisation to INT8; rules of
// moe/moe_init_routing_quant_v2/op_host/moe_init_routing_quant_v2_tiling.cpp:132-219).
aclnnStatus PlanRoutingV2(const aclTensor* x, const aclTensor* expertIdx, const aclTensor* scaleOptional,
                          const aclTensor* offsetOptional, int64_t activeNum, int64_t expertCapacity, int64_t expertNum,
                          int64_t dropPadMode, int64_t expertTokensCountOrCumsumFlag, bool expertTokensBeforeCapacityFlag,
                          int64_t quantMode, const aclTensor* expandedXOut, const aclTensor* expandedRowIdxOut,
                          const aclTensor* expertTokensCountOrCumsumOut, const aclTensor* expertTokensBeforeCapacityOut,
                          const aclTensor* dynamicQuantScaleOut, uint64_t* workspaceSize, aclOpExecutor** executor) {
    using namespace opapi;
    ClearError();
    OPAPI_CHECK_NOTNULL(x, "x");
    OPAPI_CHECK_NOTNULL(expertIdx, "expertIdx");
    OPAPI_CHECK_NOTNULL(expandedXOut, "expandedXOut");
    OPAPI_CHECK_NOTNULL(expandedRowIdxOut, "expandedRowIdxOut");
    OPAPI_CHECK_NOTNULL(workspaceSize, "workspaceSize");
    OPAPI_CHECK_NOTNULL(executor, "executor");

    constexpr aclnnStatus kInvalid = ACLNN_ERR_PARAM_INVALID;
    OPAPI_CHECK(x->dtype == ACL_FLOAT || x->dtype == ACL_FLOAT16 || x->dtype == ACL_BF16 || x->dtype == ACL_INT8, kInvalid,
                "x dtype %d is not supported (FLOAT, FLOAT16, BF16, INT8)", (int)x->dtype);
    OPAPI_CHECK(expertIdx->dtype == ACL_INT32, kInvalid, "expertIdx must be INT32");
    const bool quant = quantMode >= 0;
    if (quant) {
        OPAPI_CHECK(quantMode == 0 || quantMode == 1, kInvalid, "The quantMode should be 0 or 1.");
        OPAPI_CHECK(x->dtype != ACL_INT8, kInvalid, "quantisation takes FLOAT, FLOAT16 or BF16 rows, not INT8");
        OPAPI_CHECK(expandedXOut->dtype == ACL_INT8, kInvalid, "expandedXOut must be INT8 when the rows are quantised");
    } else {
        OPAPI_CHECK(expandedXOut->dtype == x->dtype, kInvalid, "expandedXOut dtype must equal x dtype");
    }
    OPAPI_CHECK(expandedRowIdxOut->dtype == ACL_INT32, kInvalid, "expandedRowIdxOut must be INT32");
    OPAPI_CHECK(x->dims.size() == 2, kInvalid, "The dim number of x should be 2.");
    OPAPI_CHECK(expertIdx->dims.size() == 2, kInvalid, "The dim number of expertIdx should be 2.");
    OPAPI_CHECK(x->dims[0] == expertIdx->dims[0], kInvalid, "The first dim of x and expertIdx should be equal.");
    OPAPI_CHECK(activeNum >= 0, kInvalid, "The activeNum cannot be less than 0.");
    OPAPI_CHECK(expertCapacity >= 0, kInvalid, "The expertCapacity cannot be less than 0.");
    OPAPI_CHECK(expertNum >= 0, kInvalid, "The expertNum cannot be less than 0.");
    OPAPI_CHECK(dropPadMode == 0 || dropPadMode == 1, kInvalid, "The dropPadMode should be 0 or 1.");
    OPAPI_CHECK(!(dropPadMode > 0 && (expertCapacity < 1 || expertNum < 1)), kInvalid,
                "The expertCapacity and expertNum should be greater than 0 when dropPadMode is 1");
    OPAPI_CHECK(expertTokensCountOrCumsumFlag >= 0 && expertTokensCountOrCumsumFlag <= 2, kInvalid,
                "The expertTokensCountOrCumsumFlag should be 0, 1 or 2.");
    OPAPI_CHECK(!(expertTokensCountOrCumsumFlag > 0 && expertNum <= 0), kInvalid,
                "The expertNum should be greater than 0 when expertTokensCountOrCumsumFlag is greater than 0");
    OPAPI_CHECK(!(dropPadMode > 0 && expertCapacity > x->dims[0]), kInvalid,
                "The first dim of x cannot be less than expertCapacity");
    OPAPI_CHECK(!(dropPadMode > 0 && expertNum > kMaxBins), kInvalid,
                "dropPadMode 1 supports at most %d experts in this build", kMaxBins);
    // drop/pad never emits count-or-cumsum; dropless never emits before-capacity counts
    int64_t countFlag = dropPadMode == 1 ? 0 : expertTokensCountOrCumsumFlag;
    bool beforeFlag = dropPadMode == 1 ? expertTokensBeforeCapacityFlag : false;

    // after the attribute rules, so that a negative activeNum is reported as such and not through the shapes built on it
    OPAPI_CHECK_EXTENTS(x, expertIdx, scaleOptional, offsetOptional, expandedXOut, expandedRowIdxOut, expertTokensCountOrCumsumOut,
                        expertTokensBeforeCapacityOut, dynamicQuantScaleOut);
    const int64_t tokens = x->dims[0], cols = x->dims[1], topK = expertIdx->dims[1];
    const int64_t total = tokens * topK;
    OPAPI_CHECK(total < (1ll << 31), kInvalid, "tokens * topK = %lld does not fit int32 row indices", (long long)total);
    int64_t activeRows = total;
    if (dropPadMode > 0) {
        OPAPI_CHECK(expandedXOut->dims.size() == 3, kInvalid, "The dim number of expandedX should be 3.");
        OPAPI_CHECK(expandedXOut->dims[0] == expertNum, kInvalid, "The first dim of expandedX should be %lld.",
                    (long long)expertNum);
        OPAPI_CHECK(expandedXOut->dims[1] == expertCapacity, kInvalid, "The second dim of expandedX should be %lld.",
                    (long long)expertCapacity);
        OPAPI_CHECK(expandedXOut->dims[2] == cols, kInvalid, "The third dim of expandedX should be %lld.", (long long)cols);
        OPAPI_CHECK(expertNum * expertCapacity < (1ll << 31), kInvalid, "expertNum * expertCapacity does not fit int32");
    } else {
        activeRows = activeNum == 0 ? total : (activeNum < total ? activeNum : total);
        OPAPI_CHECK(expandedXOut->dims.size() == 2, kInvalid, "The dim number of expandedX should be 2.");
        OPAPI_CHECK(expandedXOut->dims[0] == activeRows, kInvalid, "The first dim of expandedX should be %lld.",
                    (long long)activeRows);
        OPAPI_CHECK(expandedXOut->dims[1] == cols, kInvalid, "The second dim of expandedX should be %lld.", (long long)cols);
    }
    OPAPI_CHECK(expandedRowIdxOut->dims.size() == 1, kInvalid, "The dim number of expandedRowIdx should be 1.");
    OPAPI_CHECK(expandedRowIdxOut->dims[0] == total, kInvalid, "The first dim of expandedRowIdx should be %lld.",
                (long long)total);
    auto checkTokenCount = [&](const aclTensor* t, const char* name) -> aclnnStatus {
        OPAPI_CHECK(t != nullptr, ACLNN_ERR_PARAM_NULLPTR, "%s must not be null when its flag is set", name);
        OPAPI_CHECK(t->dtype == ACL_INT32, kInvalid, "%s must be INT32", name);
        OPAPI_CHECK(t->dims.size() == 1, kInvalid, "The dim number of %s should be 1.", name);
        OPAPI_CHECK(t->dims[0] == expertNum, kInvalid, "The first dim of %s should be %lld.", name, (long long)expertNum);
        OPAPI_CHECK(IsContiguous(t), kInvalid, "%s must be contiguous", name);
        return ACLNN_SUCCESS;
    };
    if (countFlag != 0) {
        aclnnStatus st = checkTokenCount(expertTokensCountOrCumsumOut, "expertTokensCountOrCumsum");
        if (st != ACLNN_SUCCESS) return st;
    }
    if (beforeFlag) {
        aclnnStatus st = checkTokenCount(expertTokensBeforeCapacityOut, "expertTokensBeforeCapacity");
        if (st != ACLNN_SUCCESS) return st;
    }
    OPAPI_CHECK(IsContiguous(expandedXOut) && IsContiguous(expandedRowIdxOut), kInvalid,
                "expandedXOut and expandedRowIdxOut must be contiguous");  // the inputs may be strided views
    if (total > 0) {
        OPAPI_CHECK(expertIdx->data != nullptr && expandedRowIdxOut->data != nullptr, ACLNN_ERR_PARAM_NULLPTR,
                    "expertIdx / expandedRowIdxOut carry no device memory");
        OPAPI_CHECK(cols == 0 || (x->data != nullptr && expandedXOut->data != nullptr), ACLNN_ERR_PARAM_NULLPTR,
                    "x / expandedXOut carry no device memory");
    }
    bool smoothPerExpert = false;
    if (quantMode == 0) {
        OPAPI_CHECK(scaleOptional != nullptr, ACLNN_ERR_PARAM_NULLPTR, "scale is nullptr!");
        OPAPI_CHECK(offsetOptional != nullptr, ACLNN_ERR_PARAM_NULLPTR, "offset is nullptr!");
        OPAPI_CHECK(scaleOptional->dtype == ACL_FLOAT, kInvalid, "The data type of scale should be float.");
        OPAPI_CHECK(offsetOptional->dtype == ACL_FLOAT, kInvalid, "The data type of offset should be float.");
        OPAPI_CHECK(scaleOptional->dims.size() == 1, kInvalid, "The dim number of scale should be 1.");
        OPAPI_CHECK(scaleOptional->dims[0] == 1, kInvalid, "The first dim of scale should be 1.");
        OPAPI_CHECK(offsetOptional->dims.size() == 1, kInvalid, "The dim number of offset should be 1.");
        OPAPI_CHECK(offsetOptional->dims[0] == 1, kInvalid, "The first dim of offset should be 1.");
        OPAPI_CHECK(scaleOptional->data != nullptr && offsetOptional->data != nullptr, ACLNN_ERR_PARAM_NULLPTR,
                    "scale / offset carry no device memory");
    } else if (quantMode == 1) {
        if (scaleOptional != nullptr) {
            OPAPI_CHECK(scaleOptional->dtype == ACL_FLOAT, kInvalid, "The data type of scale should be float.");
            OPAPI_CHECK(scaleOptional->dims.size() == 2, kInvalid, "The dim number of scale should be 2.");
            OPAPI_CHECK(scaleOptional->dims[0] == 1 || scaleOptional->dims[0] == expertNum, kInvalid,
                        "The first dim of scale should be 1 or expert_num.");
            OPAPI_CHECK(scaleOptional->dims[1] == cols, kInvalid, "The second dim of scale should be %lld.", (long long)cols);
            OPAPI_CHECK(total == 0 || scaleOptional->data != nullptr, ACLNN_ERR_PARAM_NULLPTR, "scale carries no device memory");
            smoothPerExpert = scaleOptional->dims[0] != 1;
        }
        OPAPI_CHECK(dynamicQuantScaleOut != nullptr, ACLNN_ERR_PARAM_NULLPTR, "DynamicQuantScale is nullptr!");
        OPAPI_CHECK(dynamicQuantScaleOut->dtype == ACL_FLOAT, kInvalid, "The data type of dynamicQuantScale should be FLOAT.");
        OPAPI_CHECK(dynamicQuantScaleOut->dims.size() == 1, kInvalid, "The dim number of dynamicQuantScale should be 1.");
        const int64_t want = dropPadMode == 0 ? activeRows : expertNum * expertCapacity;
        OPAPI_CHECK(dynamicQuantScaleOut->dims[0] == want, kInvalid, "The first dim of dynamicQuantScale should be %lld.",
                    (long long)want);
        OPAPI_CHECK(IsContiguous(dynamicQuantScaleOut) && (total == 0 || dynamicQuantScaleOut->data != nullptr), kInvalid,
                    "dynamicQuantScale must be contiguous device memory");
    }

    auto* ex = new (std::nothrow) InitRoutingExecutor();
    OPAPI_CHECK(ex != nullptr, ACLNN_ERR_INNER_CREATE_EXECUTOR, "out of host memory");
    if (quantMode == 0) {
        ex->staticScale = reinterpret_cast<const float*>(DataPtr(scaleOptional));
        ex->staticOffset = reinterpret_cast<const float*>(DataPtr(offsetOptional));
    } else if (quantMode == 1) {
        ex->dynamicQuant = true;
        OPAPI_BIND(ex, scaleOptional, &ex->scale);
        ex->smoothPerExpert = smoothPerExpert;
        ex->smoothRows = scaleOptional != nullptr ? scaleOptional->dims[0] : 0;
        ex->expandedScale = reinterpret_cast<float*>(DataPtr(dynamicQuantScaleOut));
    }
    ex->xDtype = x->dtype;
    ex->cols = cols;
    OPAPI_BIND(ex, x, &ex->x);
    OPAPI_BIND(ex, expertIdx, &ex->expertIdx);
    ex->expandedX = DataPtr(expandedXOut);
    ex->expandedRowIdx = reinterpret_cast<int32_t*>(DataPtr(expandedRowIdxOut));
    ex->countOrCumsum = countFlag != 0 ? reinterpret_cast<int32_t*>(DataPtr(expertTokensCountOrCumsumOut)) : nullptr;
    ex->beforeCapacity = beforeFlag ? reinterpret_cast<int32_t*>(DataPtr(expertTokensBeforeCapacityOut)) : nullptr;
    ex->tokens = tokens;
    ex->topK = topK;
    ex->rowBytes = cols * ElemSize(x->dtype);
    ex->total = total;
    ex->activeRows = activeRows;
    ex->expertNum = expertNum;
    ex->capacity = expertCapacity;
    ex->dropPad = static_cast<int>(dropPadMode);
    ex->countFlag = static_cast<int>(countFlag);
    ex->Plan();
    ex->SealWorkspace(ex->workspaceBytes);
    *workspaceSize = ex->workspaceBytes;
    *executor = ex;
    return ACLNN_SUCCESS;
}

}  // namespace

extern "C" aclnnStatus aclnnMoeInitRoutingV2GetWorkspaceSize(
    const aclTensor* x, const aclTensor* expertIdx, int64_t activeNum, int64_t expertCapacity, int64_t expertNum,
    int64_t dropPadMode, int64_t expertTokensCountOrCumsumFlag, bool expertTokensBeforeCapacityFlag,
    const aclTensor* expandedXOut, const aclTensor* expandedRowIdxOut, const aclTensor* expertTokensCountOrCumsumOut,
    const aclTensor* expertTokensBeforeCapacityOut, uint64_t* workspaceSize, aclOpExecutor** executor) {
    return PlanRoutingV2(x, expertIdx, nullptr, nullptr, activeNum, expertCapacity, expertNum, dropPadMode,
                         expertTokensCountOrCumsumFlag, expertTokensBeforeCapacityFlag, /*quantMode=*/-1, expandedXOut,
                         expandedRowIdxOut, expertTokensCountOrCumsumOut, expertTokensBeforeCapacityOut, nullptr, workspaceSize,
                         executor);
}

extern "C" aclnnStatus aclnnMoeInitRoutingQuantV2GetWorkspaceSize(
    const aclTensor* x, const aclTensor* expertIdx, const aclTensor* scaleOptional, const aclTensor* offsetOptional,
    int64_t activeNum, int64_t expertCapacity, int64_t expertNum, int64_t dropPadMode,
    int64_t expertTokensCountOrCumsumFlag, bool expertTokensBeforeCapacityFlag, int64_t quantMode,
    const aclTensor* expandedXOut, const aclTensor* expandedRowIdxOut, const aclTensor* expertTokensCountOrCumsumOutOptional,
    const aclTensor* expertTokensBeforeCapacityOutOptional, const aclTensor* dynamicQuantScaleOutOptional,
    uint64_t* workspaceSize, aclOpExecutor** executor) {
    if (quantMode < 0 || quantMode > 1) {
        opapi::ClearError();
        opapi::SetError("The quantMode should be 0 or 1.");
        return ACLNN_ERR_PARAM_INVALID;
    }
    return PlanRoutingV2(x, expertIdx, scaleOptional, offsetOptional, activeNum, expertCapacity, expertNum, dropPadMode,
                         expertTokensCountOrCumsumFlag, expertTokensBeforeCapacityFlag, quantMode, expandedXOut,
                         expandedRowIdxOut, expertTokensCountOrCumsumOutOptional, expertTokensBeforeCapacityOutOptional,
                         dynamicQuantScaleOutOptional, workspaceSize, executor);
}

extern "C" aclnnStatus aclnnMoeInitRoutingQuantV2(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor,
                                                  aclrtStream stream) {
    return opapi::RunAndRelease(workspace, workspaceSize, executor, stream);
}

extern "C" aclnnStatus aclnnMoeInitRoutingV2(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor,
                                             aclrtStream stream) {
    return opapi::RunAndRelease(workspace, workspaceSize, executor, stream);
}

// ---------------------------------------------------------------------------------------------- allocation-free second phase
// aclnnMoeInitRoutingV2StaticWorkspace: the second phase of aclnnMoeInitRoutingV2 for callers that cannot allocate
// device memory (code under HIP graph capture, serving loops, harnesses that forbid hipMalloc).  The sort tables that
// the ordinary second phase keeps in the caller's workspace live in a file-scope device array instead; every GPU the
// library runs on holds its own copy of the array until the process ends.
constexpr uint64_t kStaticScratchBytes = 4ull << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {

constexpr int kMaxScratchDevices = 64;

// Device address of `scratch` on the current device.  In host code the array's name is only a stand-in for the symbol:
// the address that kernels can use comes from hipGetSymbolAddress, asked once per device with that device current.
hipError_t StaticScratchOfCurrentDevice(void** out) {
    static std::mutex mu;
    static void* ptrOfDevice[kMaxScratchDevices] = {};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= kMaxScratchDevices) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(mu);
    if (ptrOfDevice[dev] == nullptr) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return e;
        if (p == nullptr) return hipErrorInvalidSymbol;
        ptrOfDevice[dev] = p;
    }
    *out = ptrOfDevice[dev];
    return hipSuccess;
}

}  // namespace

extern "C" aclnnStatus aclnnMoeInitRoutingV2StaticWorkspace(aclOpExecutor* executor, aclrtStream stream) {
    opapi::ClearError();
    if (executor == nullptr) {
        opapi::SetError("aclnnMoeInitRoutingV2StaticWorkspace: executor must not be null");
        return ACLNN_ERR_PARAM_NULLPTR;
    }
    const InitRoutingExecutor* const routing = dynamic_cast<const InitRoutingExecutor*>(executor);
    if (routing == nullptr || routing->v3 || routing->dynamicQuant || routing->staticScale != nullptr) {
        opapi::SetError("aclnnMoeInitRoutingV2StaticWorkspace: the executor was not made by aclnnMoeInitRoutingV2GetWorkspaceSize");
        delete executor;
        return ACLNN_ERR_PARAM_INVALID;
    }
    if (executor->workspaceBytes > kStaticScratchBytes) {
        opapi::SetError("aclnnMoeInitRoutingV2StaticWorkspace: this call needs %llu bytes of workspace, the built-in scratch "
                        "area holds %llu: use aclnnMoeInitRoutingV2 with a caller-provided workspace",
                        (unsigned long long)executor->workspaceBytes, (unsigned long long)kStaticScratchBytes);
        delete executor;
        return ACLNN_ERR_PARAM_INVALID;
    }
    void* ptr = nullptr;
    const hipError_t e = StaticScratchOfCurrentDevice(&ptr);
    if (e != hipSuccess) {
        opapi::SetError("aclnnMoeInitRoutingV2StaticWorkspace: hipGetSymbolAddress failed: %s", hipGetErrorString(e));
        delete executor;
        return ACLNN_ERR_RUNTIME_ERROR;
    }
    // Nothing in the sort tables has to start at zero (every kernel writes what the next one reads), so the contents
    // left by the previous call need no clearing.
    return opapi::RunAndRelease(ptr, kStaticScratchBytes, executor, stream);
}

// ---------------------------------------------------------------------------------------------- aclnnMoeInitRoutingV3
extern "C" aclnnStatus aclnnMoeInitRoutingV3GetWorkspaceSize(
    const aclTensor* x, const aclTensor* expertIdx, const aclTensor* scaleOptional, const aclTensor* offsetOptional,
    int64_t activeNum, int64_t expertCapacity, int64_t expertNum, int64_t dropPadMode, int64_t expertTokensNumType,
    bool expertTokensNumFlag, int64_t quantMode, const aclIntArray* activeExpertRangeOptional, int64_t rowIdxType,
    const aclTensor* expandedXOut, const aclTensor* expandedRowIdxOut, const aclTensor* expertTokensCountOrCumsumOut,
    const aclTensor* expandedScaleOut, uint64_t* workspaceSize, aclOpExecutor** executor) {
    using namespace opapi;
    ClearError();
    OPAPI_CHECK_NOTNULL(x, "x");
    OPAPI_CHECK_NOTNULL(expertIdx, "expertIdx");
    OPAPI_CHECK_NOTNULL(expandedXOut, "expandedXOut");
    OPAPI_CHECK_NOTNULL(expandedRowIdxOut, "expandedRowIdxOut");
    OPAPI_CHECK_NOTNULL(expertTokensCountOrCumsumOut, "expertTokensCountOrCumsumOut");
    OPAPI_CHECK_NOTNULL(workspaceSize, "workspaceSize");
    OPAPI_CHECK_NOTNULL(executor, "executor");
    OPAPI_CHECK_EXTENTS(x, expertIdx, scaleOptional, expandedXOut, expandedRowIdxOut, expertTokensCountOrCumsumOut, expandedScaleOut);
    (void)expertCapacity;  // unused by the reference as well (dropless only)

    constexpr aclnnStatus kInvalid = ACLNN_ERR_PARAM_INVALID;
    // attributes, in the order of the reference's CheckAttr
    int64_t expertStart = 0, expertEnd = expertNum;
    if (activeExpertRangeOptional != nullptr) {
        OPAPI_CHECK(activeExpertRangeOptional->values.size() == 2, kInvalid, "The dim number of expert_range should be 2.");
        expertStart = activeExpertRangeOptional->values[0];
        expertEnd = activeExpertRangeOptional->values[1];
    }
    OPAPI_CHECK(activeNum >= -1, kInvalid, "active_num should be greater than or equal to -1");
    OPAPI_CHECK(expertNum > 0, kInvalid, "expert_num should be greater than 0");
    OPAPI_CHECK(dropPadMode == 0, kInvalid, "drop_pad_mode currently support 0");
    OPAPI_CHECK(expertTokensNumType >= 0 && expertTokensNumType <= 2, kInvalid,
                "expert_tokens_num_type currently not support %lld", (long long)expertTokensNumType);
    OPAPI_CHECK(expertTokensNumFlag, kInvalid, "expert_tokens_num_flag currently support True");
    OPAPI_CHECK(expertStart >= 0, kInvalid, "expert_start should be greater than or equal to 0");
    OPAPI_CHECK(expertStart < expertEnd, kInvalid, "expert_start should be less than expert_end");
    OPAPI_CHECK(expertEnd <= expertNum, kInvalid, "expert_end should be less than or equal to %lld", (long long)expertNum);
    OPAPI_CHECK(expertEnd <= (expertTokensNumType == 2 ? 5120 : 10240), kInvalid,
                "expert_end should be less than or equal to %d%s", expertTokensNumType == 2 ? 5120 : 10240,
                expertTokensNumType == 2 ? " in KEY_VALUE mode" : "");
    OPAPI_CHECK(quantMode == -1 || quantMode == 1, kInvalid, "quant_mode currently support -1 or 1");
    const bool dynamicQuant = quantMode == 1;
    OPAPI_CHECK(rowIdxType == 0 || rowIdxType == 1, kInvalid, "row_idx_type currently support 1 or 0");
    // offset only matters to static quantisation; like the reference, accept a FLOAT tensor and ignore it
    OPAPI_CHECK(offsetOptional == nullptr || offsetOptional->dtype == ACL_FLOAT, kInvalid, "offset must be FLOAT");

    OPAPI_CHECK(x->dtype == ACL_FLOAT || x->dtype == ACL_FLOAT16 || x->dtype == ACL_BF16 || x->dtype == ACL_INT8, kInvalid,
                "x dtype %d is not supported (FLOAT, FLOAT16, BF16, INT8)", (int)x->dtype);
    OPAPI_CHECK(!(dynamicQuant && x->dtype == ACL_INT8), kInvalid, "quant_mode 1 quantises FLOAT, FLOAT16 or BF16 rows, not INT8");
    OPAPI_CHECK(expertIdx->dtype == ACL_INT32, kInvalid, "expertIdx must be INT32");
    OPAPI_CHECK(x->dims.size() == 2, kInvalid, "The dim number of x should be 2.");
    OPAPI_CHECK(expertIdx->dims.size() == 2, kInvalid, "The dim number of expert_idx should be 2.");
    OPAPI_CHECK(x->dims[0] == expertIdx->dims[0], kInvalid, "Input rows should be same.");
    const int64_t tokens = x->dims[0], cols = x->dims[1], topK = expertIdx->dims[1];
    const int64_t total = tokens * topK;
    OPAPI_CHECK(total < (1ll << 31), kInvalid, "tokens * topK = %lld does not fit int32 row indices", (long long)total);
    OPAPI_CHECK(activeNum == -1 || activeNum == total, kInvalid, "active_num currently should equal to %lld(bs*k)",
                (long long)total);
    const int64_t active = expertEnd - expertStart;
    const bool remap = !(expertStart == 0 && expertEnd == expertNum);
    OPAPI_CHECK(active + (remap ? 1 : 0) <= kMaxBins, kInvalid,
                "this build routes at most %d active experts (%d when the range is a proper sub-range)", kMaxBins,
                kMaxBins - 1);

    if (dynamicQuant && scaleOptional != nullptr) {  // smooth scale, one row per active expert
        OPAPI_CHECK(scaleOptional->dtype == ACL_FLOAT, kInvalid, "scale must be FLOAT");
        OPAPI_CHECK(scaleOptional->dims.size() == 2, kInvalid, "The dim number of scale should be 2.");
        OPAPI_CHECK(scaleOptional->dims[0] == active, kInvalid, "The first dim of scale should be %lld", (long long)active);
        OPAPI_CHECK(scaleOptional->dims[1] == cols, kInvalid, "The second dim of scale should be %lld", (long long)cols);
    }
    if (!dynamicQuant && scaleOptional != nullptr) {
        OPAPI_CHECK(scaleOptional->dtype == ACL_FLOAT, kInvalid, "scale must be FLOAT");
        OPAPI_CHECK(scaleOptional->dims.size() == 1, kInvalid, "The dim number of scale should be 1.");
        OPAPI_CHECK(scaleOptional->dims[0] == tokens, kInvalid, "The first dim of scale should be %lld", (long long)tokens);
    }
    if (dynamicQuant || scaleOptional != nullptr) {
        OPAPI_CHECK(expandedScaleOut != nullptr, ACLNN_ERR_PARAM_NULLPTR,
                    "expandedScaleOut must not be null when scale is given or quant_mode is 1");
        OPAPI_CHECK(expandedScaleOut->dtype == ACL_FLOAT && expandedScaleOut->dims.size() == 1 &&
                        expandedScaleOut->dims[0] == total, kInvalid, "expandedScaleOut must be FLOAT [%lld]", (long long)total);
        OPAPI_CHECK(IsContiguous(expandedScaleOut), kInvalid, "expandedScaleOut must be contiguous");
    }
    if (dynamicQuant) OPAPI_CHECK(expandedXOut->dtype == ACL_INT8, kInvalid, "expandedXOut must be INT8 when quant_mode is 1");
    else OPAPI_CHECK(expandedXOut->dtype == x->dtype, kInvalid, "expandedXOut dtype must equal x dtype without quantisation");
    OPAPI_CHECK(expandedXOut->dims.size() == 2 && expandedXOut->dims[0] == total && expandedXOut->dims[1] == cols, kInvalid,
                "expandedXOut must be [%lld, %lld]", (long long)total, (long long)cols);
    OPAPI_CHECK(expandedRowIdxOut->dtype == ACL_INT32 && expandedRowIdxOut->dims.size() == 1 &&
                    expandedRowIdxOut->dims[0] == total, kInvalid, "expandedRowIdxOut must be INT32 [%lld]", (long long)total);
    OPAPI_CHECK(expertTokensCountOrCumsumOut->dtype == ACL_INT64, kInvalid, "expertTokensCountOrCumsumOut must be INT64");
    if (expertTokensNumType == 2) {
        OPAPI_CHECK(expertTokensCountOrCumsumOut->dims.size() == 2 && expertTokensCountOrCumsumOut->dims[0] == expertNum &&
                        expertTokensCountOrCumsumOut->dims[1] == 2, kInvalid,
                    "expertTokensCountOrCumsumOut must be [%lld, 2] in KEY_VALUE mode", (long long)expertNum);
    } else {
        OPAPI_CHECK(expertTokensCountOrCumsumOut->dims.size() == 1 && expertTokensCountOrCumsumOut->dims[0] == active,
                    kInvalid, "expertTokensCountOrCumsumOut must be [%lld]", (long long)active);
    }
    OPAPI_CHECK(IsContiguous(expandedXOut) && IsContiguous(expandedRowIdxOut) && IsContiguous(expertTokensCountOrCumsumOut),
                kInvalid, "the outputs must be contiguous");  // the inputs may be strided views
    OPAPI_CHECK(expertTokensCountOrCumsumOut->data != nullptr, ACLNN_ERR_PARAM_NULLPTR,
                "expertTokensCountOrCumsumOut carries no device memory");
    if (total > 0) {
        OPAPI_CHECK(expertIdx->data != nullptr && expandedRowIdxOut->data != nullptr, ACLNN_ERR_PARAM_NULLPTR,
                    "expertIdx / expandedRowIdxOut carry no device memory");
        OPAPI_CHECK(cols == 0 || (x->data != nullptr && expandedXOut->data != nullptr), ACLNN_ERR_PARAM_NULLPTR,
                    "x / expandedXOut carry no device memory");
        OPAPI_CHECK(scaleOptional == nullptr || scaleOptional->data != nullptr, ACLNN_ERR_PARAM_NULLPTR,
                    "scale carries no device memory");
        OPAPI_CHECK(!(dynamicQuant || scaleOptional != nullptr) || expandedScaleOut->data != nullptr, ACLNN_ERR_PARAM_NULLPTR,
                    "expandedScaleOut carries no device memory");
    }

    auto* ex = new (std::nothrow) InitRoutingExecutor();
    OPAPI_CHECK(ex != nullptr, ACLNN_ERR_INNER_CREATE_EXECUTOR, "out of host memory");
    ex->v3 = true;
    OPAPI_BIND(ex, x, &ex->x);
    OPAPI_BIND(ex, expertIdx, &ex->expertIdx);
    ex->expandedX = DataPtr(expandedXOut);
    if (rowIdxType == 1) ex->expandedRowIdx = reinterpret_cast<int32_t*>(DataPtr(expandedRowIdxOut));
    else ex->gatherIdxOut = reinterpret_cast<int32_t*>(DataPtr(expandedRowIdxOut));
    ex->count64 = reinterpret_cast<int64_t*>(DataPtr(expertTokensCountOrCumsumOut));
    ex->countMode = static_cast<int>(expertTokensNumType);
    // key/value pairs written: min(active + 1, expertNum), as the reference sizes its copy-out
    ex->kvPairs = static_cast<int32_t>(active + 1 < expertNum ? active + 1 : expertNum);
    OPAPI_BIND(ex, scaleOptional, &ex->scale);
    ex->expandedScale = (dynamicQuant || scaleOptional != nullptr) ? reinterpret_cast<float*>(DataPtr(expandedScaleOut)) : nullptr;
    ex->dynamicQuant = dynamicQuant;
    ex->smoothRows = (dynamicQuant && scaleOptional != nullptr) ? scaleOptional->dims[0] : 0;
    ex->xDtype = x->dtype;
    ex->cols = cols;
    ex->expertStart = static_cast<int32_t>(expertStart);
    ex->expertEnd = static_cast<int32_t>(expertEnd);
    ex->remap = remap;
    ex->tokens = tokens;
    ex->topK = topK;
    ex->rowBytes = cols * ElemSize(x->dtype);
    ex->total = total;
    ex->activeRows = total;
    ex->expertNum = active + (remap ? 1 : 0);  // key values the sort sees
    ex->countFlag = 2;                          // the sort emits plain int32 counts; CountV3Kernel shapes the output
    ex->Plan();
    ex->SealWorkspace(ex->workspaceBytes);
    *workspaceSize = ex->workspaceBytes;
    *executor = ex;
    return ACLNN_SUCCESS;
}

extern "C" aclnnStatus aclnnMoeInitRoutingV3(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor,
                                             aclrtStream stream) {
    return opapi::RunAndRelease(workspace, workspaceSize, executor, stream);
}
