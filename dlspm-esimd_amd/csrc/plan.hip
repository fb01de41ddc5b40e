// Row plan, built on the device: the order in which a planned launch hands the rows of one matrix to its workgroups.
// The reference has no counterpart (its kernels take the rows in matrix order, SPMM/spmmesimd2.hpp:63-75).
//
// A planned launch runs one row per four-wave workgroup. Workgroups are dispatched in index order, so the rows that
// take longest should come first, and the first 8 x bins workgroups (bins = compute units of the device) all start at
// once, workgroup i of them on compute unit i mod bins: those rows ("the head") are packed into `bins` bins of equal
// size, longest row first into the least loaded bin (of its group, see below) that still has room, and bin b becomes the workgroups b, b + bins,
// b + 2 bins, ... so that a compute unit's rows add up to about the same number of nonzeros. The rows after the head
// follow longest first (whatever compute unit frees up takes the longest row left).
//
// Everything is kernels on the caller's stream: no copy to the host, no synchronisation, nothing that a HIP graph
// cannot capture. Up to 2048 rows it is ONE launch of one workgroup (sort, packing and output); beyond that the rows are
// sorted in tiles of 2048 by as many workgroups, merged in log2(tiles) passes, and one more launch packs the head and
// writes the plan.
//   sort     longest first and by row number among equals: a bitonic network over the 2048 keys of a tile, two per
//            thread in registers (32-bit keys; 64-bit keys in LDS when a row has 2^21 nonzeros or more); merging by rank
//            (every key finds its place in the sibling run by binary search).
//   packing  the bins in groups of at most 64, one wave per group (sorted row t and bin b in group t % groups and
//            b % groups), each group exactly by the sequential rule above, but in batches: with the bins sorted by
//            (load, bin), the next rows go to the bins in that order for as long as no bin that already received a row of
//            this batch would have been the least loaded one again; each batch is found in parallel (one search per bin
//            in the sorted bins) and the sorted order is carried from batch to batch. Rows without nonzeros fill the
//            positions that are left, in order.
#include "common.hpp"
#include "launch.hpp"

namespace dlspm {

namespace {

constexpr int kPlanTile = 2048;     // rows sorted by one workgroup; also the most rows a head can hold
constexpr int kPlanThreads = 1024;  // two keys per thread
constexpr int kPlanMaxBins = 256;   // 8 x bins <= kPlanTile
static_assert(kPlanTile == 2 * kPlanThreads, "the register sort holds two keys per thread");
constexpr int kHeadPerBin = 8;      // workgroups of a four-wave kernel that a compute unit holds at once
// While every row of a tile is shorter than 2^21 its sort keys fit 32 bits (length << 11 | 2047 - row in tile) and are
// sorted in registers; a bin of at most eight such rows stays below 2^24, so its (load << 8 | bin) fits 32 bits too.
constexpr int kNarrowLenBits = 21;
static_assert(kPlanTile == 1 << (32 - kNarrowLenBits), "a 32-bit sort key holds the row's place in its tile below the length");
static_assert(((long long)kHeadPerBin << kNarrowLenBits) <= (1ll << 24), "a narrow bin's load fits 24 bits");

typedef unsigned long long u64;

// longest first, and by row number among equals, is "descending" in both key formats
__device__ __forceinline__ u64 wide_key(int len, long long row) { return ((u64)(unsigned)len << 32) | (u64)(0xFFFFFFFFu - (unsigned)row); }
__device__ __forceinline__ int wide_len(u64 key) { return (int)(key >> 32); }
__device__ __forceinline__ int wide_row(u64 key) { return (int)(0xFFFFFFFFu - (unsigned)(key & 0xFFFFFFFFu)); }
__device__ __forceinline__ unsigned narrow_key(int len, int local) { return ((unsigned)len << (32 - kNarrowLenBits)) | (unsigned)(kPlanTile - 1 - local); }
__device__ __forceinline__ int narrow_len(unsigned key) { return (int)(key >> (32 - kNarrowLenBits)); }
__device__ __forceinline__ int narrow_local(unsigned key) { return kPlanTile - 1 - (int)(key & (kPlanTile - 1)); }

// ---------------------------------------------------------------------------------------------------------------------
// Sorting one tile

// s_key[0 .. n) sorted descending, n a power of two <= kPlanTile, by the whole workgroup (a bitonic network in LDS, one
// compare-exchange per thread and stage): the general form, for tiles with a row of 2^21 nonzeros or more. Thread t's
// pair of a stage with distance j < 128 lies inside the 128 keys that its own wave works on in every such stage, and a
// wave's LDS accesses execute in order: those stages need no workgroup barrier.
__device__ __forceinline__ void sort_tile_desc(u64* s_key, int n)
{
    const int t = threadIdx.x;
    for (int k = 2; k <= n; k <<= 1) {
        for (int j = k >> 1; j > 0; j >>= 1) {
            if (t < (n >> 1)) {
                const int i = ((t & ~(j - 1)) << 1) | (t & (j - 1));  // lower index of the pair (i, i + j)
                const u64 a = s_key[i], b = s_key[i + j];
                const bool descending = (i & k) == 0;  // blocks alternate direction; the last stage is one block
                if ((a < b) == descending) {
                    s_key[i] = b;
                    s_key[i + j] = a;
                }
            }
            // the next stage has distance j / 2, or k (the first stage of the next round) after j == 1
            const int next = j > 1 ? j >> 1 : (k < n ? k : kPlanTile);
            if (j >= 128 || next >= 128) __syncthreads();
            else __builtin_amdgcn_wave_barrier();  // same wave, same 128 keys: program order is enough
        }
    }
}

constexpr int kDppRowShl4 = 0x104;  // lane i <- lane i + 4 of its row of 16
constexpr int kDppRowShr4 = 0x114;  // lane i <- lane i - 4

// minimum and maximum of x and the x of lane ^ m (m a power of two below 64), without LDS
__device__ __forceinline__ void minmax_lane_xor(int m, unsigned x, unsigned& lo, unsigned& hi)
{
    unsigned a = x, b = x;
    switch (m) {
        case 1: b = (unsigned)__builtin_amdgcn_update_dpp(0, (int)x, kDppQuadSwap1, 0xF, 0xF, true); break;
        case 2: b = (unsigned)__builtin_amdgcn_update_dpp(0, (int)x, kDppQuadSwap2, 0xF, 0xF, true); break;
        case 4:  // banks (groups of four lanes) 0 and 2 of a row look four lanes up, banks 1 and 3 four lanes down
            b = (unsigned)__builtin_amdgcn_update_dpp(0, (int)x, kDppRowShl4, 0xF, 0x5, true);
            b = (unsigned)__builtin_amdgcn_update_dpp((int)b, (int)x, kDppRowShr4, 0xF, 0xA, false);
            break;
        case 8: b = (unsigned)__builtin_amdgcn_update_dpp(0, (int)x, kDppRowRor8, 0xF, 0xF, true); break;
        case 16: {  // the swap leaves {own, partner's} in the two results, in an order that depends on the row
            const auto s = __builtin_amdgcn_permlane16_swap(x, x, false, false);
            a = s[0];
            b = s[1];
            break;
        }
        default: {
            const auto s = __builtin_amdgcn_permlane32_swap(x, x, false, false);
            a = s[0];
            b = s[1];
            break;
        }
    }
    lo = min(a, b);
    hi = max(a, b);
}

// The kPlanTile keys of a tile, two per thread (thread t holds elements 2t and 2t + 1), sorted descending: the same
// bitonic network with the keys in registers. Distance 1 is inside the thread, distances 2 .. 64 are lane exchanges
// (DPP, permlane swaps), distances from 128 on go through LDS, alternating between two buffers so that one barrier
// per stage is enough (a buffer is written again only two barriers after it was read).
__device__ __forceinline__ void sort_tile_desc_registers(unsigned& x0, unsigned& x1, uint2 (*s_pair)[kPlanThreads])
{
    const int t = threadIdx.x, e = 2 * t;
    int buf = 0;
#pragma unroll
    for (int k = 2; k <= kPlanTile; k <<= 1) {
        const bool descending = (e & k) == 0;  // blocks of k alternate direction; the last round is one block
#pragma unroll
        for (int j = k >> 1; j > 0; j >>= 1) {
            if (j == 1) {
                const unsigned lo = min(x0, x1), hi = max(x0, x1);
                x0 = descending ? hi : lo;
                x1 = descending ? lo : hi;
                continue;
            }
            const bool keep_max = descending == ((e & j) == 0);  // the lower element of a pair keeps the larger key
            if (j <= 64) {
                unsigned lo, hi;
                minmax_lane_xor(j >> 1, x0, lo, hi);
                x0 = keep_max ? hi : lo;
                minmax_lane_xor(j >> 1, x1, lo, hi);
                x1 = keep_max ? hi : lo;
            } else {
                s_pair[buf][t] = make_uint2(x0, x1);
                __syncthreads();
                const uint2 p = s_pair[buf][t ^ (j >> 1)];
                x0 = keep_max ? max(x0, p.x) : min(x0, p.x);
                x1 = keep_max ? max(x1, p.y) : min(x1, p.y);
                buf ^= 1;
            }
        }
    }
}

// Sum / minimum of the per-wave figures that the waves' first lanes left in s_wave (after a barrier), in every thread:
// each lane reads one of the sixteen (an LDS read costs by the bytes per lane) and the rows of 16 lanes combine them.
static_assert(kPlanThreads / 64 == 16, "one figure per lane of a row");
__device__ __forceinline__ int sum_of_waves(const int* s_wave)
{
    int x = s_wave[threadIdx.x & 15];
    x += __builtin_amdgcn_update_dpp(0, x, kDppQuadSwap1, 0xF, 0xF, true);
    x += __builtin_amdgcn_update_dpp(0, x, kDppQuadSwap2, 0xF, 0xF, true);
    x += __builtin_amdgcn_update_dpp(0, x, kDppRowHalfMirror, 0xF, 0xF, true);
    x += __builtin_amdgcn_update_dpp(0, x, kDppRowMirror, 0xF, 0xF, true);
    return x;
}
__device__ __forceinline__ int min_of_waves(const int* s_wave)
{
    int x = s_wave[threadIdx.x & 15];
    x = min(x, __builtin_amdgcn_update_dpp(0, x, kDppQuadSwap1, 0xF, 0xF, true));
    x = min(x, __builtin_amdgcn_update_dpp(0, x, kDppQuadSwap2, 0xF, 0xF, true));
    x = min(x, __builtin_amdgcn_update_dpp(0, x, kDppRowHalfMirror, 0xF, 0xF, true));
    x = min(x, __builtin_amdgcn_update_dpp(0, x, kDppRowMirror, 0xF, 0xF, true));
    return x;
}

struct SortShared {
    union {
        u64 wide[kPlanTile];
        uint2 pair[2][kPlanThreads];
    } key;
    alignas(16) int wave_max[kPlanThreads / 64];
    alignas(16) int wave_nz[kPlanThreads / 64];
};

// longest row of the tile and the number of its rows that have nonzeros, in every thread (one barrier)
__device__ __forceinline__ void tile_stats(int len0, int len1, SortShared& sh, int& longest, int& nonzero_rows)
{
    int x = max(len0, len1);
    for (int m = 32; m >= 1; m >>= 1) x = max(x, __shfl_xor(x, m));
    const int nz = __popcll(__ballot(len0 > 0)) + __popcll(__ballot(len1 > 0));
    if ((threadIdx.x & 63) == 0) {
        sh.wave_max[threadIdx.x >> 6] = -x;  // (negated: one helper for minima)
        sh.wave_nz[threadIdx.x >> 6] = nz;
    }
    __syncthreads();
    longest = -min_of_waves(sh.wave_max);
    nonzero_rows = sum_of_waves(sh.wave_nz);
}

// Rows [first, first + valid) of the matrix, sorted: sorted place p (0 = longest) is given to put(p, length, row) by
// the thread that ends up holding it, for every p < valid. Returns the number of rows with nonzeros (they come first).
template <typename Put>
__device__ __forceinline__ int sort_tile(const int* __restrict__ row_offsets, long long first, int valid, SortShared& sh, Put put)
{
    const int t = threadIdx.x;
    // the three offsets of a thread's two rows
    int o0 = 0, o1 = 0, o2 = 0;
    if (2 * t < valid) {
        o0 = row_offsets[first + 2 * t];
        o1 = row_offsets[first + 2 * t + 1];
        o2 = 2 * t + 1 < valid ? row_offsets[first + 2 * t + 2] : o1;
    }
    const int len0 = 2 * t < valid ? max(o1 - o0, 0) : 0;  // offsets that decrease count as an empty row
    const int len1 = 2 * t + 1 < valid ? max(o2 - o1, 0) : 0;
    int longest, nonzero_rows;
    tile_stats(len0, len1, sh, longest, nonzero_rows);
    if (longest < (1 << kNarrowLenBits)) {
        // rows beyond `valid` get key 0, below every real key (a real row with key 0 would be row 2047 of a full tile)
        unsigned x0 = 2 * t < valid ? narrow_key(len0, 2 * t) : 0u;
        unsigned x1 = 2 * t + 1 < valid ? narrow_key(len1, 2 * t + 1) : 0u;
        sort_tile_desc_registers(x0, x1, sh.key.pair);
        if (2 * t < valid) put(2 * t, narrow_len(x0), first + narrow_local(x0));
        if (2 * t + 1 < valid) put(2 * t + 1, narrow_len(x1), first + narrow_local(x1));
    } else {
        int n = 2;
        while (n < valid) n <<= 1;
        for (int i = t; i < n; i += kPlanThreads) sh.key.wide[i] = 0ull;
        __syncthreads();
        if (2 * t < valid) sh.key.wide[2 * t] = wide_key(len0, first + 2 * t);
        if (2 * t + 1 < valid) sh.key.wide[2 * t + 1] = wide_key(len1, first + 2 * t + 1);
        __syncthreads();
        sort_tile_desc(sh.key.wide, n);
        for (int p = t; p < valid; p += kPlanThreads) put(p, wide_len(sh.key.wide[p]), (long long)wide_row(sh.key.wide[p]));
    }
    return nonzero_rows;
}

// ---------------------------------------------------------------------------------------------------------------------
// Packing the head

// (load, bin) of a bin as one sortable word: 32 bits while every load stays below 2^24 (bins <= 256), else 64
template <typename Word> struct BinKey;
template <> struct BinKey<unsigned> {
    static constexpr unsigned none = 0xFFFFFFFFu;
    static __device__ __forceinline__ unsigned make(int load, int bin) { return ((unsigned)load << 8) | (unsigned)bin; }
};
template <> struct BinKey<u64> {
    static constexpr u64 none = ~0ull;
    static __device__ __forceinline__ u64 make(int load, int bin) { return ((u64)(unsigned)load << 32) | (u64)bin; }
};

// The bins are packed in groups of at most kGroupBins, one wave per group, each lane of the wave keeping the books of
// one bin: sorted row t and bin b belong to group t % groups and b % groups. A group's rows are every groups-th of the
// sorted rows, so the groups hold the same mix of long and short rows, and what is lost against packing all bins
// together is small (the benchmark matrix: heaviest bin 451 nonzeros instead of 445, mean 413) beside what is won:
// nothing in the loop below leaves the wave -- no workgroup barrier, the ranking of 64 keys instead of 256.
constexpr int kGroupBins = 64;
__host__ __device__ inline int plan_groups(int bins)
{
    int groups = (bins + kGroupBins - 1) / kGroupBins;
    while (bins % groups != 0) ++groups;  // so that row t's group, (t % bins) % groups, is t % groups
    return groups;
}

constexpr int kSortedPad = 8;
template <typename Word> struct GroupKeys {
    alignas(16) Word sorted[kGroupBins + kSortedPad];  // the keys of the bins that can take a row, ascending, then all ones
    alignas(16) Word fresh[kGroupBins];                // the new keys of the bins of one batch
};
struct PackShared {
    union {
        GroupKeys<unsigned> narrow[kPlanThreads / 64];  // one set per wave
        GroupKeys<u64> wide[kPlanThreads / 64];
    } keys;
    alignas(16) int wave_free[2][kPlanThreads / 64];
    template <typename Word> __device__ __forceinline__ GroupKeys<Word>& of(int wave);
};
template <> __device__ __forceinline__ GroupKeys<unsigned>& PackShared::of<unsigned>(int wave) { return keys.narrow[wave]; }
template <> __device__ __forceinline__ GroupKeys<u64>& PackShared::of<u64>(int wave) { return keys.wide[wave]; }

// minimum over the wave, in every lane (all lanes active)
__device__ __forceinline__ int wave_min(int x)
{
    x = min(x, __builtin_amdgcn_update_dpp(0, x, kDppQuadSwap1, 0xF, 0xF, true));
    x = min(x, __builtin_amdgcn_update_dpp(0, x, kDppQuadSwap2, 0xF, 0xF, true));
    x = min(x, __builtin_amdgcn_update_dpp(0, x, kDppRowHalfMirror, 0xF, 0xF, true));
    x = min(x, __builtin_amdgcn_update_dpp(0, x, kDppRowMirror, 0xF, 0xF, true));
    const auto a = __builtin_amdgcn_permlane16_swap((unsigned)x, (unsigned)x, false, false);
    x = min((int)a[0], (int)a[1]);
    const auto b = __builtin_amdgcn_permlane32_swap((unsigned)x, (unsigned)x, false, false);
    return min((int)b[0], (int)b[1]);
}

// How many of the kGroupBins keys of the ascending array `sorted` lie below x (all ones never do): two steps of eight.
// First the last key of each eighth: as many of them as lie below x, so many whole eighths do; then the eight keys
// that follow (they exist: padding). Two round trips to LDS, where a binary search makes seven.
template <typename Word> __device__ __forceinline__ int count_below_sorted(const Word* sorted, Word x)
{
    static_assert(kGroupBins == 64 && kSortedPad >= 8, "two steps of eight");
    int n = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) n += sorted[8 * i + 7] < x ? 1 : 0;
    const int lo = 8 * n;  // <= 64
    n = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) n += sorted[lo + i] < x ? 1 : 0;
    return lo + n;
}

// How many of the kGroupBins keys of fresh[] lie below x (entries that hold no key of the batch are all ones). Every
// lane reads every key -- the addresses are the same for the whole wave -- and all the reads are issued before the first
// comparison: one round trip to LDS, not sixteen.
__device__ __forceinline__ int count_below_fresh(const unsigned* fresh, unsigned x)
{
    const uint4* chunk = reinterpret_cast<const uint4*>(fresh);
    uint4 k[kGroupBins / 4];
#pragma unroll
    for (int j = 0; j < kGroupBins / 4; ++j) k[j] = chunk[j];
    int below = 0;
#pragma unroll
    for (int j = 0; j < kGroupBins / 4; ++j) below += (k[j].x < x ? 1 : 0) + (k[j].y < x ? 1 : 0) + (k[j].z < x ? 1 : 0) + (k[j].w < x ? 1 : 0);
    return below;
}
__device__ __forceinline__ int count_below_fresh(const u64* fresh, u64 x)
{
    const ulonglong2* chunk = reinterpret_cast<const ulonglong2*>(fresh);
    int below = 0;
#pragma unroll
    for (int half = 0; half < 2; ++half) {  // 32 keys in registers at a time
        ulonglong2 k[kGroupBins / 4];
#pragma unroll
        for (int j = 0; j < kGroupBins / 4; ++j) k[j] = chunk[half * (kGroupBins / 4) + j];
#pragma unroll
        for (int j = 0; j < kGroupBins / 4; ++j) below += (k[j].x < x ? 1 : 0) + (k[j].y < x ? 1 : 0);
    }
    return below;
}

// The packing of one group by one wave: the group's rows (sorted rows g, g + groups, ... with nonzeros), longest first,
// each into the least loaded bin of the group that has room (ties: the lower bin). In batches: with the bins ranked by
// (load, bin), the next rows go to the bins in rank order for as long as no bin that already received a row of this
// batch would have been the least loaded one again, i.e. up to the smallest number of keys below any participating
// bin's key AFTER its new row (a search in the sorted keys). The order is carried from batch to batch: a bin that took
// no row moves down by the batch and up by the number of new keys below its own; a bin that took one lands behind the
// untouched keys that its search found below its new key, plus the new keys below it. Lane l keeps the books of the
// group's bin l; LDS accesses of one wave execute in order, so wave barriers (for the compiler) are all it takes.
template <typename Word>
__device__ __forceinline__ void pack_group(const int* s_len, int head, int nz, int bins, int groups, int g, int* s_order,
                                           GroupKeys<Word>& keys)
{
    using Key = BinKey<Word>;
    const int lane = threadIdx.x & 63;
    const int bin = lane * groups + g;                           // this lane's bin, if it exists
    const bool exists = lane < bins / groups && bin < head;      // ... and has a first workgroup
    const int rows = nz > g ? (nz - g + groups - 1) / groups : 0;  // rows of this group
    int load = 0, cnt = 0;
    Word mine = exists ? Key::make(0, lane) : Key::none;  // all ones: cannot take a row (any more)
    int rank = lane;                                      // empty bins rank by number
    keys.sorted[lane] = mine;
    if (lane < kSortedPad) keys.sorted[kGroupBins + lane] = Key::none;
    __builtin_amdgcn_wave_barrier();
    int t = 0;  // rows of the group placed so far
    while (t < rows) {
        const int with_room = __popcll(__ballot(mine != Key::none));
        const int most = min(with_room, rows - t);  // >= 1: the rows left have a place, so some bin has room
        const bool takes = mine != Key::none && rank < most;  // the group's row t + rank would go to this bin
        const int row = (t + rank) * groups + g;              // ... which is this one of the sorted rows
        const int len = takes ? s_len[row] : 0;
        const Word after = takes ? Key::make(load + len, lane) : Key::none;
        // the batch ends before the first rank whose bin is no longer below an earlier bin of the batch with its new row
        const int found = count_below_sorted(keys.sorted, after);
        const int batch = min(most, wave_min(takes ? found : 0x7fffffff));  // 1 <= batch <= most
        const bool took = takes && rank < batch;
        if (took) {
            s_order[cnt * bins + bin] = row;
            load += len;
            cnt += 1;
        }
        const bool room = mine != Key::none && cnt * bins + bin < head;  // the bin's next workgroup exists
        const Word next = room ? Key::make(load, lane) : Key::none;
        // the bins that took a row are the ranks 0 .. batch-1; the rest of fresh[] holds no key
        if (took) keys.fresh[rank] = next;
        if (lane >= batch) keys.fresh[lane] = Key::none;
        __builtin_amdgcn_wave_barrier();
        const int place = (took ? found : rank) - batch + count_below_fresh(keys.fresh, next);
        keys.sorted[lane] = Key::none;
        __builtin_amdgcn_wave_barrier();
        if (room) keys.sorted[place] = next;
        __builtin_amdgcn_wave_barrier();
        mine = next;
        rank = place;
        t += batch;
    }
}

// s_order[p] <- which of the sorted rows 0 .. head-1 workgroup p of the head works on. order: 0 packed (above),
// 1 groups of `bins` alternating between descending and ascending length, 2 plainly descending. nz: how many of the
// head's rows have nonzeros. s_order and s_len are visible to the whole workgroup on entry, s_order holds -1 throughout.
__device__ __forceinline__ void pack_head(const int* s_len, int head, int nz, int bins, int order, int* s_order, PackShared& sh)
{
    const int tid = threadIdx.x;
    if (order != 0) {
        for (int p = tid; p < head; p += kPlanThreads) {
            const int g = p / bins, lo = g * bins, hi = min(lo + bins, head);
            s_order[p] = (order == 1 && (g & 1)) ? lo + hi - 1 - p : p;
        }
        __syncthreads();
        return;
    }
    // a bin holds at most kHeadPerBin rows, none longer than the first: 32-bit (load, bin) words below 2^21 nonzeros
    {
        const int groups = plan_groups(bins), wave = tid >> 6;
        const bool narrow = s_len[0] < (1 << kNarrowLenBits);
        for (int g = wave; g < groups; g += kPlanThreads / 64) {  // wave-uniform
            if (narrow) pack_group<unsigned>(s_len, head, nz, bins, groups, g, s_order, sh.of<unsigned>(wave));
            else pack_group<u64>(s_len, head, nz, bins, groups, g, s_order, sh.of<u64>(wave));
        }
        __syncthreads();
    }
    if (nz == head) return;
    // rows without nonzeros: the positions still free, in ascending order, take the sorted rows nz, nz + 1, ...
    static_assert(kPlanTile == 2 * kPlanThreads, "two positions per thread: tid and tid + kPlanThreads");
    const int lane = tid & 63, wave = tid >> 6;
    const bool free0 = tid < head && s_order[tid] < 0, free1 = tid + kPlanThreads < head && s_order[tid + kPlanThreads] < 0;
    const unsigned long long mask0 = __ballot(free0), mask1 = __ballot(free1);
    if (lane == 0) {
        sh.wave_free[0][wave] = __popcll(mask0);
        sh.wave_free[1][wave] = __popcll(mask1);
    }
    __syncthreads();
    int before0 = 0, before1 = 0, total0 = 0;
#pragma unroll
    for (int x = 0; x < kPlanThreads / 64; ++x) {
        const int c0 = sh.wave_free[0][x], c1 = sh.wave_free[1][x];
        before0 += x < wave ? c0 : 0;
        before1 += x < wave ? c1 : 0;
        total0 += c0;
    }
    const unsigned long long lower = (1ull << lane) - 1;
    if (free0) s_order[tid] = nz + before0 + __popcll(mask0 & lower);
    if (free1) s_order[tid + kPlanThreads] = nz + total0 + before1 + __popcll(mask1 & lower);
    __syncthreads();
}

// plan entry p <- `row`. A cut plan (v_row != nullptr) is built over the rows and pieces in matrix order ("virtual rows":
// row_offsets are then their offsets, M their number): entry p names the matrix row v_row[row] and the slot v_slot[row].
__device__ __forceinline__ void emit(int* __restrict__ plan, int M, long long p, long long row, const int* __restrict__ row_offsets,
                                     const int* __restrict__ v_row, const int* __restrict__ v_slot)
{
    const int r = (int)min(max(row, 0ll), (long long)M - 1);
    if (v_row == nullptr) {
        plan[p] = row_offsets[r];
        plan[(size_t)M + p] = row_offsets[r + 1];
        plan[2 * (size_t)M + p] = r;
    } else {
        // a piece is entered with the range of its WHOLE row: the word says which of how many equal pieces it is, and a
        // launch takes from that the piece's share of the nonzeros (piece_range) or of the columns
        const int word = v_slot[r];
        int first = r, last = r + 1;
        if (word >= 0) {
            first = max(r - ((word >> kPieceNumberShift) & kPieceNumberMask), 0);
            last = min(first + (1 << ((word >> kPieceCountShift) & kPieceCountMask)), M);
        }
        plan[p] = row_offsets[first];
        plan[(size_t)M + p] = row_offsets[last];
        plan[2 * (size_t)M + p] = v_row[r];
        plan[3 * (size_t)M + p] = word;
    }
}

struct HeadShared {
    int len[kPlanTile];    // of the sorted rows
    int row[kPlanTile];
    int order[kPlanTile];  // which sorted row a workgroup of the head takes
    PackShared pack;
};

// M <= kPlanTile: the whole build in one workgroup
__global__ __launch_bounds__(kPlanThreads) void plan_one_block_kernel(int M, const int* __restrict__ row_offsets,
                                                                      int* __restrict__ plan, int bins, int order,
                                                                      const int* __restrict__ v_row,
                                                                      const int* __restrict__ v_slot)
{
    __shared__ SortShared sort;
    __shared__ HeadShared hs;
    const int nonzero_rows = sort_tile(row_offsets, 0, M, sort, [&](int p, int len, long long row) {
        hs.len[p] = len;
        hs.row[p] = (int)row;
        hs.order[p] = -1;
    });
    __syncthreads();
    const int head = min(M, kHeadPerBin * bins);
    pack_head(hs.len, head, min(nonzero_rows, head), bins, order, hs.order, hs.pack);
    for (int p = threadIdx.x; p < M; p += kPlanThreads)
        emit(plan, M, p, hs.row[p < head ? hs.order[p] : p], row_offsets, v_row, v_slot);
}

// M > kPlanTile, step 1: workgroup x sorts the keys of rows [x * kPlanTile, (x + 1) * kPlanTile)
__global__ __launch_bounds__(kPlanThreads) void plan_tile_sort_kernel(int M, const int* __restrict__ row_offsets,
                                                                      u64* __restrict__ keys)
{
    __shared__ SortShared sort;
    const long long first = (long long)blockIdx.x * kPlanTile;
    const int valid = (int)min((long long)kPlanTile, M - first);
    sort_tile(row_offsets, first, valid, sort, [&](int p, int len, long long row) { keys[first + p] = wide_key(len, row); });
}

// step 2, once per doubling of `run`: neighbouring sorted runs of `run` keys are merged. Key i's place is its index in
// its own run plus the number of keys of the sibling run that come before it (all keys differ), found by binary search.
__global__ __launch_bounds__(256) void plan_merge_kernel(long long M, long long run, const u64* __restrict__ in, u64* __restrict__ out)
{
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= M) return;
    const long long base = i / (2 * run) * (2 * run);
    const long long mid = min(base + run, M), end = min(base + 2 * run, M);
    const u64 key = in[i];
    const bool left = i < mid;
    long long lo = left ? mid : base, hi = left ? end : mid;  // the sibling run
    const long long sib = lo;
    while (lo < hi) {  // first key of the sibling run that is below `key`
        const long long m = (lo + hi) >> 1;
        if (in[m] > key) lo = m + 1;
        else hi = m;
    }
    out[base + (i - (left ? base : mid)) + (lo - sib)] = key;
}

// step 3: workgroup 0 packs the head and writes its entries, the others write the entries behind it
__global__ __launch_bounds__(kPlanThreads) void plan_emit_kernel(int M, const int* __restrict__ row_offsets,
                                                                 const u64* __restrict__ sorted, int* __restrict__ plan,
                                                                 int bins, int order, const int* __restrict__ v_row,
                                                                 const int* __restrict__ v_slot)
{
    const int head = min(M, kHeadPerBin * bins);
    if (blockIdx.x == 0) {
        __shared__ HeadShared hs;
        const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
        int mine = 0;  // rows with nonzeros among this thread's
        for (int i = threadIdx.x; i < head; i += kPlanThreads) {
            const u64 key = sorted[i];
            hs.len[i] = wide_len(key);
            hs.row[i] = wide_row(key);
            hs.order[i] = -1;
            mine += wide_len(key) > 0 ? 1 : 0;
        }
        for (int m = 32; m >= 1; m >>= 1) mine += __shfl_xor(mine, m);
        if (lane == 0) hs.pack.wave_free[0][wave] = mine;
        __syncthreads();
        const int nz = sum_of_waves(hs.pack.wave_free[0]);
        __syncthreads();  // wave_free is written again after the packing
        pack_head(hs.len, head, nz, bins, order, hs.order, hs.pack);
        for (int p = threadIdx.x; p < head; p += kPlanThreads)
            emit(plan, M, p, hs.row[hs.order[p]], row_offsets, v_row, v_slot);
        return;
    }
    const long long stride = (long long)(gridDim.x - 1) * kPlanThreads;
    for (long long p = head + (long long)(blockIdx.x - 1) * kPlanThreads + threadIdx.x; p < M; p += stride)
        emit(plan, M, p, wide_row(sorted[p]), row_offsets, v_row, v_slot);
}

// ---------------------------------------------------------------------------------------------------------------------
// Cut rows
//
// A row longer than one compute unit's share of the nonzeros sets the time of the whole launch through the one compute
// unit it runs on. With share = ceil(nnz / bins) (at least 1), piece = ceil(share x piece_pct / 100) and longest =
// max(piece, ceil(share x longest_pct / 100)) (the rule: 75 and 100 per cent), a row of more than `longest` nonzeros is
// cut into c pieces of ceil(length / c) nonzeros (the last one what is left; rows of a few nonzeros can end in empty ones), c the smallest power of two
// with pieces of at most `piece` nonzeros (256 at most) -- a power of two, so that a launch can also give each piece the
// row's whole length and 1/c of the COLUMNS (SpMM), and so that a piece's range follows from its row's by a shift -- and
// the plan is built over the "virtual rows" -- the rows and pieces in matrix order -- like a plan over rows. How many
// there can be: ceil(length / piece) - 1 < length / piece, summed over the cut rows at most nnz / piece <= bins x 100 /
// piece_pct =: extra; rounding up to a power of two at most doubles (pieces - 1) of a row; and fewer than max_cut =
// bins x 100 / longest_pct rows can exceed `longest`. Hence at most 2 x extra entries more than rows and 2 x extra +
// max_cut pieces, whatever the matrix. The plan is sized for those bounds (entries that are not needed hold nothing),
// so its size and the grids of its launches depend on M and the device alone.
// One workgroup: pass 1 counts the nonzeros (from the offsets themselves, so the bounds hold for any array), pass 2
// numbers the virtual rows, the pieces' slots and the cut rows with one running sum over (entries | slots << 32 | cut
// rows << 48), 1024 rows per round.
__global__ __launch_bounds__(kPlanThreads) void plan_cut_kernel(int M, const int* __restrict__ row_offsets, int bins,
                                                                int piece_pct, int longest_pct, int entries, int slots,
                                                                int max_cut,
                                                                int* __restrict__ v_off, int* __restrict__ v_row,
                                                                int* __restrict__ v_slot, int* __restrict__ cut)
{
    __shared__ long long s_nnz[kPlanThreads / 64];
    __shared__ u64 s_scan[kPlanThreads / 64];
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    long long mine = 0;
    for (int i = t; i < M; i += kPlanThreads) mine += max(row_offsets[i + 1] - row_offsets[i], 0);
    for (int m = 32; m >= 1; m >>= 1) mine += __shfl_xor(mine, m);
    if (lane == 0) s_nnz[wave] = mine;
    __syncthreads();
    long long total = 0;
#pragma unroll
    for (int x = 0; x < kPlanThreads / 64; ++x) total += s_nnz[x];
    const long long share = max((total + bins - 1) / bins, 1ll);
    const long long piece_max = max((share * piece_pct + 99) / 100, 1ll);
    const long long longest_whole = max((share * longest_pct + 99) / 100, piece_max);

    u64 carry = 0;  // virtual rows | slots << 32 | cut rows << 48 of the rows before this round
    for (int base = 0; base < M; base += kPlanThreads) {
        const int i = base + t;
        int rs = 0, len = 0, c = 0;
        bool cut_it = false;
        if (i < M) {
            rs = row_offsets[i];
            len = max(row_offsets[i + 1] - rs, 0);
            cut_it = len > longest_whole;
            if (cut_it) {  // the smallest power of two of pieces that are no longer than piece_max, 256 at most
                const long long need = (len + piece_max - 1) / piece_max;
                c = 2;
                while (c < need && c < kMaxPiecesOfARow) c *= 2;
            } else {
                c = 1;
            }
        }
        const u64 x = (u64)c | (cut_it ? ((u64)c << 32) | (1ull << 48) : 0ull);
        u64 inc = x;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const u64 y = __shfl_up(inc, d);
            inc += lane >= d ? y : 0ull;
        }
        if (lane == 63) s_scan[wave] = inc;
        __syncthreads();
        u64 before = carry, round = 0;
#pragma unroll
        for (int xw = 0; xw < kPlanThreads / 64; ++xw) {
            const u64 w = s_scan[xw];
            before += xw < wave ? w : 0ull;
            round += w;
        }
        const u64 ex = before + inc - x;
        const int e0 = (int)(ex & 0xFFFFFFFFull), s0 = (int)((ex >> 32) & 0xFFFFull), j = (int)(ex >> 48);
        if (i < M) {
            if (!cut_it) {
                if (e0 < entries) {
                    v_off[e0] = rs;
                    v_row[e0] = i;
                    v_slot[e0] = -1;
                }
            } else {
                const int lg = 31 - __clz(c);
                const int piece = (len + c - 1) >> lg;
                for (int k = 0; k < c && e0 + k < entries; ++k) {
                    v_off[e0 + k] = rs + min(len, k * piece);
                    v_row[e0 + k] = i;
                    // the slot of the piece's partial row | which piece of its row it is | log2 of how many there are
                    v_slot[e0 + k] = s0 + k < slots ? ((s0 + k) & kPieceSlotMask) | k << kPieceNumberShift | lg << kPieceCountShift
                                                    : -2;  // (beyond the bound: only if the offsets changed under the build)
                }
                if (j < max_cut) {  // one record of four ints per cut row: row, first slot, pieces, 1
                    cut[4 + 4 * j] = i;
                    cut[4 + 4 * j + 1] = s0;
                    cut[4 + 4 * j + 2] = c;
                    cut[4 + 4 * j + 3] = 1;
                }
            }
        }
        carry += round;
        __syncthreads();  // s_scan is written again in the next round
    }
    const long long used = min((long long)(carry & 0xFFFFFFFFull), (long long)entries);
    const int end = M > 0 ? row_offsets[M] : 0;
    for (long long e = used + t; e <= entries; e += kPlanThreads) {
        v_off[e] = end;
        if (e < entries) {
            v_row[e] = -1;
            v_slot[e] = -2;
        }
    }
    const int cut_rows = min((int)(carry >> 48), max_cut);
    for (int j = cut_rows + t; j < max_cut; j += kPlanThreads)  // the records that are not in use say so
        reinterpret_cast<int4*>(cut + 4)[j] = make_int4(0, 0, 0, 0);
    if (t == 0) {
        cut[0] = cut_rows;
        cut[1] = (int)min(share, 0x7fffffffll);
        cut[2] = (int)used;
        cut[3] = 0;
    }
}

// out[row] <- the sum of the row's pieces, in piece order, for every cut row (one workgroup per cut row that the plan has
// room for; those beyond the matrix's own number leave at once). Everything read from the plan is clamped to the arrays.
template <int VEC, int THREADS>
__global__ __launch_bounds__(THREADS) void cut_rows_sum_kernel(int M, int width, int slots,
                                                           const int* __restrict__ cut, const float* __restrict__ pieces,
                                                           float* __restrict__ out)
{
    using VecT = Vec<VEC>;
    // (row, first slot, pieces, in use) of cut row blockIdx.x: one scalar load, the first of two round trips to memory
    const int4 rec = reinterpret_cast<const int4*>(cut + 4)[blockIdx.x];
    if (rec.w == 0) return;
    const int row = min(max(rec.x, 0), M - 1);
    const int first = min(max(rec.y, 0), slots);
    const int cnt = min(max(rec.z, 0), slots - first);
    const float* part = pieces + (size_t)first * width;
    float* orow = out + (size_t)row * width;
    for (int col = threadIdx.x * VEC; col < width; col += THREADS * VEC) {
        const int c = min(col, width - VEC);  // the last thread of a row moves back to the row's last VEC floats
        VecT sum = VecT::zero();
#pragma unroll 4
        for (int k = 0; k < cnt; ++k) sum.add(VecT::gload(part + (size_t)k * width + c));
        sum.gstore(orow + c);
    }
}

}  // namespace

// 3 x M ints of plan; beyond one tile also two key arrays of M entries each, behind the plan, for the merge passes
size_t row_plan_bytes(int M)
{
    if (M <= 0) return 0;
    const size_t plan = (size_t)3 * (size_t)M * sizeof(int);
    return M <= kPlanTile ? plan : (plan + 7) / 8 * 8 + (size_t)2 * (size_t)M * sizeof(u64);
}

// The plan of M rows (or virtual rows, with v_row and v_slot) with offsets row_offsets; `keys`: 2 x M words for the sort
// beyond one tile.
static hipError_t build_plan(int M, const int* row_offsets, int* plan, u64* keys, int bins, int order, const int* v_row,
                             const int* v_slot, hipStream_t stream)
{
    if (M <= 0) return hipSuccess;
    bins = bins < 1 ? 1 : bins > kPlanMaxBins ? kPlanMaxBins : bins;
    if (M <= kPlanTile) {
        hipLaunchKernelGGL(plan_one_block_kernel, dim3(1), dim3(kPlanThreads), 0, stream, M, row_offsets, plan, bins, order,
                           v_row, v_slot);
        return hipGetLastError();
    }
    u64* keys_a = keys;
    u64* keys_b = keys_a + M;
    const unsigned tiles = (unsigned)ceil_div(M, kPlanTile);
    hipLaunchKernelGGL(plan_tile_sort_kernel, dim3(tiles), dim3(kPlanThreads), 0, stream, M, row_offsets, keys_a);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    u64 *in = keys_a, *out = keys_b;
    for (long long run = kPlanTile; run < M; run *= 2) {
        hipLaunchKernelGGL(plan_merge_kernel, dim3((unsigned)ceil_div(M, 256)), dim3(256), 0, stream, (long long)M, run, in, out);
        e = hipGetLastError();
        if (e != hipSuccess) return e;
        u64* tmp = in;
        in = out;
        out = tmp;
    }
    const long long tail_blocks = ceil_div(M, kPlanThreads);
    const unsigned blocks = 1 + (unsigned)(tail_blocks < 2048 ? tail_blocks : 2048);
    hipLaunchKernelGGL(plan_emit_kernel, dim3(blocks), dim3(kPlanThreads), 0, stream, M, row_offsets, in, plan, bins, order,
                       v_row, v_slot);
    return hipGetLastError();
}

hipError_t row_plan_build_launch(int M, const int* row_offsets, int* plan, int bins, int order, hipStream_t stream)
{
    u64* keys = reinterpret_cast<u64*>(reinterpret_cast<char*>(plan) + ((size_t)3 * (size_t)M * sizeof(int) + 7) / 8 * 8);
    return build_plan(M, row_offsets, plan, keys, bins, order, nullptr, nullptr, stream);
}

// ---- cut plan: layout, build, and the sum of the pieces ------------------------------------------------------------

CutPlan cut_plan_layout(int M, int width, int cus)
{
    CutPlan cp{};
    if (M <= 0 || M > kCutPlanMaxRows || width < 0) return cp;  // bytes == 0: no cut plan for this height
    cp.bins = cus < 1 ? 1 : cus > kPlanMaxBins ? kPlanMaxBins : cus;
    const Tuning& t = tuning();
    cp.piece_pct = t.cut_piece_pct > 0 ? t.cut_piece_pct : kCutPiecePct;
    cp.longest_pct = t.cut_longest_pct > 0 ? t.cut_longest_pct : kCutLongestPct;
    const int extra = (cp.bins * 100 + cp.piece_pct - 1) / cp.piece_pct;
    cp.max_cut = (cp.bins * 100 + cp.longest_pct - 1) / cp.longest_pct;
    cp.entries = M + 2 * extra;
    cp.slots = 2 * extra + cp.max_cut;
    auto align = [](size_t x, size_t a) { return (x + a - 1) / a * a; };
    size_t at = align((size_t)4 * cp.entries * sizeof(int), 8);
    cp.off_keys = at;
    if (cp.entries > kPlanTile) at += (size_t)2 * cp.entries * sizeof(u64);
    cp.off_virtual = at;
    at = align(at + ((size_t)3 * cp.entries + 1) * sizeof(int), 16);
    cp.off_cut = at;
    at = align(at + ((size_t)4 + 4 * (size_t)cp.max_cut) * sizeof(int), 256);
    cp.off_pieces = at;
    cp.bytes = at + (size_t)cp.slots * (size_t)width * sizeof(float);
    return cp;
}

hipError_t cut_plan_build_launch(int M, const int* row_offsets, const CutPlan& cp, void* plan, int order, hipStream_t stream)
{
    if (M <= 0 || cp.bytes == 0) return hipErrorInvalidValue;
    char* base = static_cast<char*>(plan);
    int* v_off = reinterpret_cast<int*>(base + cp.off_virtual);
    int* v_row = v_off + cp.entries + 1;
    int* v_slot = v_row + cp.entries;
    int* cut = reinterpret_cast<int*>(base + cp.off_cut);
    hipLaunchKernelGGL(plan_cut_kernel, dim3(1), dim3(kPlanThreads), 0, stream, M, row_offsets, cp.bins, cp.piece_pct,
                       cp.longest_pct, cp.entries, cp.slots, cp.max_cut, v_off, v_row, v_slot, cut);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    return build_plan(cp.entries, v_off, reinterpret_cast<int*>(base), reinterpret_cast<u64*>(base + cp.off_keys), cp.bins, order,
                      v_row, v_slot, stream);
}

hipError_t cut_rows_sum_launch(int M, int width, const CutPlan& cp, const void* plan, float* out, hipStream_t stream)
{
    if (M <= 0 || width <= 0) return hipSuccess;
    const char* base = static_cast<const char*>(plan);
    const int* cut = reinterpret_cast<const int*>(base + cp.off_cut);
    const float* pieces = reinterpret_cast<const float*>(base + cp.off_pieces);
    if (width > 256)
        hipLaunchKernelGGL((cut_rows_sum_kernel<4, 256>), dim3(cp.max_cut), dim3(256), 0, stream, M, width, cp.slots, cut, pieces, out);
    else if (width >= 4)  // one wave covers the row
        hipLaunchKernelGGL((cut_rows_sum_kernel<4, 64>), dim3(cp.max_cut), dim3(64), 0, stream, M, width, cp.slots, cut, pieces, out);
    else
        hipLaunchKernelGGL((cut_rows_sum_kernel<1, 64>), dim3(cp.max_cut), dim3(64), 0, stream, M, width, cp.slots, cut, pieces, out);
    return hipGetLastError();
}

}  // namespace dlspm
