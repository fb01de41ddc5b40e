// Row plan, built on the device: the order in which a planned launch hands the rows of one matrix to its workgroups.
// The reference has no counterpart (its kernels take the rows in matrix order, SPMM/spmmesimd2.hpp:63-75).
//
// A planned launch runs one row per four-wave workgroup. Workgroups are dispatched in index order, so the rows that
// take longest should come first, and the first 8 x bins workgroups (bins = compute units of the device) all start at
// once, workgroup i of them on compute unit i mod bins: those rows ("the head") are packed into `bins` bins of equal
// size, longest row first into the least loaded bin that still has room, and bin b becomes the workgroups b, b + bins,
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
//   packing  exactly the sequential rule above, but in batches: with the bins sorted by (load, bin), the next rows go
//            to the bins in that order for as long as no bin that already received a row of this batch would have
//            been the least loaded one again; each batch is found in parallel (one search per bin in the sorted bins)
//            and the sorted order is carried from batch to batch. Rows without nonzeros fill the positions that are
//            left, in order.
#include "common.hpp"
#include "launch.hpp"

namespace dlspm {

namespace {

constexpr int kPlanTile = 2048;     // rows sorted by one workgroup; also the most rows a head can hold
constexpr int kPlanThreads = 1024;  // two keys per thread
constexpr int kPlanMaxBins = 256;   // 8 x bins <= kPlanTile
static_assert(kPlanThreads == 4 * kPlanMaxBins, "the packing counts with four threads per bin");
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

constexpr int kSortedPad = 64;  // the search below looks up to 63 places past the last key
template <typename Word> struct PackKeys {
    alignas(16) Word sorted[2][kPlanMaxBins + kSortedPad];  // the keys of the bins that can take a row, ascending, then all ones
    alignas(16) Word fresh[kPlanMaxBins];                   // the new keys of the bins of one batch
};
struct PackShared {
    union {
        PackKeys<unsigned> narrow;
        PackKeys<u64> wide;
    } keys;
    alignas(16) int wave_min[kPlanThreads / 64];   // per wave: where its bins would end the batch
    alignas(16) int wave_room[kPlanThreads / 64];  // per wave: bins that can still take a row
    alignas(16) int wave_free[2][kPlanThreads / 64];
    template <typename Word> __device__ __forceinline__ PackKeys<Word>& of();
};
template <> __device__ __forceinline__ PackKeys<unsigned>& PackShared::of<unsigned>() { return keys.narrow; }
template <> __device__ __forceinline__ PackKeys<u64>& PackShared::of<u64>() { return keys.wide; }

// sum over the four lanes of a quad, in every lane of it
__device__ __forceinline__ int quad_sum(int x)
{
    x += __builtin_amdgcn_update_dpp(0, x, kDppQuadSwap1, 0xF, 0xF, true);
    x += __builtin_amdgcn_update_dpp(0, x, kDppQuadSwap2, 0xF, 0xF, true);
    return x;
}
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

// How many keys of the ascending array `sorted` (kPlanMaxBins keys, then kSortedPad times all ones) lie below x: a
// search by the four lanes of a quad in two steps of sixteen. First the last key of each sixteenth of the array, four per
// lane: as many of them as lie below x, so many whole sixteenths do; then the sixteen keys that follow, four per lane.
template <typename Word> __device__ __forceinline__ int count_below_sorted(const Word* sorted, int q, Word x)
{
    static_assert(kPlanMaxBins == 256 && kSortedPad >= 16, "two steps of sixteen");
    int n = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) n += sorted[16 * (4 * q + i) + 15] < x ? 1 : 0;
    const int lo = 16 * quad_sum(n);  // <= 256: the sixteen keys from there on exist (padding)
    n = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) n += sorted[lo + 4 * q + i] < x ? 1 : 0;
    return lo + quad_sum(n);
}

// How many of fresh[0 .. n) lie below x (n a multiple of the keys in 64 bytes), summed over the four lanes of a quad:
// lane q looks at the 16-byte chunks q, q + 4, ... (neighbouring lanes read neighbouring chunks: no bank conflicts).
__device__ __forceinline__ int count_below_fresh(const unsigned* fresh, int n, int q, unsigned x)
{
    const uint4* chunk = reinterpret_cast<const uint4*>(fresh);
    int below = 0;
    for (int j = 0; 16 * j < n; ++j) {
        const uint4 k = chunk[4 * j + q];
        below += (k.x < x ? 1 : 0) + (k.y < x ? 1 : 0) + (k.z < x ? 1 : 0) + (k.w < x ? 1 : 0);
    }
    return quad_sum(below);
}
__device__ __forceinline__ int count_below_fresh(const u64* fresh, int n, int q, u64 x)
{
    const ulonglong2* chunk = reinterpret_cast<const ulonglong2*>(fresh);
    int below = 0;
    for (int j = 0; 8 * j < n; ++j) {
        const ulonglong2 k = chunk[4 * j + q];
        below += (k.x < x ? 1 : 0) + (k.y < x ? 1 : 0);
    }
    return quad_sum(below);
}

// The packing proper: rows 0 .. nz-1 of the sorted head (those with nonzeros), longest first, each into the least loaded
// bin that has room (ties: the lower bin). In batches: with the bins ranked by (load, bin), the next rows go to the bins
// in rank order for as long as no bin that already received a row of this batch would have been the least loaded one
// again, i.e. up to the smallest number of keys below any participating bin's key AFTER its new row (a search in the
// sorted keys). The four lanes of a quad keep the books of one bin (identically) and share its searches and counts.
// The order is carried from batch to batch: a bin that took no row moves down by the batch and up by the number of new
// keys below its own; a bin that took one lands behind the untouched keys that its search found below its new key, plus
// the new keys below it. Only the new keys of a batch are counted one by one. Three workgroup barriers per batch.
template <typename Word>
__device__ __forceinline__ void pack_batches(const int* s_len, int head, int nz, int bins, int* s_order, PackShared& sh)
{
    using Key = BinKey<Word>;
    constexpr int kFreshPad = 64 / (int)sizeof(Word);  // one 16-byte chunk per lane of a quad
    PackKeys<Word>& keys = sh.of<Word>();
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int bin = tid >> 2, q = tid & 3;  // kPlanThreads = 4 x kPlanMaxBins
    const int open = min(bins, head);       // bins that exist and have a first workgroup
    int load = 0, cnt = 0;
    Word mine = bin < open ? Key::make(0, bin) : Key::none;  // all ones: cannot take a row (any more)
    int rank = bin;                                          // empty bins rank by number
    for (int i = tid; i < kPlanMaxBins + kSortedPad; i += kPlanThreads) keys.sorted[0][i] = i < open ? Key::make(0, i) : Key::none;
    __syncthreads();
    int with_room = open;  // bins that can still take a row
    int cur = 0;
    int t = 0;  // rows placed so far; the same in every thread
    while (t < nz) {
        const int most = min(with_room, nz - t);  // >= 1: t < nz <= head rows are unplaced, so some bin has room
        const bool takes = mine != Key::none && rank < most;  // row t + rank would go to this bin
        const int len = takes ? s_len[t + rank] : 0;
        const Word after = takes ? Key::make(load + len, bin) : Key::none;
        // the batch ends before the first rank whose bin is no longer below an earlier bin of the batch with its new row
        const int found = count_below_sorted(keys.sorted[cur], q, after);
        const int wave_ends = wave_min(takes ? found : 0x7fffffff);
        if (lane == 0) sh.wave_min[wave] = wave_ends;
        for (int i = tid; i < kPlanMaxBins + kSortedPad; i += kPlanThreads) keys.sorted[cur ^ 1][i] = Key::none;
        __syncthreads();
        const int batch = min(most, min_of_waves(sh.wave_min));  // 1 <= batch <= most
        const bool took = takes && rank < batch;
        if (took) {
            if (q == 0) s_order[cnt * bins + bin] = t + rank;
            load += len;
            cnt += 1;
        }
        const bool room = mine != Key::none && cnt * bins + bin < head;  // the bin's next workgroup exists
        const Word next = room ? Key::make(load, bin) : Key::none;
        // the bins that took a row are the ranks 0 .. batch-1
        if (took && q == 0) keys.fresh[rank] = next;
        const int padded = (batch + kFreshPad - 1) / kFreshPad * kFreshPad;
        if (tid >= batch && tid < padded) keys.fresh[tid] = Key::none;
        const unsigned long long rooms = __ballot(q == 0 && room);
        if (lane == 0) sh.wave_room[wave] = __popcll(rooms);
        __syncthreads();
        with_room = sum_of_waves(sh.wave_room);
        const int place = (took ? found : rank) - batch + count_below_fresh(keys.fresh, padded, q, next);
        if (room && q == 0) keys.sorted[cur ^ 1][place] = next;
        __syncthreads();
        mine = next;
        rank = place;
        cur ^= 1;
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
    // a bin holds at most kHeadPerBin rows, none longer than the first
    if (s_len[0] < (1 << kNarrowLenBits)) pack_batches<unsigned>(s_len, head, nz, bins, s_order, sh);
    else pack_batches<u64>(s_len, head, nz, bins, s_order, sh);
    if (nz == head) return;  // (the loop above ended with a barrier)
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

// plan entry p <- `row`
__device__ __forceinline__ void emit(int* __restrict__ plan, int M, long long p, long long row, const int* __restrict__ row_offsets)
{
    const int r = (int)min(max(row, 0ll), (long long)M - 1);
    plan[p] = row_offsets[r];
    plan[(size_t)M + p] = row_offsets[r + 1];
    plan[2 * (size_t)M + p] = r;
}

struct HeadShared {
    int len[kPlanTile];    // of the sorted rows
    int row[kPlanTile];
    int order[kPlanTile];  // which sorted row a workgroup of the head takes
    PackShared pack;
};

// M <= kPlanTile: the whole build in one workgroup
__global__ __launch_bounds__(kPlanThreads) void plan_one_block_kernel(int M, const int* __restrict__ row_offsets,
                                                                      int* __restrict__ plan, int bins, int order)
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
    for (int p = threadIdx.x; p < M; p += kPlanThreads) emit(plan, M, p, hs.row[p < head ? hs.order[p] : p], row_offsets);
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
                                                                 int bins, int order)
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
        if (lane == 0) hs.pack.wave_room[wave] = mine;
        __syncthreads();
        const int nz = sum_of_waves(hs.pack.wave_room);
        __syncthreads();  // wave_room is written again by the packing
        pack_head(hs.len, head, nz, bins, order, hs.order, hs.pack);
        for (int p = threadIdx.x; p < head; p += kPlanThreads) emit(plan, M, p, hs.row[hs.order[p]], row_offsets);
        return;
    }
    const long long stride = (long long)(gridDim.x - 1) * kPlanThreads;
    for (long long p = head + (long long)(blockIdx.x - 1) * kPlanThreads + threadIdx.x; p < M; p += stride)
        emit(plan, M, p, wide_row(sorted[p]), row_offsets);
}

}  // namespace

// 3 x M ints of plan; beyond one tile also two key arrays of M entries each, behind the plan, for the merge passes
size_t row_plan_bytes(int M)
{
    if (M <= 0) return 0;
    const size_t plan = (size_t)3 * (size_t)M * sizeof(int);
    return M <= kPlanTile ? plan : (plan + 7) / 8 * 8 + (size_t)2 * (size_t)M * sizeof(u64);
}

hipError_t row_plan_build_launch(int M, const int* row_offsets, int* plan, int bins, int order, hipStream_t stream)
{
    if (M <= 0) return hipSuccess;
    bins = bins < 1 ? 1 : bins > kPlanMaxBins ? kPlanMaxBins : bins;
    if (M <= kPlanTile) {
        hipLaunchKernelGGL(plan_one_block_kernel, dim3(1), dim3(kPlanThreads), 0, stream, M, row_offsets, plan, bins, order);
        return hipGetLastError();
    }
    u64* keys_a = reinterpret_cast<u64*>(reinterpret_cast<char*>(plan) + ((size_t)3 * (size_t)M * sizeof(int) + 7) / 8 * 8);
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
    hipLaunchKernelGGL(plan_emit_kernel, dim3(blocks), dim3(kPlanThreads), 0, stream, M, row_offsets, in, plan, bins, order);
    return hipGetLastError();
}

}  // namespace dlspm
