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
//   sort     keys (length << 32 | ~row) descending, i.e. longest first and by row number among equals: a bitonic sort
//            of one tile in LDS; merging by rank (every key finds its place in the sibling run by binary search).
//   packing  exactly the sequential rule above, but in batches: with the bins sorted by (load, bin), the next rows go
//            to the bins in that order for as long as no bin that already received a row of this batch would have
//            been the least loaded one again; each batch is found in parallel (a rank count over the bins and one binary
//            search per bin). Rows without nonzeros fill the positions that are left, in order.
#include "common.hpp"
#include "launch.hpp"

namespace dlspm {

namespace {

constexpr int kPlanTile = 2048;     // rows sorted by one workgroup; also the most rows a head can hold
constexpr int kPlanThreads = 1024;  // one compare-exchange per thread and stage
constexpr int kPlanMaxBins = 256;   // 8 x bins <= kPlanTile
static_assert(kPlanThreads == 4 * kPlanMaxBins, "the packing counts with four threads per bin");
constexpr int kHeadPerBin = 8;      // workgroups of a four-wave kernel that a compute unit holds at once

typedef unsigned long long u64;

__device__ __forceinline__ u64 plan_key(const int* __restrict__ row_offsets, int row)
{
    const int len = max(row_offsets[row + 1] - row_offsets[row], 0);  // offsets that decrease count as an empty row
    return ((u64)(unsigned)len << 32) | (u64)(0xFFFFFFFFu - (unsigned)row);
}
__device__ __forceinline__ int key_len(u64 key) { return (int)(key >> 32); }
__device__ __forceinline__ int key_row(u64 key) { return (int)(0xFFFFFFFFu - (unsigned)(key & 0xFFFFFFFFu)); }

// s_key[0 .. n) sorted descending, n a power of two <= kPlanTile, by the whole workgroup (a bitonic network, one
// compare-exchange per thread and stage). Thread t's pair of a stage with distance j < 128 lies inside the 128 keys
// that its own wave works on in every such stage, and a wave's LDS accesses execute in order: those stages need no
// workgroup barrier, only the stages that exchange keys between waves do (15 barriers instead of 66 for 2048 keys).
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

struct PackShared {
    alignas(16) u64 bkey[kPlanMaxBins];  // (load, bin) of a bin that can still take a row, else all ones (32-bit words: the first half)
    int wave_min[kPlanThreads / 64];     // per wave: where its bins would end the batch
    int wave_room[kPlanThreads / 64];    // per wave: bins that can still take a row
    int wave_free[kPlanThreads / 64];
    int nz;                              // head rows that have nonzeros (they come first in the sorted order)
};

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
    x = min(x, __builtin_amdgcn_update_dpp(x, x, kDppQuadSwap1, 0xF, 0xF, false));
    x = min(x, __builtin_amdgcn_update_dpp(x, x, kDppQuadSwap2, 0xF, 0xF, false));
    x = min(x, __builtin_amdgcn_update_dpp(x, x, kDppRowHalfMirror, 0xF, 0xF, false));
    x = min(x, __builtin_amdgcn_update_dpp(x, x, kDppRowMirror, 0xF, 0xF, false));
    const auto a = __builtin_amdgcn_permlane16_swap((unsigned)x, (unsigned)x, false, false);
    x = min((int)a[0], (int)a[1]);
    const auto b = __builtin_amdgcn_permlane32_swap((unsigned)x, (unsigned)x, false, false);
    return min((int)b[0], (int)b[1]);
}

// How many of the kPlanMaxBins keys lie below x, summed over the four lanes of a quad: lane q of the quad looks at the
// 16-byte chunks q, q + 4, q + 8, ... of the key array (neighbouring lanes read neighbouring chunks: no bank conflicts).
__device__ __forceinline__ int count_below(const unsigned* keys, int q, unsigned x)
{
    const uint4* chunk = reinterpret_cast<const uint4*>(keys);
    int n = 0;
#pragma unroll
    for (int j = 0; j < kPlanMaxBins / 16; ++j) {
        const uint4 k = chunk[4 * j + q];
        n += (k.x < x ? 1 : 0) + (k.y < x ? 1 : 0) + (k.z < x ? 1 : 0) + (k.w < x ? 1 : 0);
    }
    return quad_sum(n);
}
__device__ __forceinline__ int count_below(const u64* keys, int q, u64 x)
{
    const ulonglong2* chunk = reinterpret_cast<const ulonglong2*>(keys);
    int n = 0;
#pragma unroll
    for (int j = 0; j < kPlanMaxBins / 8; ++j) {
        const ulonglong2 k = chunk[4 * j + q];
        n += (k.x < x ? 1 : 0) + (k.y < x ? 1 : 0);
    }
    return quad_sum(n);
}

// The packing proper: rows 0 .. nz-1 of the sorted head (those with nonzeros), longest first, each into the least loaded
// bin that has room (ties: the lower bin). In batches: with the bins ranked by (load, bin), the next rows go to the bins
// in rank order for as long as no bin that already received a row of this batch would have been the least loaded one
// again, i.e. up to the smallest number of keys below any participating bin's key AFTER its new row. Both steps are
// "how many of the 256 keys lie below x", counted by the four lanes of a quad per bin, a quarter of the keys each; lane
// 0 of the quad keeps the bin's books. Two workgroup barriers per batch.
template <typename Word>
__device__ __forceinline__ void pack_batches(const u64* s_key, int head, int nz, int bins, int* s_order, PackShared& sh)
{
    using Key = BinKey<Word>;
    Word* bkey = reinterpret_cast<Word*>(sh.bkey);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int bin = tid >> 2, q = tid & 3;  // kPlanThreads = 4 x kPlanMaxBins
    const bool owner = q == 0 && bin < bins;
    int load = 0, cnt = 0;  // the bin's books, kept by its owner lane
    bool room = owner && bin < head;
    if (q == 0) bkey[bin] = room ? Key::make(0, bin) : Key::none;  // empty bins; beyond `bins`: padding
    unsigned long long rooms = __ballot(room);
    if (lane == 0) sh.wave_room[wave] = __popcll(rooms);
    __syncthreads();
    int t = 0;  // rows placed so far; the same in every thread
    while (t < nz) {
        int with_room = 0;
#pragma unroll
        for (int x = 0; x < kPlanThreads / 64; ++x) with_room += sh.wave_room[x];
        const int most = min(with_room, nz - t);  // >= 1: t < nz <= head rows are unplaced, so some bin has room
        const Word mine = bkey[bin];
        const int rank = count_below(bkey, q, mine);
        const bool takes = mine != Key::none && rank < most;  // row t + rank would go to this bin
        const int len = takes ? key_len(s_key[t + rank]) : 0;
        const int load_now = __builtin_amdgcn_update_dpp(0, load, 0x00, 0xF, 0xF, true);  // quad_perm [0,0,0,0]: the owner's
        const Word after = takes ? Key::make(load_now + len, bin) : Key::none;
        // the batch ends before the first rank whose bin is no longer below an earlier bin of the batch with its new row
        const int ends = takes ? count_below(bkey, q, after) : 0x7fffffff;
        const int wave_ends = wave_min(ends);
        if (lane == 0) sh.wave_min[wave] = wave_ends;
        __syncthreads();
        int batch = most;  // 1 <= batch <= most
#pragma unroll
        for (int x = 0; x < kPlanThreads / 64; ++x) batch = min(batch, sh.wave_min[x]);
        if (owner) {
            if (takes && rank < batch) {
                s_order[cnt * bins + bin] = t + rank;
                load += len;
                cnt += 1;
            }
            room = cnt * bins + bin < head;  // the bin's next workgroup exists
            bkey[bin] = room ? Key::make(load, bin) : Key::none;
        }
        rooms = __ballot(owner && room);
        if (lane == 0) sh.wave_room[wave] = __popcll(rooms);
        __syncthreads();
        t += batch;
    }
}

// s_order[p] <- which of the sorted rows 0 .. head-1 workgroup p of the head works on. order: 0 packed (above),
// 1 groups of `bins` alternating between descending and ascending length, 2 plainly descending.
__device__ __forceinline__ void pack_head(const u64* s_key, int head, int bins, int order, int* s_order, PackShared& sh)
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
    for (int p = tid; p < head; p += kPlanThreads) s_order[p] = -1;
    if (tid == 0) sh.nz = 0;
    __syncthreads();
    for (int p = tid; p < head; p += kPlanThreads)  // the last row with nonzeros (lengths descend)
        if (key_len(s_key[p]) > 0 && (p + 1 == head || key_len(s_key[p + 1]) == 0)) sh.nz = p + 1;
    __syncthreads();
    const int nz = sh.nz;
    // a bin holds at most kHeadPerBin rows, none longer than the first: 32-bit (load, bin) words while that fits 24 bits
    if ((long long)key_len(s_key[0]) * kHeadPerBin < (1ll << 24)) pack_batches<unsigned>(s_key, head, nz, bins, s_order, sh);
    else pack_batches<u64>(s_key, head, nz, bins, s_order, sh);
    // rows without nonzeros: the positions still free, in ascending order, take the sorted rows nz, nz + 1, ...
    const int lane = tid & 63, wave = tid >> 6;
    int next = nz;
    for (int p0 = 0; p0 < head; p0 += kPlanThreads) {
        const int p = p0 + tid;
        const bool is_free = p < head && s_order[p] < 0;
        const unsigned long long mask = __ballot(is_free);
        if (lane == 0) sh.wave_free[wave] = __popcll(mask);
        __syncthreads();
        int before = 0, total = 0;
        for (int x = 0; x < kPlanThreads / 64; ++x) {
            const int c = sh.wave_free[x];
            before += x < wave ? c : 0;
            total += c;
        }
        if (is_free) s_order[p] = next + before + __popcll(mask & ((1ull << lane) - 1));
        next += total;
        __syncthreads();
    }
}

// plan entry p <- the row of `key`
__device__ __forceinline__ void emit(int* __restrict__ plan, int M, int p, u64 key, const int* __restrict__ row_offsets)
{
    const int row = min(max(key_row(key), 0), M - 1);
    plan[p] = row_offsets[row];
    plan[(size_t)M + p] = row_offsets[row + 1];
    plan[2 * (size_t)M + p] = row;
}

// M <= kPlanTile: the whole build in one workgroup
__global__ __launch_bounds__(kPlanThreads) void plan_one_block_kernel(int M, const int* __restrict__ row_offsets,
                                                                      int* __restrict__ plan, int bins, int order)
{
    __shared__ u64 s_key[kPlanTile];
    __shared__ int s_order[kPlanTile];
    __shared__ PackShared sh;
    int n = 2;
    while (n < M) n <<= 1;
    for (int i = threadIdx.x; i < n; i += kPlanThreads) s_key[i] = i < M ? plan_key(row_offsets, i) : 0ull;
    __syncthreads();
    sort_tile_desc(s_key, n);
    const int head = min(M, kHeadPerBin * bins);
    pack_head(s_key, head, bins, order, s_order, sh);
    for (int p = threadIdx.x; p < M; p += kPlanThreads) emit(plan, M, p, s_key[p < head ? s_order[p] : p], row_offsets);
}

// M > kPlanTile, step 1: workgroup x sorts the keys of rows [x * kPlanTile, (x + 1) * kPlanTile)
__global__ __launch_bounds__(kPlanThreads) void plan_tile_sort_kernel(int M, const int* __restrict__ row_offsets,
                                                                      u64* __restrict__ keys)
{
    __shared__ u64 s_key[kPlanTile];
    const long long first = (long long)blockIdx.x * kPlanTile;
    const int valid = (int)min((long long)kPlanTile, M - first);
    for (int i = threadIdx.x; i < kPlanTile; i += kPlanThreads) s_key[i] = i < valid ? plan_key(row_offsets, (int)(first + i)) : 0ull;
    __syncthreads();
    sort_tile_desc(s_key, kPlanTile);  // the padding (key 0) is below every real key and ends up behind them
    for (int i = threadIdx.x; i < valid; i += kPlanThreads) keys[first + i] = s_key[i];
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
        __shared__ u64 s_key[kPlanTile];
        __shared__ int s_order[kPlanTile];
        __shared__ PackShared sh;
        for (int i = threadIdx.x; i < head; i += kPlanThreads) s_key[i] = sorted[i];
        __syncthreads();
        pack_head(s_key, head, bins, order, s_order, sh);
        for (int p = threadIdx.x; p < head; p += kPlanThreads) emit(plan, M, p, s_key[s_order[p]], row_offsets);
        return;
    }
    const long long stride = (long long)(gridDim.x - 1) * kPlanThreads;
    for (long long p = head + (long long)(blockIdx.x - 1) * kPlanThreads + threadIdx.x; p < M; p += stride)
        emit(plan, M, (int)p, sorted[p], row_offsets);
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
