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
constexpr int kHeadPerBin = 8;      // workgroups of a four-wave kernel that a compute unit holds at once

typedef unsigned long long u64;

__device__ __forceinline__ u64 plan_key(const int* __restrict__ row_offsets, int row)
{
    const int len = max(row_offsets[row + 1] - row_offsets[row], 0);  // offsets that decrease count as an empty row
    return ((u64)(unsigned)len << 32) | (u64)(0xFFFFFFFFu - (unsigned)row);
}
__device__ __forceinline__ int key_len(u64 key) { return (int)(key >> 32); }
__device__ __forceinline__ int key_row(u64 key) { return (int)(0xFFFFFFFFu - (unsigned)(key & 0xFFFFFFFFu)); }

// s_key[0 .. n) sorted descending, n a power of two <= kPlanTile, by the whole workgroup
__device__ void sort_tile_desc(u64* s_key, int n)
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
            __syncthreads();
        }
    }
}

struct PackShared {
    u64 bkey[kPlanMaxBins];   // (load, bin) of a bin that can still take a row, else all ones
    u64 skey[kPlanMaxBins];   // the same, sorted ascending
    int sbin[kPlanMaxBins];   // bin at each sorted position
    int load[kPlanMaxBins];   // nonzeros handed to a bin so far
    int cnt[kPlanMaxBins];    // rows handed to a bin so far
    int wave_free[kPlanThreads / 64];
    int nz;                   // head rows that have nonzeros (they come first in the sorted order)
    int batch;                // rows placed by the current batch
    int base;
};

// s_order[p] <- which of the sorted rows 0 .. head-1 workgroup p of the head works on. order: 0 packed (above),
// 1 groups of `bins` alternating between descending and ascending length, 2 plainly descending.
__device__ void pack_head(const u64* s_key, int head, int bins, int order, int* s_order, PackShared& sh)
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
    if (tid < bins) {
        sh.load[tid] = 0;
        sh.cnt[tid] = 0;
    }
    if (tid == 0) sh.nz = 0;
    __syncthreads();
    for (int p = tid; p < head; p += kPlanThreads)  // the last row with nonzeros (lengths descend)
        if (key_len(s_key[p]) > 0 && (p + 1 == head || key_len(s_key[p + 1]) == 0)) sh.nz = p + 1;
    __syncthreads();
    const int nz = sh.nz;
    int t = 0;  // rows placed so far; the same in every thread
    while (t < nz) {
        if (tid < bins) {
            const bool room = sh.cnt[tid] * bins + tid < head;  // the bin's next workgroup exists
            sh.bkey[tid] = room ? ((u64)(unsigned)sh.load[tid] << 32) | (u64)tid : ~0ull;
        }
        if (tid == 0) sh.batch = 0x7fffffff;
        __syncthreads();
        int with_room = 0;
        if (tid < bins) {  // position of this bin among the bins by (load, bin), and how many bins have room
            const u64 mine = sh.bkey[tid];
            int rank = 0;
            for (int k = 0; k < bins; ++k) {
                const u64 other = sh.bkey[k];
                rank += other < mine ? 1 : 0;
                with_room += other != ~0ull ? 1 : 0;
            }
            if (mine != ~0ull) {
                sh.sbin[rank] = tid;
                sh.skey[rank] = mine;
            }
        }
        if (tid == 0) sh.base = with_room;
        __syncthreads();
        const int most = min(sh.base, nz - t);  // >= 1: t < nz <= head rows are unplaced, so some bin has room
        if (tid < most) {
            // Row t + tid would go to the bin at sorted position tid. That holds as long as no earlier bin of this
            // batch, with its new row, is again below a later bin: this bin ends the batch at the first later
            // position whose (load, bin) is not below its own new (load + length, bin).
            const int b = sh.sbin[tid];
            const u64 after = ((u64)(unsigned)(sh.load[b] + key_len(s_key[t + tid])) << 32) | (u64)b;
            int lo = tid + 1, hi = most;
            while (lo < hi) {
                const int mid = (lo + hi) >> 1;
                if (sh.skey[mid] < after) lo = mid + 1;
                else hi = mid;
            }
            atomicMin(&sh.batch, lo);
        }
        __syncthreads();
        const int batch = sh.batch;  // 1 <= batch <= most
        if (tid < batch) {
            const int b = sh.sbin[tid];
            s_order[sh.cnt[b] * bins + b] = t + tid;
            sh.load[b] += key_len(s_key[t + tid]);
            sh.cnt[b] += 1;
        }
        __syncthreads();
        t += batch;
    }
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
