// One look at the matrix, one answer: dlspm_analyze (a single synchronising pass over the CSR structure on the device)
// and dlspm_advise (host only: what to allocate, what to build and which hint bits to pass for an op and a width).
// The reference sizes its launches from M and N alone (SPMM/spmmesimd2.hpp:30-60); everything here is what that leaves
// out: how uneven the rows are, and whether the columns of neighbouring rows lie near each other.
#include "../../include/dlspm_hip.h"

#include <algorithm>
#include <mutex>

#include "common.hpp"
#include "launch.hpp"

namespace dlspm {

namespace {

constexpr int kEighths = 8;  // the row blocks are dealt to eight XCDs; DLSPM_HINT_BANDED gives each a contiguous eighth
// stats: [0] longest row, [1] rows without nonzeros, [2] widest row (largest - smallest column + 1),
// [3 .. 10] smallest column of each eighth of the rows, [11 .. 18] largest, [19 .. 26] nonzeros of each eighth
constexpr int kStats = 3 + 3 * kEighths;

// Where the kernel leaves its figures: one of 64 slots of a static device array (32 ints each), taken for the length of
// one call, and the same slot of a pinned host array (8 KiB per device, allocated at the first call on that device and
// kept) for the copy back. An allocation per call would cost the host several times what the pass itself does
// (hipMalloc + hipFree: about 0.4 ms; a copy into pageable memory: 0.06 ms). With all 64 slots in use at once (64 host
// threads inside dlspm_analyze) a call allocates after all.
constexpr int kSlots = 64, kSlotInts = 32;
static_assert(kStats <= kSlotInts, "a slot holds the figures of one call");
static __device__ __align__(256) int g_analyze_slots[kSlots * kSlotInts];

struct SlotPool {
    std::mutex mutex;
    unsigned long long busy[64] = {};  // per device: bit s set = slot s is in use
    int* base[64] = {};                // per device: the array's address on that device
    int* host[64] = {};                // per device: pinned host memory, slot for slot (nullptr: could not be had)
};
SlotPool& slot_pool()
{
    static SlotPool pool;
    return pool;
}
// A free slot of the current device's array (nullptr: none free, or the address cannot be had); *slot names it for
// release, *pinned is the slot's host side (nullptr: copy into ordinary memory).
int* acquire_slot(int dev, int* slot, int** pinned)
{
    *slot = -1;
    *pinned = nullptr;
    if (dev < 0 || dev >= 64) return nullptr;
    SlotPool& pool = slot_pool();
    std::lock_guard<std::mutex> lock(pool.mutex);
    if (!pool.base[dev]) {
        void* p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(g_analyze_slots)) != hipSuccess || !p) {
            (void)hipGetLastError();
            return nullptr;
        }
        pool.base[dev] = static_cast<int*>(p);
        void* h = nullptr;
        if (hipHostMalloc(&h, sizeof(int) * kSlots * kSlotInts, hipHostMallocDefault) == hipSuccess) pool.host[dev] = static_cast<int*>(h);
        else (void)hipGetLastError();
    }
    for (int s = 0; s < kSlots; ++s) {
        if (!(pool.busy[dev] >> s & 1ull)) {
            pool.busy[dev] |= 1ull << s;
            *slot = s;
            if (pool.host[dev]) *pinned = pool.host[dev] + s * kSlotInts;
            return pool.base[dev] + s * kSlotInts;
        }
    }
    return nullptr;
}
void release_slot(int dev, int slot)
{
    if (slot < 0) return;
    SlotPool& pool = slot_pool();
    std::lock_guard<std::mutex> lock(pool.mutex);
    pool.busy[dev] &= ~(1ull << slot);
}

__global__ void analyze_init_kernel(int* __restrict__ stats)
{
    const int i = threadIdx.x;
    if (i < kStats) stats[i] = (i >= 3 && i < 3 + kEighths) ? 0x7fffffff : (i >= 3 + kEighths && i < 3 + 2 * kEighths) ? -1 : 0;
}

__device__ __forceinline__ int wave_max_int(int x)
{
    for (int m = 32; m >= 1; m >>= 1) x = max(x, __shfl_xor(x, m));
    return x;
}
__device__ __forceinline__ int wave_min_int(int x)
{
    for (int m = 32; m >= 1; m >>= 1) x = min(x, __shfl_xor(x, m));
    return x;
}

// eighth x holds the rows [x * M / 8, (x + 1) * M / 8)
__device__ __forceinline__ int eighth_of(long long row, int M) { return (int)min((row * kEighths) / max(M, 1), (long long)kEighths - 1); }

// Every wave walks a contiguous run of rows (so nearly all of them in one eighth), 64 column indices at a time, and
// keeps its own figures; they reach memory once per eighth and wave.
__global__ __launch_bounds__(256) void analyze_kernel(int M, int K, int rows_per_wave, const int* __restrict__ row_offsets,
                                                      const int* __restrict__ col_indices, int* __restrict__ stats)
{
    const int lane = threadIdx.x & 63;
    const long long wave = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
    const long long first = wave * rows_per_wave;
    if (first >= M) return;
    const int last = (int)min(first + rows_per_wave, (long long)M);
    int longest = 0, empty = 0, widest = 0;
    int cur = eighth_of(first, M), lo = 0x7fffffff, hi = -1;
    auto flush = [&]() {
        if (lane == 0 && hi >= 0) {
            atomicMin(&stats[3 + cur], lo);
            atomicMax(&stats[3 + kEighths + cur], hi);
        }
    };
    for (int r = (int)first; r < last; ++r) {
        const int e = eighth_of(r, M);
        if (e != cur) {
            flush();
            cur = e;
            lo = 0x7fffffff;
            hi = -1;
        }
        const int rs = row_offsets[r], re = row_offsets[r + 1];
        const int len = max(re - rs, 0);
        longest = max(longest, len);
        empty += len == 0 ? 1 : 0;
        int rlo = 0x7fffffff, rhi = -1;
        for (int p = rs + lane; p < re; p += kWave) {
            const int c = min(max(col_indices[p], 0), max(K - 1, 0));
            rlo = min(rlo, c);
            rhi = max(rhi, c);
        }
        rlo = wave_min_int(rlo);
        rhi = wave_max_int(rhi);
        if (rhi >= 0) {
            widest = max(widest, rhi - rlo + 1);
            lo = min(lo, rlo);
            hi = max(hi, rhi);
        }
    }
    flush();
    if (lane == 0) {
        if (longest > 0) atomicMax(&stats[0], longest);
        if (empty > 0) atomicAdd(&stats[1], empty);
        if (widest > 0) atomicMax(&stats[2], widest);
    }
    if (wave == 0 && lane < kEighths) {  // the nonzeros of each eighth, from the offsets at its ends
        const long long a = (long long)lane * M / kEighths, b = (long long)(lane + 1) * M / kEighths;
        stats[3 + 2 * kEighths + lane] = max(row_offsets[b] - row_offsets[a], 0);
    }
}

}  // namespace

}  // namespace dlspm

using namespace dlspm;

extern "C" {

int dlspm_analyze(int M, int K, int nnz, const int* row_offsets, const int* col_indices, void* stream, dlspm_matrix_info* info)
{
    if (!info || M < 0 || K < 0 || nnz < 0) return DLSPM_E_INVALID_ARG;
    if ((long long)nnz > (long long)M * K) return DLSPM_E_INVALID_ARG;
    if (M > 0 && !row_offsets) return DLSPM_E_INVALID_ARG;
    if (nnz > 0 && !col_indices) return DLSPM_E_INVALID_ARG;
    *info = dlspm_matrix_info{M, K, nnz, 0, 0, 0, 0, 0};
    if (M == 0) return DLSPM_OK;
    const DeviceInfo& dev = device_info();
    if (!dev.present || !dev.gfx950) return DLSPM_E_NO_DEVICE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    int device = -1, slot = -1;
    hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess) return fail_hip(e);
    int* pinned = nullptr;
    int* d = acquire_slot(device, &slot, &pinned);
    if (!d) {
        e = hipMalloc(&d, kStats * sizeof(int));
        if (e != hipSuccess) return fail_hip(e);
    }
    int pageable[kStats] = {};
    int* h = pinned ? pinned : pageable;
    hipLaunchKernelGGL(analyze_init_kernel, dim3(1), dim3(64), 0, s, d);
    e = hipGetLastError();
    if (e == hipSuccess) {
        // One to sixteen waves per compute unit, each a run of rows, about 2048 nonzeros per wave: every wave ends with a
        // handful of atomic operations on the same few words, which is what a small matrix would otherwise wait for
        // (2048 rows of 50 nonzeros: 117 us of host time per call with a wave per row, 44 us with eight rows per wave).
        const long long waves_wanted = std::min<long long>(16ll * dev.cus, std::max<long long>(dev.cus, nnz / 2048));
        const int rows_per_wave = (int)std::max<long long>(ceil_div(M, std::max<long long>(waves_wanted, 1)), 1);
        const long long waves = ceil_div(M, rows_per_wave);
        hipLaunchKernelGGL(analyze_kernel, dim3((unsigned)ceil_div(waves, 4)), dim3(256), 0, s, M, K, rows_per_wave, row_offsets,
                           col_indices, d);
        e = hipGetLastError();
    }
    if (e == hipSuccess) e = hipMemcpyAsync(h, d, kStats * sizeof(int), hipMemcpyDeviceToHost, s);
    if (e == hipSuccess) e = hipStreamSynchronize(s);
    int got[kStats];
    for (int i = 0; i < kStats; ++i) got[i] = h[i];
    h = got;  // (the slot, and with it the pinned memory, goes back before the figures are used)
    if (slot >= 0) release_slot(device, slot);
    else (void)hipFree(d);
    if (e != hipSuccess) return fail_hip(e);
    info->max_row_len = h[0];
    info->empty_rows = h[1];
    info->max_col_span = h[2];
    long long cover = 0, heaviest = 0, total = 0;
    for (int x = 0; x < kEighths; ++x) {
        if (h[3 + kEighths + x] >= 0) cover += (long long)h[3 + kEighths + x] - h[3 + x] + 1;
        heaviest = std::max<long long>(heaviest, h[3 + 2 * kEighths + x]);
        total += h[3 + 2 * kEighths + x];
    }
    info->eighths_cover_permille = K > 0 ? (int)std::min<long long>(cover * 1000 / K, 1000ll * kEighths) : 0;
    info->eighths_nnz_permille = total > 0 ? (int)std::min<long long>(heaviest * 1000 * kEighths / total, 1000ll * kEighths) : 0;
    return DLSPM_OK;
}

// A band: every XCD, handed a contiguous eighth of the rows, gathers from about its own eighth of the K-side operand
// (together at most a quarter of what eight L2s fetching everything would: cover <= 2 x K), the eighths hold about the
// same number of nonzeros (or the XCDs would be loaded unevenly), and the operand is large enough for the L2s to matter.
static bool looks_banded(const DeviceInfo& dev, int op, int width, const dlspm_matrix_info& m)
{
    if (m.M < 8 * kEighths || m.nnz <= 0) return false;
    const double operand_bytes = (double)m.K * width * sizeof(float) * (op == DLSPM_OP_FUSED ? 2.0 : 1.0);
    return m.eighths_cover_permille > 0 && m.eighths_cover_permille <= 2000 && m.eighths_nnz_permille <= 1250 &&
           operand_bytes > (double)dev.l2_bytes;
}

constexpr int kClusteredEighthPermille = 1600;  // (1000: every eighth of the rows holds an eighth of the nonzeros)

int dlspm_advise(int op, int N_or_D, const dlspm_matrix_info* info, dlspm_call_plan* plan)
{
    if (!info || !plan || N_or_D < 0) return DLSPM_E_INVALID_ARG;
    if (op != DLSPM_OP_SPMM && op != DLSPM_OP_SDDMM && op != DLSPM_OP_FUSED) return DLSPM_E_INVALID_ARG;
    *plan = dlspm_call_plan{DLSPM_BUILD_NOTHING, 0, 0};
    const int M = info->M, K = info->K, nnz = info->nnz, longest = info->max_row_len;
    if (M <= 0 || K <= 0 || nnz <= 0 || N_or_D <= 0) return DLSPM_OK;
    const DeviceInfo& dev = device_info();
    const bool even = (double)longest <= 1.5 * ((double)nnz / M);
    // 1. a band: row blocks dealt to the XCDs in contiguous runs, no memory (with the even-rows hint where that holds too)
    if (looks_banded(dev, op, N_or_D, *info)) {
        plan->hints = DLSPM_HINT_BANDED | (even ? DLSPM_HINT_ROWS_EVEN : 0);
        return DLSPM_OK;
    }
    // 2. uneven rows: a row plan, with the longest rows cut where that pays
    const int planned = dlspm_row_plan_advice(op, M, K, N_or_D, nnz, longest);
    if (planned == 2) {
        plan->build = DLSPM_BUILD_CUT_PLAN;
        plan->bytes = dlspm_row_plan_bytes_for(op, M, N_or_D);
        plan->hints = DLSPM_HINT_CUT_PLAN;
        if (plan->bytes > 0) return DLSPM_OK;
    }
    if (planned >= 1) {
        plan->build = DLSPM_BUILD_ROW_PLAN;
        plan->bytes = dlspm_row_plan_bytes(M);
        plan->hints = DLSPM_HINT_ROW_PLAN;
        // (the plan serves SDDMM and the fused op at these heights only with the word that the rows are very uneven)
        if (op != DLSPM_OP_SPMM && (double)longest * M >= 20.0 * (double)nnz) plan->hints |= DLSPM_HINT_ROWS_SKEWED;
        return DLSPM_OK;
    }
    // 3. schedule memory (column slices, flat schedule), the even-rows hint, or nothing
    const int passing = dlspm_workspace_advice(op, M, K, N_or_D, nnz, longest);
    if (passing == DLSPM_PASS_WORKSPACE) plan->bytes = dlspm_workspace_bytes(op, M, K, N_or_D, nnz);
    else if (passing == DLSPM_PASS_ROWS_EVEN) plan->hints = DLSPM_HINT_ROWS_EVEN;
    // long rows that lie next to each other (one eighth of the rows holds 1.6 times its share, the longest row eight
    // times the mean): the word that keeps the size rule from putting sixteen of them into one workgroup
    else if (passing == DLSPM_PASS_NULL && info->eighths_nnz_permille >= kClusteredEighthPermille && (double)longest * M >= 8.0 * (double)nnz)
        plan->hints = DLSPM_HINT_ROWS_SKEWED;
    return DLSPM_OK;
}

}  // extern "C"
