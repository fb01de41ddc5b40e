// C ABI of libdlspm_hip: argument validation, launch-shape selection and the device-side CSR check.
// The entry points and what each one replaces in the reference are documented in include/dlspm_hip.h.
#include "../../include/dlspm_hip.h"

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <algorithm>
#include <cstdlib>
#include <mutex>
#include <vector>
#include <cstring>

#include "common.hpp"
#include "launch.hpp"

namespace dlspm {

static thread_local int t_last_hip_error = 0;

static int fail_hip(hipError_t e)
{
    t_last_hip_error = (int)e;
    return DLSPM_E_LAUNCH;
}


// Optional launch-shape override for tuning sweeps: DLSPM_SPLIT="W,R", read at every call.
static bool split_override(int& W, int& R)
{
    const char* e = std::getenv("DLSPM_SPLIT");
    int w = 0, r = 0;
    if (e && std::sscanf(e, "%d,%d", &w, &r) == 2) {
        W = w;
        R = r;
        return true;
    }
    return false;
}

// Flat schedule (every wave owns a fixed number of consecutive nonzeros; partial rows in the caller's workspace):
// chosen when the matrix is large enough that the second launch does not matter, its rows are long enough that a wave
// walks few of them in sequence, and a dense row is wide enough to keep a whole wave or half of one busy. Measured on
// MI355X against the workgroup-per-row-block schedule (SpMM and fused, 0.5-27 M nonzeros, widths 128 and 256): 5-40 %
// slower on even row lengths (most below 2 M nonzeros), 10-60 % faster on lognormal row lengths (sigma 1-2); below
// these sizes it loses even there (short rows cost a wave one dependent memory round trip each). Passing the
// workspace is therefore the caller's way of saying that the rows are uneven (dlspm_csr_row_stats tells).
// DLSPM_FLAT=0/1 overrides the rule and DLSPM_FLAT_CHUNK the nonzeros per wave, for tuning sweeps and tests.
constexpr int kFlatMinNnz = 1 << 19;
constexpr int kFlatMinRow = 64;          // mean nonzeros per row
constexpr int kFlatMinLanes = 32;        // lanes per dense row (widths above 64 floats)
constexpr int kFlatTargetUnits = 32768;  // waves wanted at least: four rounds of 8 waves on each of 1024 SIMDs
// SDDMM takes the flat schedule by this rule alone (it needs no workspace, so the caller has no say): only where it
// was measured to be equal on even rows
constexpr int kFlatMinNnzSddmm = 1 << 21;
constexpr int kFlatMinRowSddmm = 256;

FlatPlan flat_plan(int M, int nnz, int width, int G)
{
    FlatPlan p{0, 0, 0};
    if (M <= 0 || nnz <= 0 || width <= 0) return p;
    int force = -1;
    if (const char* e = std::getenv("DLSPM_FLAT")) force = std::atoi(e);
    const bool by_rule = nnz >= kFlatMinNnz && (long long)nnz >= (long long)kFlatMinRow * M && G >= kFlatMinLanes;
    if (force == 0 || (force < 0 && !by_rule)) return p;
    long long chunk = nnz >= (1 << 21) ? 512 : 256;  // at least eight (four) passes of 64 nonzeros per wave
    const long long even = ((long long)nnz + kFlatTargetUnits - 1) / kFlatTargetUnits;
    if (even > chunk) chunk = (even + 63) / 64 * 64;
    if (const char* e = std::getenv("DLSPM_FLAT_CHUNK")) {
        const int c = std::atoi(e);
        if (c >= 64) chunk = c;
    }
    p.chunk = (int)chunk;
    p.units = (int)(((long long)nnz + chunk - 1) / chunk);
    p.bytes = (size_t)p.units * 2 * (size_t)width * sizeof(float);
    return p;
}

static FlatPlan sddmm_flat_plan(int M, int nnz, int D)
{
    int force = -1;
    if (const char* e = std::getenv("DLSPM_FLAT")) force = std::atoi(e);
    if (force < 0 && (nnz < kFlatMinNnzSddmm || (long long)nnz < (long long)kFlatMinRowSddmm * M)) return FlatPlan{0, 0, 0};
    return flat_plan(M, nnz, D, kWave);
}

// Column-sliced schedule (the device works through the column ranges of the sparse matrix one after the other, partial
// rows in the caller's workspace): chosen when the dense operands gathered per nonzero are together larger than one
// XCD's 4 MiB L2; the slices are cut to 2 MiB of them (8/3 MiB with partial rows). Measured on MI355X (8192 x 8192, 30 % dense, lognormal rows,
// sigma 0.6; row-block / flat / sliced): fused, D = 128 (8 MiB of Kmat and V): 1429 / 1374 / 676 us, D = 256 (16 MiB):
// 4024 / 3946 / 1328 us; SpMM, N = 256: 1472 / 1390 / 685 us; slices of 4 MiB instead: 769, 1441, 803 us. SpMM and
// the fused op write a partial row per row and slice, and slices of 8/3 MiB instead of 2 MiB are 3 % faster for them in
// the geometric mean of 24 cases (0.88 ... 1.09; most on a tall B under wide dense rows); SDDMM has no partial rows and
// gains nothing from larger slices (0.92 ... 1.04, mean 1.00). Operands of
// exactly 4 MiB (8192 x 128 floats) gain 13-16 % at 10-30 % density and lose 5 % at 3 %: sliced in two for long rows
// only. Like the flat schedule only from half a million nonzeros on (two more launches). DLSPM_SLICES=0 switches it
// off, DLSPM_SLICES=n forces n slices (tuning, tests).
constexpr long long kSliceMinOperand = 4ll << 20;  // bytes gathered from; above this the operand is sliced
constexpr long long kSlicesPer8MiB = 4;            // slices of 2 MiB of it: half the L2 each
constexpr long long kSlicesPer8MiBPartial = 3;     // ... of 8/3 MiB where every slice costs a partial row per row
constexpr int kSliceMaxSlices = 16;
constexpr int kSliceMinRow = 16;  // least mean nonzeros of a row inside one slice; fewer slices rather than shorter shares
constexpr int kSliceMinRowAtL2 = 256;  // the same for an operand of exactly kSliceMinOperand bytes

SlicePlan slice_plan(int M, int K, int width, int nnz, int operands, int partial_width, int G, bool partial_rows,
                     int slots, int min_blocks)
{
    SlicePlan p{0, 1, 0, 0};
    if (M <= 0 || K <= 0 || nnz <= 0 || width <= 0 || G <= 0) return p;  // G == 0: no sliced kernel for this layout
    int force = -1;
    if (const char* e = std::getenv("DLSPM_SLICES")) force = std::atoi(e);
    const long long bytes = (long long)K * width * (long long)sizeof(float) * operands;
    long long slices = (bytes * (partial_rows ? kSlicesPer8MiBPartial : kSlicesPer8MiB) + (8ll << 20) - 1) / (8ll << 20);
    if (slices > kSliceMaxSlices) slices = kSliceMaxSlices;
    // Slices that leave a row its minimum share: 16 nonzeros per slice for dense rows of 256 floats and more, in
    // inverse proportion more for narrower ones (measured with D = 64: 28 per slice lost 20 %, 48 and more gained; with
    // D = 32: 48 lost, 164 gained). An operand that just fills the L2 is worth slicing for long rows only, and only
    // for dense rows of at least 128 floats (narrower: 327 nonzeros per slice still lost 10 %).
    const bool just_fills = bytes <= kSliceMinOperand;
    const int per_width = 4096 / width;
    const int min_row = just_fills ? kSliceMinRowAtL2 : per_width > kSliceMinRow ? per_width : kSliceMinRow;
    if (just_fills && width < 128) slices = 0;
    const long long fit = (long long)nnz / ((long long)min_row * M);
    if (slices > fit) slices = fit;
    const bool by_rule = bytes >= kSliceMinOperand && nnz >= kSlicedMinNnz && slices >= 2;
    if (force == 0 || force == 1 || (force < 0 && !by_rule)) return p;
    if (force >= 2) slices = force < kSliceMaxSlices ? force : kSliceMaxSlices;
    if (slices > K) slices = K;
    if (slices < 2) return p;
    p.slices = (int)slices;
    int W = 4;
    choose_split(M, 1, (int)(nnz / slices), SplitRule{min_blocks, 4, slots, false}, false, W, p.R);
    if (W != 4) p.R = 1;  // only four-wave workgroups are built for this schedule
    p.bounds_bytes = (((size_t)(slices + 1) * M * sizeof(int)) + 255) / 256 * 256;
    p.bytes = p.bounds_bytes + (size_t)slices * M * (size_t)partial_width * sizeof(float);
    return p;
}

void choose_split(int M, long long col_tiles, int nnz, const SplitRule& rule, bool rows_even, int& W, int& R)
{
    static const int kPairs[][2] = {{4, 16}, {4, 8}, {4, 4}, {4, 2}, {4, 1}, {8, 4}, {8, 2}, {8, 1}, {16, 1}};
    if (split_override(W, R)) {
        for (const auto& pr : kPairs)
            if (pr[0] == W && pr[1] == R && W <= rule.max_w) return;
    }
    // Measured on MI355X over the benchmark configurations and the 12 x {32,128} x {0.3,0.2,0.1} sweep grid:
    // four-wave workgroups win whenever the matrix has enough rows to fill the device (16-wave workgroups were up
    // to 2x slower on long rows: their barrier makes every wave wait for the slowest of sixteen), and rows are
    // grouped only as far as the grid keeps `min_blocks` workgroups and a workgroup stays below ~512 nonzeros.
    const double avg = M > 0 ? (double)nnz / M : 0.0;
    const long long work_rows = (long long)M * col_tiles;
    W = work_rows >= 512 ? 4 : work_rows >= 256 ? 8 : 16;
    // very long rows in a tall matrix: sixteen waves per row gain 5-8 % in SpMM (24576 and 32768 rows of ~2000
    // nonzeros); with 8192 rows they lose as much, and the fused kernel loses 25-50 % with them at any height
    if (rule.w16_long_rows && avg >= 1536.0 && work_rows >= 16384) W = 16;
    // few rows, each long (pruned ResNet-50 layers at small batch): four waves per row leave the device with a
    // couple of waves per SIMD, each walking hundreds of steps in sequence (measured 15-25 % slower); a step
    // takes `slots` nonzeros of the row at once
    const double steps = avg / (rule.slots > 0 ? rule.slots : 1);
    if (work_rows < 1024 && steps >= 768.0) W = 16;
    else if (work_rows < 1024 && steps >= 384.0 && W < 8) W = 8;
    if (W > rule.max_w) W = rule.max_w;
    R = 1;
    if (W == 4) {
        for (int r = 2; r <= 16; r *= 2) {
            const long long blocks = (long long)((M + r - 1) / r) * col_tiles;
            if (blocks < rule.min_blocks || avg * r > 512.0) break;
            R = r;
        }
        // Rows known to be even: four rows per four-wave workgroup, which the kernels then run as one whole row per
        // wave (no partial sums, no barrier, one chain of accesses per row instead of four): 3-17 % faster than one
        // row per workgroup from 2048 rows on, and 1.3-1.7x where the gathered operands exceed one L2 (8192 x 128
        // floats twice in the fused op), because waves that start together then sweep the columns together. With
        // uneven rows the same grouping is 5-20 % slower (four rows of work per workgroup make the tail of the
        // launch coarser), hence only on the caller's word. Rows below 128 nonzeros keep the grouping of the size rule
        // (4096 rows of ~100: four per workgroup measured 6 % slower than two).
        if (rows_even && R < 4 && avg >= 128.0 && (long long)((M + 3) / 4) * col_tiles >= 512) R = 4;
    }
}

// longest row and number of rows without nonzeros (dlspm_csr_row_stats); stats[0] = max, stats[1] = empty rows
__global__ void row_stats_kernel(int M, const int* __restrict__ row_offsets, int* __restrict__ stats)
{
    int longest = 0, empty = 0;
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < M; i += gridDim.x * blockDim.x) {
        const int len = row_offsets[i + 1] - row_offsets[i];
        longest = max(longest, len);
        empty += len == 0 ? 1 : 0;
    }
    if (longest > 0) atomicMax(&stats[0], longest);
    if (empty > 0) atomicAdd(&stats[1], empty);
}

// D == 0 in SDDMM: every dot product is the empty sum (a kernel, not a memset, so that callers may capture the call)
__global__ void fill_zero_kernel(float* __restrict__ out, int n)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = 0.f;
}

// ---- device-side CSR check ------------------------------------------------------------------------
// flag bits: 1 nnz > M*K | 2 row_offsets[M] != nnz | 4 offsets decrease | 8 row longer than K
//            16 column >= K | 32 row_offsets[0] != 0 | 64 negative column
__global__ void csr_check_kernel(int M, int K, int nnz, const int* __restrict__ row_offsets,
                                 const int* __restrict__ col_indices, int* __restrict__ flags)
{
    const int tid = blockIdx.x * blockDim.x + threadIdx.x;
    const int stride = gridDim.x * blockDim.x;
    int f = 0;
    if (tid == 0) {
        if (row_offsets[M] != nnz) f |= 2;
        if (row_offsets[0] != 0) f |= 32;
    }
    for (int i = tid; i < M; i += stride) {
        const int lo = row_offsets[i], hi = row_offsets[i + 1];
        if (hi < lo) f |= 4;
        if (hi - lo > K) f |= 8;
    }
    if (!(f & 2)) {
        for (int i = tid; i < nnz; i += stride) {
            const int c = col_indices[i];
            if (c >= K) f |= 16;
            if (c < 0) f |= 64;
        }
    }
    if (f) atomicOr(flags, f);
}

// the sliced plan of each op, from its lane layout (0 slices: not used)
static SlicePlan spmm_slice_plan(int M, int K, int N, int nnz, const SpmmShape& s)
{
    const int tw = s.G * s.vec * s.V;
    // the column tiles are worked through one after the other: one tile's slab of B is what is gathered from at a time
    // and the workgroups of one (slice, tile) pair should fill the device by themselves, or it gathers from several
    // slabs at once: rows per workgroup as if there were one tile (4096 x 65536, N = 3136, 25 tiles of 128, 131 or
    // 656 nonzeros per row: 856 -> 716 us and 2320 -> 2133 us)
    SlicePlan p = slice_plan(M, K, N < tw ? N : tw, nnz, 1, 0, s.vec == 4 ? s.G : 0, true, kWave / s.G, 2048);
    p.bytes = p.slices > 0 ? p.bounds_bytes + (size_t)p.slices * M * (size_t)N * sizeof(float) : 0;
    return p;
}
static SlicePlan fused_slice_plan(int M, int K, int D, int nnz, const FusedShape& s)
{
    const int tw = s.G * s.vec * s.V;
    const bool built = s.vec == 4 && s.G1 == 8 && s.DS > 0 && tw >= D;  // the widths the sliced kernels are built for (17 .. 512)
    return slice_plan(M, K, D, nnz, 2, D, built ? s.G : 0, true, kWave / s.G, 512);
}
static SlicePlan sddmm_slice_plan(int M, int K, int D, int nnz, const SddmmShape& s)
{
    const bool built = s.vec == 4 && s.G1 == 8 && s.DS >= 1;  // 16 < D <= 512
    return slice_plan(M, K, D, nnz, 1, 0, built ? kWave : 0, false, kWave / s.G1, 512);
}

}  // namespace dlspm

using namespace dlspm;

extern "C" {

int spmm_csr_f32(int M, int K, int N, int nnz, const int* row_offsets, const int* col_indices, const float* values,
                 const float* B, float* C, void* workspace, size_t workspace_bytes, void* stream)
{
    if (M < 0 || K < 0 || N < 0 || nnz < 0) return DLSPM_E_INVALID_ARG;
    if ((long long)nnz > (long long)M * K) return DLSPM_E_INVALID_ARG;
    if (M == 0 || N == 0) return DLSPM_OK;
    if (!row_offsets || !C) return DLSPM_E_INVALID_ARG;
    if (nnz > 0 && (!col_indices || !values || !B)) return DLSPM_E_INVALID_ARG;
    const bool vec4 = N >= 4;  // dwordx4 accesses need only dword alignment
    const SpmmArgs args{M, K, N, nnz, row_offsets, col_indices, values, B, C};
    const bool even = workspace == DLSPM_ROWS_EVEN;  // a constant that says something about the rows, not memory
    const bool memory = !even && workspace != nullptr && workspace_bytes > 0;
    const SpmmShape shape = spmm_choose(M, K, N, nnz, vec4, even, !memory);
    hipError_t e;
    if (memory) {
        const SlicePlan sliced = spmm_slice_plan(M, K, N, nnz, shape);
        const FlatPlan plan = sliced.slices > 0 ? FlatPlan{0, 0, 0} : flat_plan(M, nnz, N, shape.G);
        if (workspace_bytes < (sliced.slices > 0 ? sliced.bytes : plan.bytes)) return DLSPM_E_WORKSPACE;
        if (sliced.slices > 0)
            e = spmm_sliced_launch(args, shape, sliced, workspace, static_cast<hipStream_t>(stream));
        else if (plan.chunk > 0)
            e = spmm_flat_launch(args, shape, plan, static_cast<float*>(workspace), static_cast<hipStream_t>(stream));
        else
            e = spmm_launch(args, shape, static_cast<hipStream_t>(stream));
    } else {
        e = spmm_launch(args, shape, static_cast<hipStream_t>(stream));
    }
    return e == hipSuccess ? DLSPM_OK : fail_hip(e);
}

// ---- the entry point that allocates nothing --------------------------------------------------------------------
// Scratch memory of spmm_csr_f32_static: one array per GPU, part of the loaded code object, held until the process ends.
// `scratch` is the host-side handle of that array, not a device address: the address on the current device comes
// from hipGetSymbolAddress, once per device, and only that address is ever handed to a kernel.
constexpr size_t kStaticScratchBytes = (size_t)8 << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};

// address of `scratch` on the current device (looked up at the first call on that device), or nullptr with `e` set
void* static_scratch(hipError_t& e)
{
    int dev = -1;
    e = hipGetDevice(&dev);
    if (e != hipSuccess) return nullptr;
    if (dev < 0 || dev >= kMaxDevices) {
        e = hipErrorInvalidDevice;
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return nullptr;
        g_scratch_ptr[dev] = ptr;
    }
    return g_scratch_ptr[dev];
}
}  // namespace

size_t dlspm_static_scratch_bytes(void) { return kStaticScratchBytes; }

int spmm_csr_f32_static(int M, int K, int N, int nnz, const int* row_offsets, const int* col_indices, const float* values,
                        const float* B, float* C, void* stream)
{
    if (M < 0 || K < 0 || N < 0 || nnz < 0) return DLSPM_E_INVALID_ARG;
    if ((long long)nnz > (long long)M * K) return DLSPM_E_INVALID_ARG;
    const size_t need = dlspm_workspace_bytes(DLSPM_OP_SPMM, M, K, N, nnz);
    if (need > kStaticScratchBytes) return DLSPM_E_STATIC_LIMIT;
    if (need == 0)  // the schedule of these sizes keeps everything in registers and LDS
        return spmm_csr_f32(M, K, N, nnz, row_offsets, col_indices, values, B, C, nullptr, 0, stream);
    hipError_t e = hipSuccess;
    void* ptr = static_scratch(e);
    if (!ptr) return fail_hip(e);
    return spmm_csr_f32(M, K, N, nnz, row_offsets, col_indices, values, B, C, ptr, kStaticScratchBytes, stream);
}

size_t dlspm_row_plan_bytes(int M) { return M > 0 ? (size_t)3 * (size_t)M * sizeof(int) : 0; }

int dlspm_row_plan_build(int M, const int* row_offsets, void* plan, size_t plan_bytes, void* stream)
{
    if (M < 0) return DLSPM_E_INVALID_ARG;
    if (M == 0) return DLSPM_OK;
    if (!row_offsets || !plan) return DLSPM_E_INVALID_ARG;
    if (plan_bytes < dlspm_row_plan_bytes(M)) return DLSPM_E_WORKSPACE;
    hipStream_t st = static_cast<hipStream_t>(stream);
    std::vector<int> ro((size_t)M + 1);
    hipError_t e = hipMemcpyAsync(ro.data(), row_offsets, ro.size() * sizeof(int), hipMemcpyDeviceToHost, st);
    if (e == hipSuccess) e = hipStreamSynchronize(st);
    if (e != hipSuccess) return fail_hip(e);
    // Longest rows first: workgroups are dispatched in index order, so the rows that take longest start first and the
    // short ones fill the gaps as compute units free up. The first kResident workgroups all start at once (eight
    // four-wave workgroups on each of 256 compute units) and workgroup i of them runs on compute unit i mod 256, so
    // those rows are packed into 256 bins of equal size, longest row first into the least loaded bin that has
    // room, and bin b becomes the workgroups b, b + 256, b + 512, ... A compute unit's rows then add up to about
    // the same number of nonzeros (2048 x 512, lognormal rows, N = 256: 7.6 us in matrix order, 7.2 us longest first,
    // 7.0 us with the groups of 256 alternating between descending and ascending length, 6.1 us packed; bins of 8,
    // one per XCD, do nothing: 7.2 us). DLSPM_PLAN_ORDER=1|2 gives the alternating and the plain descending order.
    constexpr int kBins = 256, kResident = 2048;
    std::vector<int> order((size_t)M);
    for (int i = 0; i < M; ++i) order[i] = i;
    auto len = [&](int i) { return ro[(size_t)i + 1] - ro[i]; };
    std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return len(a) > len(b); });
    const int head = M < kResident ? M : kResident;
    int variant = 0;
    if (const char* e = std::getenv("DLSPM_PLAN_ORDER")) variant = std::atoi(e);
    if (variant == 1) {
        for (int g = kBins; g < head; g += 2 * kBins) std::reverse(order.begin() + g, order.begin() + (g + kBins < head ? g + kBins : head));
    } else if (variant != 2) {
        const int cap = (head + kBins - 1) / kBins;
        std::vector<long long> load(kBins, 0);
        std::vector<int> cnt(kBins, 0), placed((size_t)head, -1);
        for (int i = 0; i < head; ++i) {
            int best = -1;  // a bin's next workgroup must exist: the last round of bins may be a partial one
            for (int b = 0; b < kBins; ++b)
                if (cnt[b] < cap && cnt[b] * kBins + b < head && (best < 0 || load[b] < load[best])) best = b;
            placed[(size_t)cnt[best] * kBins + best] = order[i];
            load[best] += len(order[i]);
            ++cnt[best];
        }
        for (int i = 0; i < head; ++i) order[i] = placed[i];
    }
    std::vector<int> host((size_t)3 * M);
    for (int i = 0; i < M; ++i) {
        host[i] = ro[order[i]];
        host[(size_t)M + i] = ro[(size_t)order[i] + 1];
        host[2 * (size_t)M + i] = order[i];
    }
    e = hipMemcpyAsync(plan, host.data(), host.size() * sizeof(int), hipMemcpyHostToDevice, st);
    if (e == hipSuccess) e = hipStreamSynchronize(st);
    return e == hipSuccess ? DLSPM_OK : fail_hip(e);
}

int dlspm_row_plan_advice(int op, int M, int K, int N_or_D, int nnz, int max_row_len)
{
    if (M <= 0 || K <= 0 || N_or_D <= 0 || nnz <= 0) return 0;
    const bool vec4 = N_or_D >= 4;
    if (op == DLSPM_OP_SPMM) {
        SpmmShape shape = spmm_choose(M, K, N_or_D, nnz, vec4, false, true);
        if (!spmm_plan_applies(shape, M, N_or_D, nnz)) return 0;
    } else if (op == DLSPM_OP_SDDMM) {
        SddmmShape shape = sddmm_choose(M, N_or_D, nnz, vec4);
        if (!sddmm_plan_applies(shape, M, N_or_D, nnz)) return 0;
    } else if (op == DLSPM_OP_FUSED) {
        FusedShape shape = fused_choose(M, N_or_D, nnz, vec4);
        if (!fused_plan_applies(shape, M, N_or_D, nnz)) return 0;
    } else {
        return 0;
    }
    // rows known to be even gain nothing from another order (and DLSPM_ROWS_EVEN may serve them better)
    if (max_row_len >= 0 && max_row_len <= 1.5 * ((double)nnz / M)) return 0;
    // dense operands well beyond one L2 need the column-sliced schedule's workspace more than they need balance; the
    // flat schedule, though, is behind the plan wherever both apply (SpMM, lognormal rows, sigma 1 ... 2, row-block /
    // flat / plan: 8192 x 2048, N = 128: 45.4 / 41.2 / 30.8 us; 16384 x 4096: 121 / 105 / 86.6 us; 32768 x 8192: 525 / 466
    // / 424 us)
    int slices = 0;
    (void)dlspm_describe_slices(op, M, K, N_or_D, nnz, &slices, nullptr);
    return slices >= 3 ? 0 : 1;
}

int spmm_csr_f32_planned(int M, int K, int N, int nnz, const int* row_offsets, const int* col_indices,
                         const float* values, const float* B, float* C, const void* plan, size_t plan_bytes,
                         void* stream)
{
    if (M < 0 || K < 0 || N < 0 || nnz < 0) return DLSPM_E_INVALID_ARG;
    if ((long long)nnz > (long long)M * K) return DLSPM_E_INVALID_ARG;
    if (!plan) return spmm_csr_f32(M, K, N, nnz, row_offsets, col_indices, values, B, C, nullptr, 0, stream);
    if (plan_bytes < dlspm_row_plan_bytes(M)) return DLSPM_E_WORKSPACE;
    if (M == 0 || N == 0) return DLSPM_OK;
    if (!row_offsets || !C) return DLSPM_E_INVALID_ARG;
    if (nnz > 0 && (!col_indices || !values || !B)) return DLSPM_E_INVALID_ARG;
    SpmmShape shape = spmm_choose(M, K, N, nnz, N >= 4, false, true);
    if (!spmm_plan_applies(shape, M, N, nnz))  // short rows grouped per workgroup, or column tiles: the plan has no say
        return spmm_csr_f32(M, K, N, nnz, row_offsets, col_indices, values, B, C, nullptr, 0, stream);
    const SpmmArgs args{M, K, N, nnz, row_offsets, col_indices, values, B, C};
    const hipError_t e = spmm_planned_launch(args, shape, static_cast<const int*>(plan), static_cast<hipStream_t>(stream));
    return e == hipSuccess ? DLSPM_OK : fail_hip(e);
}

int sddmm_csr_f32_planned(int M, int K, int D, int nnz, const int* row_offsets, const int* col_indices, const float* lhs,
                          const float* rhs, float* out_values, const void* plan, size_t plan_bytes, void* stream)
{
    if (M < 0 || K < 0 || D < 0 || nnz < 0) return DLSPM_E_INVALID_ARG;
    if ((long long)nnz > (long long)M * K) return DLSPM_E_INVALID_ARG;
    if (!plan) return sddmm_csr_f32(M, K, D, nnz, row_offsets, col_indices, lhs, rhs, out_values, nullptr, 0, stream);
    if (plan_bytes < dlspm_row_plan_bytes(M)) return DLSPM_E_WORKSPACE;
    if (M == 0 || nnz == 0) return DLSPM_OK;
    if (!row_offsets || !col_indices || !out_values) return DLSPM_E_INVALID_ARG;
    if (D > 0 && (!lhs || !rhs)) return DLSPM_E_INVALID_ARG;
    SddmmShape shape = sddmm_choose(M, D, nnz, D >= 4);
    if (D == 0 || !sddmm_plan_applies(shape, M, D, nnz))
        return sddmm_csr_f32(M, K, D, nnz, row_offsets, col_indices, lhs, rhs, out_values, nullptr, 0, stream);
    const SddmmArgs args{M, K, D, nnz, row_offsets, col_indices, lhs, rhs, out_values};
    const hipError_t e = sddmm_planned_launch(args, shape, static_cast<const int*>(plan), static_cast<hipStream_t>(stream));
    return e == hipSuccess ? DLSPM_OK : fail_hip(e);
}

int fused_sddmm_spmm_f32_planned(int M, int K, int D, int nnz, const int* row_offsets, const int* col_indices, const float* Q,
                                 const float* Kmat, const float* V, float scale, float* O, const void* plan,
                                 size_t plan_bytes, void* stream)
{
    if (M < 0 || K < 0 || D < 0 || nnz < 0) return DLSPM_E_INVALID_ARG;
    if ((long long)nnz > (long long)M * K) return DLSPM_E_INVALID_ARG;
    if (!plan) return fused_sddmm_spmm_f32(M, K, D, nnz, row_offsets, col_indices, Q, Kmat, V, scale, O, nullptr, 0, stream);
    if (plan_bytes < dlspm_row_plan_bytes(M)) return DLSPM_E_WORKSPACE;
    if (M == 0 || D == 0) return DLSPM_OK;
    if (!row_offsets || !O) return DLSPM_E_INVALID_ARG;
    if (nnz > 0 && (!col_indices || !Q || !Kmat || !V)) return DLSPM_E_INVALID_ARG;
    FusedShape shape = fused_choose(M, D, nnz, D >= 4);
    if (!fused_plan_applies(shape, M, D, nnz))
        return fused_sddmm_spmm_f32(M, K, D, nnz, row_offsets, col_indices, Q, Kmat, V, scale, O, nullptr, 0, stream);
    const FusedArgs args{M, K, D, nnz, row_offsets, col_indices, Q, Kmat, V, scale, O};
    const hipError_t e = fused_planned_launch(args, shape, static_cast<const int*>(plan), static_cast<hipStream_t>(stream));
    return e == hipSuccess ? DLSPM_OK : fail_hip(e);
}

int sddmm_csr_f32(int M, int K, int D, int nnz, const int* row_offsets, const int* col_indices, const float* lhs,
                  const float* rhs, float* out_values, void* workspace, size_t workspace_bytes, void* stream)
{
    if (M < 0 || K < 0 || D < 0 || nnz < 0) return DLSPM_E_INVALID_ARG;
    if ((long long)nnz > (long long)M * K) return DLSPM_E_INVALID_ARG;
    if (M == 0 || nnz == 0) return DLSPM_OK;
    if (!row_offsets || !col_indices || !out_values) return DLSPM_E_INVALID_ARG;
    if (D > 0 && (!lhs || !rhs)) return DLSPM_E_INVALID_ARG;
    if (D == 0) {
        const unsigned blocks = (unsigned)((nnz + 255) / 256);
        hipLaunchKernelGGL(fill_zero_kernel, dim3(blocks), dim3(256), 0, static_cast<hipStream_t>(stream), out_values, nnz);
        const hipError_t e0 = hipGetLastError();
        return e0 == hipSuccess ? DLSPM_OK : fail_hip(e0);
    }
    const bool vec4 = D >= 4;  // dwordx4 accesses need only dword alignment
    const SddmmShape shape = sddmm_choose(M, D, nnz, vec4, workspace == DLSPM_ROWS_EVEN);
    const SddmmArgs args{M, K, D, nnz, row_offsets, col_indices, lhs, rhs, out_values};
    // the flat schedule needs no workspace here (nothing to combine), so the size rule alone decides; it has no
    // width condition for SDDMM (measured for D = 32 ... 256: equal on uniform rows, 15-33 % faster on skewed ones)
    if (workspace != nullptr && workspace != DLSPM_ROWS_EVEN && workspace_bytes > 0) {
        // with a workspace for the slice boundaries: the column-sliced schedule where the rhs operand exceeds one L2
        const SlicePlan sliced = sddmm_slice_plan(M, K, D, nnz, shape);
        if (workspace_bytes < sliced.bytes) return DLSPM_E_WORKSPACE;
        if (sliced.slices > 0) {
            const hipError_t es = sddmm_sliced_launch(args, shape, sliced, workspace, static_cast<hipStream_t>(stream));
            return es == hipSuccess ? DLSPM_OK : fail_hip(es);
        }
    }
    const FlatPlan plan = sddmm_flat_plan(M, nnz, D);
    const hipError_t e = plan.chunk > 0 ? sddmm_flat_launch(args, shape, plan.chunk, static_cast<hipStream_t>(stream))
                                        : sddmm_launch(args, shape, static_cast<hipStream_t>(stream));
    return e == hipSuccess ? DLSPM_OK : fail_hip(e);
}

int fused_sddmm_spmm_f32(int M, int K, int D, int nnz, const int* row_offsets, const int* col_indices, const float* Q,
                         const float* Kmat, const float* V, float scale, float* O, void* workspace,
                         size_t workspace_bytes, void* stream)
{
    if (M < 0 || K < 0 || D < 0 || nnz < 0) return DLSPM_E_INVALID_ARG;
    if ((long long)nnz > (long long)M * K) return DLSPM_E_INVALID_ARG;
    if (M == 0 || D == 0) return DLSPM_OK;
    if (!row_offsets || !O) return DLSPM_E_INVALID_ARG;
    if (nnz > 0 && (!col_indices || !Q || !Kmat || !V)) return DLSPM_E_INVALID_ARG;
    const bool vec4 = D >= 4;
    const bool even = workspace == DLSPM_ROWS_EVEN;
    const FusedShape shape = fused_choose(M, D, nnz, vec4, even);
    const FusedArgs args{M, K, D, nnz, row_offsets, col_indices, Q, Kmat, V, scale, O};
    hipError_t e;
    if (!even && workspace != nullptr && workspace_bytes > 0) {
        const SlicePlan sliced = fused_slice_plan(M, K, D, nnz, shape);
        const FlatPlan plan = sliced.slices > 0 ? FlatPlan{0, 0, 0} : flat_plan(M, nnz, D, shape.G);
        if (workspace_bytes < (sliced.slices > 0 ? sliced.bytes : plan.bytes)) return DLSPM_E_WORKSPACE;
        if (sliced.slices > 0)
            e = fused_sliced_launch(args, shape, sliced, workspace, static_cast<hipStream_t>(stream));
        else if (plan.chunk > 0)
            e = fused_flat_launch(args, shape, plan, static_cast<float*>(workspace), static_cast<hipStream_t>(stream));
        else
            e = fused_launch(args, shape, static_cast<hipStream_t>(stream));
    } else {
        e = fused_launch(args, shape, static_cast<hipStream_t>(stream));
    }
    return e == hipSuccess ? DLSPM_OK : fail_hip(e);
}

size_t dlspm_workspace_bytes(int op, int M, int K, int N_or_D, int nnz)
{
    // The workgroup-per-row-block schedule splits the work from row_offsets alone and keeps partial sums in LDS: no
    // scratch. Where flat_plan's rule selects the flat schedule for SpMM or the fused op, its partial rows live in the
    // workspace; a call without workspace runs the row-block schedule instead.
    if (M <= 0 || N_or_D <= 0 || nnz <= 0) return 0;
    if (op == DLSPM_OP_SPMM) {
        const SpmmShape s = spmm_choose(M, K, N_or_D, nnz, N_or_D >= 4, false, false);  // a call with memory
        const SlicePlan sliced = spmm_slice_plan(M, K, N_or_D, nnz, s);
        return sliced.slices > 0 ? sliced.bytes : flat_plan(M, nnz, N_or_D, s.G).bytes;
    }
    if (op == DLSPM_OP_FUSED) {
        const FusedShape s = fused_choose(M, N_or_D, nnz, N_or_D >= 4);
        const SlicePlan sliced = fused_slice_plan(M, K, N_or_D, nnz, s);
        return sliced.slices > 0 ? sliced.bytes : flat_plan(M, nnz, N_or_D, s.G).bytes;
    }
    if (op == DLSPM_OP_SDDMM) {  // every result goes into its own CSR slot: only the slice boundaries need memory
        const SddmmShape s = sddmm_choose(M, N_or_D, nnz, N_or_D >= 4);
        return sddmm_slice_plan(M, K, N_or_D, nnz, s).bytes;
    }
    return 0;
}

int dlspm_csr_check(int M, int K, int nnz, const int* row_offsets, const int* col_indices, void* stream)
{
    if (M < 0 || K < 0 || nnz < 0) return DLSPM_E_INVALID_ARG;
    if ((long long)nnz > (long long)M * K) return DLSPM_E_INVALID_CSR;
    if (!row_offsets) return DLSPM_E_INVALID_ARG;
    if (nnz > 0 && !col_indices) return DLSPM_E_INVALID_ARG;
    hipStream_t s = static_cast<hipStream_t>(stream);
    int* d_flags = nullptr;
    hipError_t e = hipMalloc(&d_flags, sizeof(int));
    if (e != hipSuccess) return fail_hip(e);
    int h_flags = 0;
    e = hipMemsetAsync(d_flags, 0, sizeof(int), s);
    if (e == hipSuccess) {
        const long long work = (long long)(M > nnz ? M : nnz);
        int blocks = (int)((work + 255) / 256);
        blocks = blocks < 1 ? 1 : blocks > 2048 ? 2048 : blocks;
        hipLaunchKernelGGL(csr_check_kernel, dim3(blocks), dim3(256), 0, s, M, K, nnz, row_offsets, col_indices, d_flags);
        e = hipGetLastError();
    }
    if (e == hipSuccess) e = hipMemcpyAsync(&h_flags, d_flags, sizeof(int), hipMemcpyDeviceToHost, s);
    if (e == hipSuccess) e = hipStreamSynchronize(s);
    (void)hipFree(d_flags);
    if (e != hipSuccess) return fail_hip(e);
    return h_flags == 0 ? DLSPM_OK : DLSPM_E_INVALID_CSR;
}

int dlspm_csr_row_stats(int M, const int* row_offsets, void* stream, int* max_row_len, int* empty_rows)
{
    if (M < 0 || (M > 0 && !row_offsets)) return DLSPM_E_INVALID_ARG;
    int h[2] = {0, 0};
    if (M > 0) {
        hipStream_t s = static_cast<hipStream_t>(stream);
        int* d = nullptr;
        hipError_t e = hipMalloc(&d, 2 * sizeof(int));
        if (e != hipSuccess) return fail_hip(e);
        e = hipMemsetAsync(d, 0, 2 * sizeof(int), s);
        if (e == hipSuccess) {
            int blocks = (M + 255) / 256;
            blocks = blocks > 1024 ? 1024 : blocks;
            hipLaunchKernelGGL(row_stats_kernel, dim3(blocks), dim3(256), 0, s, M, row_offsets, d);
            e = hipGetLastError();
        }
        if (e == hipSuccess) e = hipMemcpyAsync(h, d, 2 * sizeof(int), hipMemcpyDeviceToHost, s);
        if (e == hipSuccess) e = hipStreamSynchronize(s);
        (void)hipFree(d);
        if (e != hipSuccess) return fail_hip(e);
    }
    if (max_row_len) *max_row_len = h[0];
    if (empty_rows) *empty_rows = h[1];
    return DLSPM_OK;
}

int dlspm_describe_launch_rows(int op, int M, int K, int N_or_D, int nnz, int passing, int* shape)
{
    if (passing != DLSPM_PASS_NULL && passing != DLSPM_PASS_ROWS_EVEN && passing != DLSPM_PASS_WORKSPACE)
        return DLSPM_E_INVALID_ARG;
    const bool even = passing == DLSPM_PASS_ROWS_EVEN;
    const bool memory = passing == DLSPM_PASS_WORKSPACE;
    if (!shape || M < 0 || N_or_D < 0 || nnz < 0) return DLSPM_E_INVALID_ARG;
    const int n = N_or_D;
    const bool vec4 = n >= 4;
    for (int i = 0; i < 10; ++i) shape[i] = 0;
    if (op == DLSPM_OP_SPMM) {
        const SpmmShape s = spmm_choose(M, K, n, nnz, vec4, even, !memory);
        const int tw = s.G * s.vec * s.V;
        shape[0] = s.vec; shape[1] = s.G; shape[2] = s.V; shape[5] = s.W; shape[6] = s.R; shape[7] = (n + tw - 1) / tw;
        const FlatPlan fp = flat_plan(M, nnz, n, s.G);
        shape[8] = fp.chunk; shape[9] = fp.units;
    } else if (op == DLSPM_OP_SDDMM) {
        const SddmmShape s = sddmm_choose(M, n, nnz, vec4, even);
        shape[0] = s.vec; shape[3] = s.G1; shape[4] = s.DS; shape[5] = s.W; shape[6] = s.R; shape[7] = 1;
        const FlatPlan fp = sddmm_flat_plan(M, nnz, n);
        shape[8] = fp.chunk; shape[9] = fp.units;
    } else if (op == DLSPM_OP_FUSED) {
        const FusedShape s = fused_choose(M, n, nnz, vec4, even);
        const int tw = s.G * s.vec * s.V;
        shape[0] = s.vec; shape[1] = s.G; shape[2] = s.V; shape[3] = s.G1; shape[4] = s.DS; shape[5] = s.W; shape[6] = s.R;
        shape[7] = (n + tw - 1) / tw;
        const FlatPlan fp = flat_plan(M, nnz, n, s.G);
        shape[8] = fp.chunk; shape[9] = fp.units;
    } else {
        return DLSPM_E_INVALID_ARG;
    }
    return DLSPM_OK;
}

int dlspm_describe_launch(int op, int M, int K, int N_or_D, int nnz, int* shape)
{
    return dlspm_describe_launch_rows(op, M, K, N_or_D, nnz, DLSPM_PASS_NULL, shape);
}

int dlspm_workspace_advice(int op, int M, int K, int N_or_D, int nnz, int max_row_len)
{
    if (M <= 0 || K <= 0 || N_or_D <= 0 || nnz <= 0) return DLSPM_PASS_NULL;
    if (op != DLSPM_OP_SPMM && op != DLSPM_OP_SDDMM && op != DLSPM_OP_FUSED) return DLSPM_PASS_NULL;
    int slices = 0;
    (void)dlspm_describe_slices(op, M, K, N_or_D, nnz, &slices, nullptr);
    const size_t want = dlspm_workspace_bytes(op, M, K, N_or_D, nnz);
    const double mean = (double)nnz / M;
    const bool known = max_row_len >= 0;
    const bool even = known && max_row_len <= 1.5 * mean, uneven = known && max_row_len >= 4.0 * mean;
    // even rows and an operand that only just exceeds the L2 (two slices): one whole row per wave does as well or better
    // (measured: SpMM and fused 5-9 % faster at exactly 4 MiB, equal at 8 MiB; SDDMM 2-12 % slower)
    bool sliced = slices > 0 && !(even && slices <= 2 && op != DLSPM_OP_SDDMM);
    // SpMM on rows below ~128 nonzeros: a call without memory that works in narrower column tiles is faster than the
    // slices (8192 x 32768, N = 256: 51 against 66 us at 70 per row, equal at 140, 157 against 139 us at 328;
    // 32768 x 32768, N = 256: 228 against 282 us at 128; 16384 x 32768, N = 1024: 418 against 459 us at 70,
    // 788 against 590 us at 140)
    if (sliced && op == DLSPM_OP_SPMM && mean < 128.0) {
        const SpmmShape without = spmm_choose(M, K, N_or_D, nnz, N_or_D >= 4, false, true);
        const SpmmShape with = spmm_choose(M, K, N_or_D, nnz, N_or_D >= 4, false, false);
        if (without.tile_major && without.G * without.V < with.G * with.V) sliced = false;
    }
    if (sliced || (uneven && want > 0 && slices == 0)) return DLSPM_PASS_WORKSPACE;
    return even ? DLSPM_PASS_ROWS_EVEN : DLSPM_PASS_NULL;
}

int dlspm_describe_slices(int op, int M, int K, int N_or_D, int nnz, int* slices, int* rows_per_workgroup)
{
    if (M < 0 || K < 0 || N_or_D < 0 || nnz < 0) return DLSPM_E_INVALID_ARG;
    SlicePlan p{0, 1, 0, 0};
    if (op == DLSPM_OP_SPMM) p = spmm_slice_plan(M, K, N_or_D, nnz, spmm_choose(M, K, N_or_D, nnz, N_or_D >= 4, false, false));
    else if (op == DLSPM_OP_FUSED) p = fused_slice_plan(M, K, N_or_D, nnz, fused_choose(M, N_or_D, nnz, N_or_D >= 4));
    else if (op == DLSPM_OP_SDDMM) p = sddmm_slice_plan(M, K, N_or_D, nnz, sddmm_choose(M, N_or_D, nnz, N_or_D >= 4));
    else return DLSPM_E_INVALID_ARG;
    if (slices) *slices = p.slices;
    if (rows_per_workgroup) *rows_per_workgroup = p.R;
    return DLSPM_OK;
}

const char* dlspm_status_string(int status)
{
    switch (status) {
        case DLSPM_OK: return "ok";
        case DLSPM_E_INVALID_ARG: return "invalid argument (negative size, NULL operand, or nnz larger than M*K)";
        case DLSPM_E_WORKSPACE: return "workspace smaller than dlspm_workspace_bytes()";
        case DLSPM_E_LAUNCH: return "HIP runtime error at launch (see dlspm_last_hip_error)";
        case DLSPM_E_INVALID_CSR: return "malformed CSR structure";
        case DLSPM_E_NO_DEVICE: return "no gfx950 device is current";
        case DLSPM_E_STATIC_LIMIT: return "the problem needs more scratch memory than spmm_csr_f32_static holds (dlspm_static_scratch_bytes)";
        default: return "unknown status";
    }
}

int dlspm_last_hip_error(void) { return t_last_hip_error; }

const char* dlspm_version(void) { return "dlspm_hip 0.1 gfx950"; }

}  // extern "C"
