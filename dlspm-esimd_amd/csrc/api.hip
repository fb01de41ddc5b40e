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

int fail_hip(hipError_t e)
{
    t_last_hip_error = (int)e;
    return DLSPM_E_LAUNCH;
}


// ---- tuning overrides ------------------------------------------------------------------------------------------------
// One set per host thread (dlspm_set_tuning). A thread that never called it uses the process default, which is read
// from the environment exactly once: DLSPM_SPLIT="W,R", DLSPM_FLAT=0|1, DLSPM_FLAT_CHUNK=n, DLSPM_SLICES=0|n,
// DLSPM_TILE_MAJOR=0|1, DLSPM_TILE_WIDTH=512|..|32, DLSPM_PLAN_ORDER=0|1|2, DLSPM_XCD_CONTIGUOUS=0|1, DLSPM_STREAM_RESULTS=0|1 (so that the drivers can be swept from a
// shell without a rebuild). No launch path reads the environment.
static Tuning tuning_from_environment()
{
    Tuning t;
    auto env = [](const char* name) { return std::getenv(name); };
    if (const char* e = env("DLSPM_SPLIT")) {
        int w = 0, r = 0;
        if (std::sscanf(e, "%d,%d", &w, &r) == 2) {
            t.split_w = w;
            t.split_r = r;
        }
    }
    auto number = [&](const char* name, int& field) {
        if (const char* e = env(name)) field = std::atoi(e);
    };
    number("DLSPM_FLAT", t.flat);
    number("DLSPM_FLAT_CHUNK", t.flat_chunk);
    number("DLSPM_SLICES", t.slices);
    number("DLSPM_TILE_MAJOR", t.tile_major);
    number("DLSPM_TILE_WIDTH", t.tile_width);
    number("DLSPM_PLAN_ORDER", t.plan_order);
    number("DLSPM_XCD_CONTIGUOUS", t.xcd_contiguous);
    number("DLSPM_STREAM_RESULTS", t.stream_results);
    number("DLSPM_CUT_PIECE_PCT", t.cut_piece_pct);
    number("DLSPM_CUT_LONGEST_PCT", t.cut_longest_pct);
    number("DLSPM_RULES_OFF", t.rules_off);
    number("DLSPM_COMPUTE_UNITS", t.compute_units);
    if (t.compute_units < 8 || t.compute_units > 1024 || t.compute_units % 8 != 0) t.compute_units = 0;
    return t;
}
static const Tuning& process_tuning()
{
    static const Tuning t = tuning_from_environment();
    return t;
}
static thread_local bool t_tuning_set = false;
static thread_local Tuning t_tuning;
const Tuning& tuning() { return t_tuning_set ? t_tuning : process_tuning(); }

// ---- the current device ----------------------------------------------------------------------------------------------
constexpr int kMaxDevices = 64;
static const DeviceInfo kNoDevice{256, 4ll << 20, false, false};
static const DeviceInfo& current_device_info()
{
    static std::mutex mutex;
    static DeviceInfo cache[kMaxDevices];
    static bool known[kMaxDevices] = {};
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        (void)hipGetLastError();  // a machine without a device is not an error of the caller's next HIP call
        return kNoDevice;
    }
    // the device this thread asked about last: no lock on that path (an entry of the cache never changes once written)
    static thread_local int t_last_dev = -1;
    static thread_local const DeviceInfo* t_last_info = nullptr;
    if (dev == t_last_dev) return *t_last_info;
    std::lock_guard<std::mutex> lock(mutex);
    if (!known[dev]) {
        DeviceInfo d = kNoDevice;
        hipDeviceProp_t prop;
        if (hipGetDeviceProperties(&prop, dev) == hipSuccess) {
            d.present = true;
            d.gfx950 = std::strncmp(prop.gcnArchName, "gfx950", 6) == 0;
            if (prop.multiProcessorCount > 0) d.cus = prop.multiProcessorCount;
            // the size of ONE L2 (each XCD has its own); a figure outside 1 ... 64 MiB is not believed
            if (prop.l2CacheSize >= (1 << 20) && prop.l2CacheSize <= (64 << 20)) d.l2_bytes = prop.l2CacheSize;
        } else {
            (void)hipGetLastError();
        }
        cache[dev] = d;
        known[dev] = true;
    }
    t_last_dev = dev;
    t_last_info = &cache[dev];
    return cache[dev];
}
// (with dlspm_tuning.compute_units set: the same device with that many compute units, for this host thread)
const DeviceInfo& device_info()
{
    const DeviceInfo& real = current_device_info();
    const int cus = tuning().compute_units;
    if (cus <= 0) return real;
    static thread_local DeviceInfo t_resized;
    t_resized = real;
    t_resized.cus = cus;
    return t_resized;
}
// DLSPM_OK if the current device can run the kernels
static int require_device(const DeviceInfo& d) { return d.present && d.gfx950 ? DLSPM_OK : DLSPM_E_NO_DEVICE; }

// What the caller passed as (workspace, workspace_bytes): device memory, and the hints in the upper bits of the size.
struct WorkspaceArg {
    void* mem;
    size_t bytes;
    bool rows_even;
    bool row_plan;
    bool cut_plan;
    bool banded;
    bool skewed;
    bool bad_hint;  // a bit of the hint byte that means nothing, or a row plan of a size no plan has
};
static WorkspaceArg workspace_arg(void* workspace, size_t workspace_bytes)
{
    WorkspaceArg a{};
    a.rows_even = (workspace_bytes & DLSPM_HINT_ROWS_EVEN) != 0 || workspace == DLSPM_ROWS_EVEN;
    a.row_plan = (workspace_bytes & DLSPM_HINT_ROW_PLAN) != 0;
    a.cut_plan = (workspace_bytes & DLSPM_HINT_CUT_PLAN) != 0;
    a.banded = (workspace_bytes & DLSPM_HINT_BANDED) != 0;
    a.skewed = (workspace_bytes & DLSPM_HINT_ROWS_SKEWED) != 0;
    a.bytes = workspace_bytes & ~DLSPM_HINT_MASK;
    // A caller that passes "plenty" (SIZE_MAX) as the size of scratch memory would set every hint bit: bits without a
    // meaning are refused, and so is a plan of 2^48 bytes and more (no plan is that large; a size with stray upper bits is)
    constexpr size_t known =
        DLSPM_HINT_ROWS_EVEN | DLSPM_HINT_ROW_PLAN | DLSPM_HINT_CUT_PLAN | DLSPM_HINT_BANDED | DLSPM_HINT_ROWS_SKEWED;
    a.bad_hint = (workspace_bytes & DLSPM_HINT_MASK & ~known) != 0 || ((a.row_plan || a.cut_plan) && a.bytes >= ((size_t)1 << 48)) ||
                 (a.row_plan && a.cut_plan) || (a.rows_even && a.skewed) || (workspace == DLSPM_ROWS_EVEN && a.bytes != 0);
    a.mem = workspace == DLSPM_ROWS_EVEN ? nullptr : workspace;
    if (!a.mem || a.bytes == 0) {
        a.mem = nullptr;
        a.bytes = 0;
    }
    return a;
}

// Flat schedule (every wave owns a fixed number of consecutive nonzeros; partial rows in the caller's workspace):
// chosen when the matrix is large enough that the second launch does not matter, its rows are long enough that a wave
// walks few of them in sequence, and a dense row is wide enough to keep a whole wave or half of one busy. Measured on
// MI355X against the workgroup-per-row-block schedule (SpMM and fused, 0.5-27 M nonzeros, widths 128 and 256): 5-40 %
// slower on even row lengths (most below 2 M nonzeros), 10-60 % faster on lognormal row lengths (sigma 1-2); below
// these sizes it loses even there (short rows cost a wave one dependent memory round trip each). Passing the
// workspace is therefore the caller's way of saying that the rows are uneven (dlspm_csr_row_stats tells).
// dlspm_tuning.flat = 0/1 overrides the rule and .flat_chunk the nonzeros per wave, for tuning sweeps and tests.
constexpr int kFlatMinNnz = 1 << 19;
constexpr int kFlatMinRow = 64;          // mean nonzeros per row
constexpr int kFlatMinLanes = 32;        // lanes per dense row (widths above 64 floats)
constexpr int kFlatUnitsPerCu = 128;     // waves wanted at least: four rounds of 8 waves on each of a compute unit's 4 SIMDs
// SDDMM takes the flat schedule by this rule alone (it needs no workspace, so the caller has no say): only where it
// was measured to be equal on even rows
constexpr int kFlatMinNnzSddmm = 1 << 21;
constexpr int kFlatMinRowSddmm = 256;

FlatPlan flat_plan(const DeviceInfo& dev, int M, int nnz, int width, int G)
{
    FlatPlan p{0, 0, 0};
    if (M <= 0 || nnz <= 0 || width <= 0) return p;
    const int force = tuning().flat;
    const bool by_rule = nnz >= kFlatMinNnz && (long long)nnz >= (long long)kFlatMinRow * M && G >= kFlatMinLanes;
    if (force == 0 || (force < 0 && !by_rule)) return p;
    long long chunk = nnz >= (1 << 21) ? 512 : 256;  // at least eight (four) passes of 64 nonzeros per wave
    const long long target_units = (long long)kFlatUnitsPerCu * dev.cus;
    const long long even = ceil_div(nnz, target_units);
    if (even > chunk) chunk = (even + 63) / 64 * 64;
    if (tuning().flat_chunk >= 64) chunk = tuning().flat_chunk;
    p.chunk = (int)chunk;
    p.units = (int)(((long long)nnz + chunk - 1) / chunk);
    p.bytes = (size_t)p.units * 2 * (size_t)width * sizeof(float);
    return p;
}

// Not by itself where rhs exceeds one L2 under rows of a thousand nonzeros and more: the four waves of a row-block workgroup,
// and the workgroups of neighbouring rows, go through such rows' columns together and find each other's rows of rhs in
// the L2, where the flat schedule's waves each start somewhere else (Bernoulli rows, flat / row-block: 8192 x 8192 of 1229
// per row, D = 256 711 / 537 us, of 2458 per row 1388 / 789 us, D = 384 2704 / 1681 us; 4096 x 16384 of 3277, D = 192 811 /
// 481 us; lognormal rows lose 0-7 % by it; rows of 819: 1.01-1.03 either way; rhs of exactly one L2: 1.02-1.11).
static FlatPlan sddmm_flat_plan(const DeviceInfo& dev, int M, int K, int nnz, int D)
{
    const int force = tuning().flat;
    if (force < 0 && (nnz < kFlatMinNnzSddmm || (long long)nnz < (long long)kFlatMinRowSddmm * M)) return FlatPlan{0, 0, 0};
    if (force < 0 && (long long)K * D * (long long)sizeof(float) > dev.l2_bytes && (long long)nnz >= 1024ll * M) return FlatPlan{0, 0, 0};
    return flat_plan(dev, M, nnz, D, kWave);
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
// only. Like the flat schedule only from half a million nonzeros on (two more launches). dlspm_tuning.slices = 0
// switches it off, = n forces n slices (tuning, tests). The 4 MiB are the device's own figure for one L2
// (DeviceInfo::l2_bytes): an operand above it is sliced, in slices of half of it (two thirds with partial rows).
constexpr long long kSlicesPer2L2 = 4;             // slices of half an L2 of operand each
constexpr long long kSlicesPer2L2Partial = 3;      // ... of two thirds of an L2 where every slice costs a partial row per row
constexpr int kSliceMaxSlices = 16;
constexpr int kSliceMinRow = 16;  // least mean nonzeros of a row inside one slice; fewer slices rather than shorter shares
constexpr int kSliceMinRowAtL2 = 256;  // the same for an operand that just fills one L2

SlicePlan slice_plan(const DeviceInfo& dev, int M, int K, int width, int nnz, int operands, int partial_width, int G, bool partial_rows,
                     int slots, int blocks_per_cu)
{
    SlicePlan p{0, 1, 0, 0};
    if (M <= 0 || K <= 0 || nnz <= 0 || width <= 0 || G <= 0) return p;  // G == 0: no sliced kernel for this layout
    const int force = tuning().slices;
    const long long l2 = dev.l2_bytes;
    // (sizes no device holds are cut off at 2^50 bytes: they take the largest number of slices either way)
    const double bytes_exact = (double)K * (double)width * (double)sizeof(float) * (double)operands;
    const long long bytes = bytes_exact < (double)(1ll << 50) ? (long long)bytes_exact : (1ll << 50);
    long long slices = ceil_div(bytes * (partial_rows ? kSlicesPer2L2Partial : kSlicesPer2L2), 2 * l2);
    if (slices > kSliceMaxSlices) slices = kSliceMaxSlices;
    // Slices that leave a row its minimum share: 16 nonzeros per slice for dense rows of 256 floats and more, in
    // inverse proportion more for narrower ones (measured with D = 64: 28 per slice lost 20 %, 48 and more gained; with
    // D = 32: 48 lost, 164 gained). An operand that just fills the L2 is worth slicing for long rows only, and only
    // for dense rows of at least 128 floats (narrower: 327 nonzeros per slice still lost 10 %).
    const bool just_fills = bytes <= l2;
    const int per_width = 4096 / width;
    const int min_row = just_fills ? kSliceMinRowAtL2 : per_width > kSliceMinRow ? per_width : kSliceMinRow;
    if (just_fills && width < 128) slices = 0;
    const long long fit = (long long)nnz / ((long long)min_row * M);
    if (slices > fit) slices = fit;
    // Fewer than four rows per compute unit: one slice's share of the rows does not fill the device and the launches that
    // follow each other cost more than the cache misses they save (512 rows of ~2050 nonzeros, K = 8192 / 32768, without /
    // with slices: SpMM at N = 256 42.7 / 48.7 and 53.2 / 62.7 us, SDDMM at D = 128 23.4 / 27.8 and 29.8 / 33.9 us, fused at
    // D = 128 40.8 / 48.4 and 57.3 / 61.0 us; 1024 rows: 84.5 / 80.7 and 178.8 / 94.7 us, 40.9 / 44.8 and 114.0 / 51.9 us,
    // 86.2 / 80.8 and 169.0 / 96.7 us).
    const bool rows_fill = (long long)M >= kSlicedMinRowsPerCu * dev.cus;
    const bool by_rule = bytes >= l2 && nnz >= kSlicedMinNnz && slices >= 2 && rows_fill;
    if (force == 0 || force == 1 || (force < 0 && !by_rule)) return p;
    if (force >= 2) slices = force < kSliceMaxSlices ? force : kSliceMaxSlices;
    if (slices > K) slices = K;
    if (slices < 2) return p;
    p.slices = (int)slices;
    int W = 4;
    choose_split(dev, M, 1, (int)(nnz / slices), SplitRule{blocks_per_cu, 4, slots, false}, false, W, p.R);
    if (W != 4) p.R = 1;  // only four-wave workgroups are built for this schedule
    p.bounds_bytes = (((size_t)(slices + 1) * M * sizeof(int)) + 255) / 256 * 256;
    p.bytes = p.bounds_bytes + (size_t)slices * M * (size_t)partial_width * sizeof(float);
    return p;
}

void choose_split(const DeviceInfo& dev, int M, long long col_tiles, int nnz, const SplitRule& rule, int rows, int& W, int& R)
{
    const bool rows_even = rows == kRowsEven;
    if (tuning().split_w > 0 && split_is_built(tuning().split_w, tuning().split_r, rule.max_w)) {  // (else: ignored)
        W = tuning().split_w;
        R = tuning().split_r;
        return;
    }
    const long long cus = dev.cus;  // the thresholds below were measured on 256 compute units and scale with them
    // Measured on MI355X over the benchmark configurations and the 12 x {32,128} x {0.3,0.2,0.1} sweep grid:
    // four-wave workgroups win whenever the matrix has enough rows to fill the device (16-wave workgroups were up
    // to 2x slower on long rows: their barrier makes every wave wait for the slowest of sixteen), and rows are
    // grouped only as far as the grid keeps `blocks_per_cu` workgroups per compute unit and a workgroup stays below ~512 nonzeros.
    // Fewer rows than two per compute unit: four waves per row; SDDMM and the fused op take eight from about a hundred
    // nonzeros per row on (the reference's ResNet-50 and transformer layers of 64 ... 256 rows, 200 launches in a graph,
    // four / eight / sixteen waves: 128 x 512 with 26 per row, SpMM at N = 256 2.6 / 2.7 / 3.2 us, SDDMM 2.1 / 2.1 / 2.6 us;
    // 256 x 2304 with 208 per row: SpMM 5.4 / 5.2 / 5.5 us, SDDMM 3.8 / 3.4 / 3.9 us, fused 4.7 / 4.3 / 4.7 us; SpMM in
    // column tiles, 64 x 576 with 414 per row at N = 3136: 18.7 / 22.2 / 24.5 us): more waves than a row has passes for
    // only add to the partial sums behind the barrier.
    const double avg = M > 0 ? (double)nnz / M : 0.0;
    const long long work_rows = (long long)M * col_tiles;
    W = rule.w8_few_rows_avg > 0 && work_rows < 2 * cus && avg >= rule.w8_few_rows_avg && rule_on(kRuleEightWavesFewRows) ? 8 : 4;
    // Very long rows (SpMM only; times inside a graph, rule on / off):
    //  * in a tall matrix sixteen waves per row gain 4-13 % from 24576 rows of ~1600 nonzeros on (24576 x 8192 at density
    //    0.2, N = 128: 792 / 840 us; 32768 x 8192 at 0.3, N = 32: 475 / 551 us); at 16384 rows they gain nothing and keep
    //    the even-rows grouping from applying (N = 128: 490 / 453 us under the hint), hence from 96 rows per compute unit on;
    //  * in few rows (pruned ResNet-50 layers at small batch): four waves per row leave the device with a couple of waves
    //    per SIMD, each walking hundreds of steps in sequence (256 x 8192 at 0.5, N = 128: 23.4 / 32.3 us; 128 x 4608,
    //    N = 256: 24.1 / 34.3 us); with two rows per compute unit the same choice loses (512 x 8192 at 0.25, N = 256:
    //    45.9 / 39.9 us), hence up to one and a half. A step takes `slots` nonzeros of the row at once.
    // SDDMM is indifferent to both (within 1 %) and loses the even-rows grouping to the first (24576 x 8192 at 0.2, D = 256,
    // under the hint: 2586 / 1577 us); the fused op loses 3-17 % with the second (512 x 8192, D = 256: 87.2 / 72.8 us) and
    // 25-50 % with the first.
    if (rule.more_waves_long_rows) {
        if (avg >= 1536.0 && work_rows >= 96 * cus && rule_on(kRuleSixteenWavesTallLongRows)) W = 16;
        const double steps = avg / (rule.slots > 0 ? rule.slots : 1);
        if (2 * work_rows <= 3 * cus && steps >= 768.0 && rule_on(kRuleMoreWavesFewLongRows)) W = 16;
        else if (2 * work_rows <= 3 * cus && steps >= 384.0 && W < 8 && rule_on(kRuleMoreWavesFewLongRows)) W = 8;
    }
    if (W > rule.max_w) W = rule.max_w;
    R = 1;
    if (W == 4) {
        for (int r = 2; r <= 16 && rule_on(kRuleGroupRows); r *= 2) {
            const long long blocks = ceil_div(M, r) * col_tiles;
            if (blocks < rule.blocks_per_cu * cus || avg * r > 512.0) break;
            R = r;
        }
        // Rows known to be even: four rows per four-wave workgroup, which the kernels then run as one whole row per
        // wave (no partial sums, no barrier, one chain of accesses per row instead of four): 3-17 % faster than one
        // row per workgroup from 2048 rows on, and 1.3-1.7x where the gathered operands exceed one L2 (8192 x 128
        // floats twice in the fused op), because waves that start together then sweep the columns together. With
        // uneven rows the same grouping is 5-20 % slower (four rows of work per workgroup make the tail of the
        // launch coarser), hence only on the caller's word. Rows below 128 nonzeros keep the grouping of the size rule
        // (4096 rows of ~100: four per workgroup measured 6 % slower than two) -- except in SpMM where a row of the dense
        // operand takes a whole wave (from 256 columns on; rule.even_rows_avg): there the grouping pays from about a
        // hundred nonzeros per row (2048 x 512 with 102 per row: N = 392 14.9 -> 14.5 us, N = 256 9.7 -> 8.9 us).
        if (rows_even && R < 4 && avg >= rule.even_rows_avg && ceil_div(M, 4) * col_tiles >= 2 * cus) R = 4;
        // Long rows known to lie next to each other (DLSPM_HINT_ROWS_SKEWED without a plan: dlspm_advise gives it where one
        // eighth of the rows holds 1.6 times its share of the nonzeros): a workgroup of sixteen such rows has sixteen mean
        // workgroups' work and four waves to do it with. Four rows at most, eight in the fused op (the reference's 33288 x 512
        // embedding, 17.6 nonzeros per row, a run of rows of 300 at its start: SpMM N = 256 57.2 -> 27.8 us, SDDMM D = 128
        // 35.5 -> 22.0 us, fused D = 64 34.8 -> 27.5 us with eight and 31.7 with four; with lengths independent of the position, sixteen rows lose nothing to four rows even at
        // sigma 1.2, and short even rows need the sixteen: 65536 rows of 8, fused 30.8 against 44.5 us).
        if (rows == kRowsSkewed && R > rule.skewed_rows_cap) R = rule.skewed_rows_cap;
    }
}

constexpr int kCutPlanAdviceMaxRows = 16384;     // the cut rule is one workgroup's work: 16 rounds of 1024 rows
constexpr double kCutPlanMinGainNs = 2500.0;      // fused, SpMM with partial rows: the kernel that adds the pieces must be paid for
constexpr double kCutPlanMinGainNsOneKernel = 300.0;  // SDDMM, and SpMM where the pieces share the columns: no second kernel
constexpr int kCutPlanMinNnzSpmm = 5000;            // SpMM: no cut plan for fewer nonzeros
constexpr double kCutPlanMinGainNsSddmmOneRowEach = 1000.0;  // ... one and a half to two rows per compute unit: eight waves per row do nearly as well

// longest row and number of rows without nonzeros (dlspm_csr_row_stats); stats[0] = max, stats[1] = empty rows
__global__ void row_stats_kernel(int M, const int* __restrict__ row_offsets, int* __restrict__ stats)
{
    int longest = 0, empty = 0;
    const long long stride = (long long)gridDim.x * blockDim.x;  // 64-bit: i + stride must not wrap for M near INT_MAX
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < M; i += stride) {
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
    const long long tid = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    const long long stride = (long long)gridDim.x * blockDim.x;  // 64-bit: i + stride must not wrap near INT_MAX
    int f = 0;
    if (tid == 0) {
        if (row_offsets[M] != nnz) f |= 2;
        if (row_offsets[0] != 0) f |= 32;
    }
    for (long long i = tid; i < M; i += stride) {
        const int lo = row_offsets[i], hi = row_offsets[i + 1];
        if (hi < lo) f |= 4;
        if (hi - lo > K) f |= 8;
    }
    if (!(f & 2)) {
        for (long long i = tid; i < nnz; i += stride) {
            const int c = col_indices[i];
            if (c >= K) f |= 16;
            if (c < 0) f |= 64;
        }
    }
    if (f) atomicOr(flags, f);
}

// the sliced plan of each op, from its lane layout (0 slices: not used)
static SlicePlan spmm_slice_plan(const DeviceInfo& dev, int M, int K, int N, int nnz, const SpmmShape& s)
{
    const int tw = s.G * s.vec * s.V;
    // the column tiles are worked through one after the other: one tile's slab of B is what is gathered from at a time
    // and the workgroups of one (slice, tile) pair should fill the device by themselves, or it gathers from several
    // slabs at once: rows per workgroup as if there were one tile (4096 x 65536, N = 3136, 25 tiles of 128, 131 or
    // 656 nonzeros per row: 856 -> 716 us and 2320 -> 2133 us)
    SlicePlan p = slice_plan(dev, M, K, N < tw ? N : tw, nnz, 1, 0, s.vec == 4 ? s.G : 0, true, kWave / s.G, 8);
    p.bytes = p.slices > 0 ? p.bounds_bytes + (size_t)p.slices * M * (size_t)N * sizeof(float) : 0;
    return p;
}
static SlicePlan fused_slice_plan(const DeviceInfo& dev, int M, int K, int D, int nnz, const FusedShape& s)
{
    const int tw = s.G * s.vec * s.V;
    const bool built = s.vec == 4 && s.G1 == 8 && s.DS > 0 && tw >= D;  // the widths the sliced kernels are built for (17 .. 512)
    return slice_plan(dev, M, K, D, nnz, 2, D, built ? s.G : 0, true, kWave / s.G, 2);
}
static SlicePlan sddmm_slice_plan(const DeviceInfo& dev, int M, int K, int D, int nnz, const SddmmShape& s)
{
    const bool built = s.vec == 4 && s.G1 == 8 && s.DS >= 1;  // 16 < D <= 512
    return slice_plan(dev, M, K, D, nnz, 1, 0, built ? kWave : 0, false, kWave / s.G1, 2);
}

}  // namespace dlspm

using namespace dlspm;

extern "C" {

void dlspm_tuning_default(dlspm_tuning* t)
{
    if (!t) return;
    const Tuning d;
    *t = dlspm_tuning{d.split_w, d.split_r, d.flat, d.flat_chunk, d.slices, d.tile_major, d.tile_width, d.plan_order,
                      d.xcd_contiguous, d.stream_results, d.cut_piece_pct, d.cut_longest_pct, d.rules_off, d.compute_units};
}

int dlspm_set_tuning(const dlspm_tuning* t)
{
    if (!t) {  // back to the process default
        t_tuning_set = false;
        return DLSPM_OK;
    }
    if (t->split_w < 0 || t->split_r < 0 || t->flat < -1 || t->flat > 1 || t->flat_chunk < 0 || t->slices < -1 ||
        t->tile_major < -1 || t->tile_major > 3 || t->tile_width < 0 || t->plan_order < 0 || t->plan_order > 2 ||
        t->xcd_contiguous < 0 || t->xcd_contiguous > 1 || t->stream_results < -1 || t->stream_results > 1 ||
        (t->cut_piece_pct != 0 && (t->cut_piece_pct < 10 || t->cut_piece_pct > 1000)) ||
        (t->cut_longest_pct != 0 && (t->cut_longest_pct < 10 || t->cut_longest_pct > 1000)) || t->rules_off < 0 || t->rules_off > 2047 ||
        (t->compute_units != 0 && (t->compute_units < 8 || t->compute_units > 1024 || t->compute_units % 8 != 0)))
        return DLSPM_E_INVALID_ARG;
    t_tuning.split_w = t->split_w;
    t_tuning.split_r = t->split_r;
    t_tuning.flat = t->flat;
    t_tuning.flat_chunk = t->flat_chunk;
    t_tuning.slices = t->slices;
    t_tuning.tile_major = t->tile_major;
    t_tuning.tile_width = t->tile_width;
    t_tuning.plan_order = t->plan_order;
    t_tuning.xcd_contiguous = t->xcd_contiguous;
    t_tuning.stream_results = t->stream_results;
    t_tuning.cut_piece_pct = t->cut_piece_pct;
    t_tuning.cut_longest_pct = t->cut_longest_pct;
    t_tuning.rules_off = t->rules_off;
    t_tuning.compute_units = t->compute_units;
    t_tuning_set = true;
    return DLSPM_OK;
}

int dlspm_get_tuning(dlspm_tuning* t)
{
    if (!t) return DLSPM_E_INVALID_ARG;
    const Tuning& c = tuning();
    *t = dlspm_tuning{c.split_w, c.split_r, c.flat, c.flat_chunk, c.slices, c.tile_major, c.tile_width, c.plan_order,
                      c.xcd_contiguous, c.stream_results, c.cut_piece_pct, c.cut_longest_pct, c.rules_off, c.compute_units};
    return DLSPM_OK;
}

int dlspm_device_info(int* compute_units, long long* l2_bytes, int* is_gfx950)
{
    const DeviceInfo& d = device_info();
    if (compute_units) *compute_units = d.cus;
    if (l2_bytes) *l2_bytes = d.l2_bytes;
    if (is_gfx950) *is_gfx950 = d.present && d.gfx950 ? 1 : 0;
    return d.present ? DLSPM_OK : DLSPM_E_NO_DEVICE;
}

int spmm_csr_f32(int M, int K, int N, int nnz, const int* row_offsets, const int* col_indices, const float* values,
                 const float* B, float* C, void* workspace, size_t workspace_bytes, void* stream)
{
    if (M < 0 || K < 0 || N < 0 || nnz < 0) return DLSPM_E_INVALID_ARG;
    if ((long long)nnz > (long long)M * K) return DLSPM_E_INVALID_ARG;
    const WorkspaceArg ws = workspace_arg(workspace, workspace_bytes);
    if (ws.bad_hint) return DLSPM_E_INVALID_ARG;
    if (ws.row_plan && ws.mem && ws.bytes < row_plan_bytes(M)) return DLSPM_E_WORKSPACE;
    if (M == 0 || N == 0) return DLSPM_OK;
    if (!row_offsets || !C) return DLSPM_E_INVALID_ARG;
    if (nnz > 0 && (!col_indices || !values || !B)) return DLSPM_E_INVALID_ARG;
    const DeviceInfo& dev = device_info();
    if (const int st = require_device(dev)) return st;
    const bool vec4 = N >= 4;  // dwordx4 accesses need only dword alignment
    const SpmmArgs args{M, K, N, nnz, row_offsets, col_indices, values, B, C, ws.banded ? 1 : 0};
    hipStream_t st = static_cast<hipStream_t>(stream);
    hipError_t e;
    if (ws.cut_plan && ws.mem) {
        // the memory holds the cut plan of this matrix and room for the partial rows of its pieces
        const CutPlan cp = cut_plan_layout(M, N, dev.cus);
        if (cp.bytes == 0 || ws.bytes < cp.bytes) return DLSPM_E_WORKSPACE;
        SpmmShape shape = spmm_choose(dev, M, K, N, nnz, vec4, false, true);
        e = spmm_plan_applies(dev, shape, M, N, nnz) ? spmm_pieces_launch(args, shape, cp, ws.mem, st)
                                                : spmm_launch(args, spmm_choose(dev, M, K, N, nnz, vec4, false, true, false, true), st);
        return e == hipSuccess ? DLSPM_OK : fail_hip(e);
    }
    if (ws.row_plan && ws.mem) {
        // the memory holds the row plan of this matrix; sizes a planned launch is not built for run as with NULL
        SpmmShape shape = spmm_choose(dev, M, K, N, nnz, vec4, false, true);
        e = spmm_plan_applies(dev, shape, M, N, nnz) ? spmm_planned_launch(args, shape, static_cast<const int*>(ws.mem), st)
                                                : spmm_launch(args, spmm_choose(dev, M, K, N, nnz, vec4, false, true, false, true), st);
        return e == hipSuccess ? DLSPM_OK : fail_hip(e);
    }
    // a banded matrix (DLSPM_HINT_BANDED) runs as row blocks whatever memory came with the call: column slices and
    // the flat schedule are answers to columns spread over all of K and to uneven rows
    const bool memory = !ws.rows_even && !ws.banded && ws.mem != nullptr;
    const SpmmShape shape = spmm_choose(dev, M, K, N, nnz, vec4, ws.rows_even ? kRowsEven : ws.skewed ? kRowsSkewed : kRowsUnknown, !memory, ws.banded, !memory);
    if (memory) {
        const SlicePlan sliced = spmm_slice_plan(dev, M, K, N, nnz, shape);
        const FlatPlan plan = sliced.slices > 0 ? FlatPlan{0, 0, 0} : flat_plan(dev, M, nnz, N, shape.G);
        if (ws.bytes < (sliced.slices > 0 ? sliced.bytes : plan.bytes)) return DLSPM_E_WORKSPACE;
        if (sliced.slices > 0)
            e = spmm_sliced_launch(args, shape, sliced, ws.mem, st);
        else if (plan.chunk > 0)
            e = spmm_flat_launch(args, shape, plan, static_cast<float*>(ws.mem), st);
        else
            e = spmm_launch(args, shape, st);
    } else {
        e = spmm_launch(args, shape, st);
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
    const size_t need = dlspm_workspace_bytes(DLSPM_OP_SPMM, M, K, N, nnz);  // of the flat or column-sliced schedule
    if (need > kStaticScratchBytes) return DLSPM_E_STATIC_LIMIT;
    if (need == 0)  // the schedule of these sizes keeps everything in registers and LDS
        return spmm_csr_f32(M, K, N, nnz, row_offsets, col_indices, values, B, C, nullptr, 0, stream);
    hipError_t e = hipSuccess;
    void* ptr = static_scratch(e);
    if (!ptr) return fail_hip(e);
    return spmm_csr_f32(M, K, N, nnz, row_offsets, col_indices, values, B, C, ptr, kStaticScratchBytes, stream);
}

size_t dlspm_row_plan_bytes(int M) { return row_plan_bytes(M); }

static int cut_plan_width(int op, int N_or_D) { return op == DLSPM_OP_SDDMM ? 0 : N_or_D; }

size_t dlspm_row_plan_bytes_for(int op, int M, int N_or_D)
{
    const DeviceInfo& dev = device_info();
    if ((op != DLSPM_OP_SPMM && op != DLSPM_OP_SDDMM && op != DLSPM_OP_FUSED) || N_or_D < 0) return 0;
    return cut_plan_layout(M, cut_plan_width(op, N_or_D), dev.cus).bytes;
}

int dlspm_row_plan_build_cut(int M, const int* row_offsets, void* plan, size_t plan_bytes, void* stream)
{
    if (M < 0 || M > kCutPlanMaxRows) return DLSPM_E_INVALID_ARG;
    if (M == 0) return DLSPM_OK;
    if (!row_offsets || !plan) return DLSPM_E_INVALID_ARG;
    const DeviceInfo& dev = device_info();
    if (const int st = require_device(dev)) return st;
    const CutPlan cp = cut_plan_layout(M, 0, dev.cus);  // what the build writes ends where the partial rows begin
    if (plan_bytes < cp.bytes) return DLSPM_E_WORKSPACE;
    const hipError_t e = cut_plan_build_launch(M, row_offsets, cp, plan, tuning().plan_order, static_cast<hipStream_t>(stream));
    return e == hipSuccess ? DLSPM_OK : fail_hip(e);
}

int dlspm_row_plan_build(int M, const int* row_offsets, void* plan, size_t plan_bytes, void* stream)
{
    if (M < 0) return DLSPM_E_INVALID_ARG;
    if (M == 0) return DLSPM_OK;
    if (!row_offsets || !plan) return DLSPM_E_INVALID_ARG;
    if (plan_bytes < row_plan_bytes(M)) return DLSPM_E_WORKSPACE;
    const DeviceInfo& dev = device_info();
    if (const int st = require_device(dev)) return st;
    // one bin per compute unit: the first 8 x bins workgroups of a launch start together, eight on each compute unit
    const hipError_t e = row_plan_build_launch(M, row_offsets, static_cast<int*>(plan), dev.cus,
                                               tuning().plan_order, static_cast<hipStream_t>(stream));
    return e == hipSuccess ? DLSPM_OK : fail_hip(e);
}

// Whether cutting the longest rows (a cut plan) is expected to beat the plan over whole rows. The longest row runs on
// one compute unit, which gathers about 48 bytes per clock (115 bytes per nanosecond at 2.4 GHz) of dense rows; cut, no
// entry is longer than one and a half shares. What that saves is set against what the cut plan costs: where the pieces
// leave partial rows (the fused op; SpMM outside 33 ... 512 columns) the second kernel that adds them (about 2 us between
// two graph nodes), else (SDDMM; SpMM where the pieces share the row's columns) only a grid that is two entries per
// compute unit larger. `spread`: the workgroups over which a call without plan spreads every row by itself (few rows: SpMM's
// column tiles, SDDMM's row pieces); the longest row then keeps one compute unit busy for that fraction of its length only.
static bool cut_plan_pays(const DeviceInfo& dev, int op, int M, int width, int nnz, int max_row_len, bool second_kernel, int spread = 1)
{
    if (max_row_len <= 0 || M > kCutPlanAdviceMaxRows) return false;
    const long long cus = dev.cus;
    // With a second kernel: only where a share holds at least two mean rows, so that the rows above one and a half
    // shares are the exception and the kernel that adds their pieces has little to do (the reference's layers of 64 ...
    // 256 rows, where most rows would be cut: 0.85 ... 1.5 times the time of the plan over whole rows; 512 rows: 0.66 ... 1.0)
    // The fused op on few rows is the exception: one row per compute unit, eight waves on it, most of the device idle, so a
    // long row pays for the second kernel from a gain of 6 us by this model on (10 us below 32 rows, where a share is a
    // handful of nonzeros), shares of 32 nonzeros and more (lognormal rows, sigma 0.8, NULL / cut plan: 64 x 2304 of 230
    // per row, D = 128: 14.5 / 10.1 us; 32 x 4608 of 1380, D = 256: 82.6 / 16.8 us; even rows 64 x 4608, D = 128: 17.2 /
    // 10.5 us; below the threshold the cut plan loses 5-60 %: the reference's layers of 128 ... 256 rows, D = 64: 1.2-1.5x).
    const bool few_rows_fused = op == DLSPM_OP_FUSED && M < 2 * cus;
    if (second_kernel && M < 2 * cus && !few_rows_fused) return false;
    // SpMM on a handful of nonzeros is all start-up, and the cut plan's larger grid adds to it (the reference's data set at
    // N = 256, cut plan / NULL: 1.10 below 2500 nonzeros (21 files), 1.00 below 5000 (23), 0.92 below 10 000 (49); SDDMM gains
    // at every size: 0.89 / 0.91 / 0.88)
    if (op == DLSPM_OP_SPMM && nnz < kCutPlanMinNnzSpmm) return false;
    const long long share = std::max<long long>(ceil_div(nnz, cus), 1);
    const long long longest_whole = (share * kCutAdvicePct + 99) / 100;
    const long long longest_unit = ceil_div(max_row_len, std::max(spread, 1));
    if (longest_unit <= longest_whole) return false;
    const double bytes_per_nonzero = (op == DLSPM_OP_FUSED ? 2.0 : 1.0) * (double)std::min(width, 512) * sizeof(float);
    const double saved_ns = (double)(longest_unit - longest_whole) * bytes_per_nonzero / 115.0;
    if (few_rows_fused) return share >= 32 && saved_ns >= (M < 32 ? 10000.0 : 6000.0);
    if (second_kernel) return saved_ns >= kCutPlanMinGainNs;
    // (SpMM, N = 256, the 302 files of the reference's data set with a row above one and a half shares, against the better
    // of NULL and the plan over whole rows: 0.99 of the time below 300 ns by this model, 0.96 / 0.91 / 0.84 / 0.81 from 300 /
    // 600 / 1000 / 2500 ns on, at every height from 64 to 2048 rows)
    if (op == DLSPM_OP_SDDMM && 2 * M > 3 * cus && M < 2 * cus) return saved_ns >= kCutPlanMinGainNsSddmmOneRowEach;
    return saved_ns >= kCutPlanMinGainNsOneKernel;
}

// the longest row at least twenty times the mean: what DLSPM_HINT_ROWS_SKEWED says
static bool rows_are_skewed(int M, int nnz, int max_row_len)
{
    return M > 0 && max_row_len >= 0 && (double)max_row_len * M >= 20.0 * (double)nnz;
}

int dlspm_row_plan_advice(int op, int M, int K, int N_or_D, int nnz, int max_row_len)
{
    const DeviceInfo& dev = device_info();
    if (M <= 0 || K <= 0 || N_or_D <= 0 || nnz <= 0) return 0;
    const bool vec4 = N_or_D >= 4;
    bool second_kernel = op == DLSPM_OP_FUSED;  // a cut plan's pieces leave partial rows for a second kernel to add
    int spread = 1;  // workgroups over which a call without plan spreads each row by itself
    int model_width = N_or_D;  // floats gathered per nonzero by one workgroup
    if (op == DLSPM_OP_SPMM) {
        SpmmShape shape = spmm_choose(dev, M, K, N_or_D, nnz, vec4, false, true);
        if (!spmm_plan_applies(dev, shape, M, N_or_D, nnz)) return 0;
        second_kernel = !spmm_cut_by_columns(shape, N_or_D);
        // few rows: a call without plan works in narrower column tiles than a planned launch does
        const SpmmShape plain = spmm_choose(dev, M, K, N_or_D, nnz, vec4, false, true, false, true);
        const long long tiles = ceil_div(N_or_D, shape.G * shape.vec * shape.V), tiles_plain = ceil_div(N_or_D, plain.G * plain.vec * plain.V);
        if (!plain.tile_major && tiles_plain > tiles) spread = (int)(tiles_plain / tiles);
        // dense rows in column tiles: a workgroup gathers one tile's width per nonzero, and that is what a cut would save
        model_width = std::min(N_or_D, shape.G * shape.vec * shape.V);
    } else if (op == DLSPM_OP_SDDMM) {
        SddmmShape shape = sddmm_choose(dev, M, N_or_D, nnz, vec4);
        if (!sddmm_plan_applies(dev, shape, M, N_or_D, nnz, rows_are_skewed(M, nnz, max_row_len))) {
            // fewer rows than compute units: only a cut plan helps (its pieces fill the device)
            SddmmShape few = sddmm_choose(dev, M, N_or_D, nnz, vec4), plain = few;
            sddmm_few_rows_pieces(dev, plain, M, nnz);  // what a call without plan does by itself
            // (from three quarters of a compute unit's count of rows on, its two workgroups per row fill the device no
            // better than the rows themselves would: lognormal rows on 200 ... 384 rows, D = 64 ... 256, a cut plan against
            // the call without: 0.95 of the time and less from 300 ns by the model of whole rows on, 0.5 ... 0.8 from 2000 ns)
            const int spread = 4ll * M > 3ll * dev.cus ? 1 : 1 << plain.pieces_lg;
            return sddmm_cut_plan_applies(dev, few, M, N_or_D, nnz) &&
                           cut_plan_pays(dev, op, M, N_or_D, nnz, max_row_len, false, spread)
                       ? 2
                       : 0;
        }
    } else if (op == DLSPM_OP_FUSED) {
        FusedShape shape = fused_choose(dev, M, N_or_D, nnz, vec4);
        if (!fused_plan_applies(dev, shape, M, N_or_D, nnz, rows_are_skewed(M, nnz, max_row_len))) {
            // fewer rows than two per compute unit (eight waves per row): only a cut plan helps, where a row is long enough
            // to pay for the kernel that adds its pieces
            FusedShape few = fused_choose(dev, M, N_or_D, nnz, vec4);
            return fused_cut_plan_applies(dev, few, M, N_or_D, nnz) && cut_plan_pays(dev, op, M, N_or_D, nnz, max_row_len, true) ? 2 : 0;
        }
    } else {
        return 0;
    }
    // rows known to be even gain nothing from another order (and the even-rows hint may serve them better)
    if (max_row_len >= 0 && max_row_len <= 1.5 * ((double)nnz / M)) return 0;
    // SDDMM on short rows groups them by the size rule, and gives that up for the plan's order only where they are far
    // from even (2048 x 512 of the reference's data set, 10 per row, D = 128: longest 158, 3.56 -> 2.65 us; longest 23,
    // 3.34 -> 3.66 us; over the files of that shape: a longest row of 4 ... 8 times the mean +4 ... 6 %, of 8 ... 12 times
    // -4 %, beyond that -8 ... 14 %)
    if (op == DLSPM_OP_SDDMM && (long long)nnz < 32ll * M && max_row_len >= 0 && max_row_len < 8.0 * ((double)nnz / M)) return 0;
    // dense operands well beyond one L2 need the column-sliced schedule's workspace more than they need balance; the
    // flat schedule, though, is behind the plan wherever both apply (SpMM, lognormal rows, sigma 1 ... 2, row-block /
    // flat / plan: 8192 x 2048, N = 128: 45.4 / 41.2 / 30.8 us; 16384 x 4096: 121 / 105 / 86.6 us; 32768 x 8192: 525 / 466
    // / 424 us)
    int slices = 0;
    (void)dlspm_describe_slices(op, M, K, N_or_D, nnz, &slices, nullptr);
    if (slices >= 3) return 0;
    // (dense rows in column tiles: the tiles already spread a long row over several workgroups, and the partial rows of a cut
    // would be N floats wide: lognormal rows, sigma 1.2, cut plan / plan over whole rows: 512 x 2048, N = 1024: 23.6 / 16.0 us;
    // 1024 x 1152, N = 12544: 229 / 203 us; 512 x 4608, N = 3136: 121 / 132 us)
    const bool tiled = op == DLSPM_OP_SPMM && model_width < N_or_D;
    if (!tiled && cut_plan_pays(dev, op, M, model_width, nnz, max_row_len, second_kernel, spread)) return 2;
    return spread > 1 ? 0 : 1;  // (a plan over whole rows would undo the spread)
}

int sddmm_csr_f32(int M, int K, int D, int nnz, const int* row_offsets, const int* col_indices, const float* lhs,
                  const float* rhs, float* out_values, void* workspace, size_t workspace_bytes, void* stream)
{
    if (M < 0 || K < 0 || D < 0 || nnz < 0) return DLSPM_E_INVALID_ARG;
    if ((long long)nnz > (long long)M * K) return DLSPM_E_INVALID_ARG;
    const WorkspaceArg ws = workspace_arg(workspace, workspace_bytes);
    if (ws.bad_hint) return DLSPM_E_INVALID_ARG;
    if (ws.row_plan && ws.mem && ws.bytes < row_plan_bytes(M)) return DLSPM_E_WORKSPACE;
    if (M == 0 || nnz == 0) return DLSPM_OK;
    if (!row_offsets || !col_indices || !out_values) return DLSPM_E_INVALID_ARG;
    if (D > 0 && (!lhs || !rhs)) return DLSPM_E_INVALID_ARG;
    const DeviceInfo& dev = device_info();
    if (const int st = require_device(dev)) return st;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (D == 0) {
        const unsigned blocks = (unsigned)ceil_div(nnz, 256);
        hipLaunchKernelGGL(fill_zero_kernel, dim3(blocks), dim3(256), 0, st, out_values, nnz);
        const hipError_t e0 = hipGetLastError();
        return e0 == hipSuccess ? DLSPM_OK : fail_hip(e0);
    }
    const bool vec4 = D >= 4;  // dwordx4 accesses need only dword alignment
    const SddmmArgs args{M, K, D, nnz, row_offsets, col_indices, lhs, rhs, out_values, ws.banded ? 1 : 0, dev.l2_bytes, dev.cus};
    if (ws.cut_plan && ws.mem) {
        const CutPlan cp = cut_plan_layout(M, 0, dev.cus);
        if (cp.bytes == 0 || ws.bytes < cp.bytes) return DLSPM_E_WORKSPACE;
        SddmmShape shape = sddmm_choose(dev, M, D, nnz, vec4);
        if (sddmm_cut_plan_applies(dev, shape, M, D, nnz)) {
            const hipError_t e = sddmm_pieces_launch(args, shape, cp, ws.mem, st);
            return e == hipSuccess ? DLSPM_OK : fail_hip(e);
        }
    }
    if (ws.row_plan && ws.mem) {
        SddmmShape shape = sddmm_choose(dev, M, D, nnz, vec4);
        if (sddmm_plan_applies(dev, shape, M, D, nnz, ws.skewed)) {
            const hipError_t e = sddmm_planned_launch(args, shape, static_cast<const int*>(ws.mem), st);
            return e == hipSuccess ? DLSPM_OK : fail_hip(e);
        }
        // sizes a planned launch is not built for run as with NULL
    }
    const SddmmShape shape = sddmm_choose(dev, M, D, nnz, vec4, ws.rows_even ? kRowsEven : ws.skewed ? kRowsSkewed : kRowsUnknown);
    // the flat schedule needs no workspace here (nothing to combine), so the size rule alone decides; it has no
    // width condition for SDDMM (measured for D = 32 ... 256: equal on uniform rows, 15-33 % faster on skewed ones)
    if (ws.mem && !ws.rows_even && !ws.row_plan && !ws.cut_plan && !ws.banded) {
        // with a workspace for the slice boundaries: the column-sliced schedule where the rhs operand exceeds one L2
        const SlicePlan sliced = sddmm_slice_plan(dev, M, K, D, nnz, shape);
        if (ws.bytes < sliced.bytes) return DLSPM_E_WORKSPACE;
        if (sliced.slices > 0) {
            const hipError_t es = sddmm_sliced_launch(args, shape, sliced, ws.mem, st);
            return es == hipSuccess ? DLSPM_OK : fail_hip(es);
        }
    }
    // (rows known to be even have nothing to gain from the flat schedule, which costs them 4 ... 12 % today: the reference's
    // grid at density 0.1, 12288 ... 32768 rows of 410 ... 819 nonzeros, D = 32 and 128)
    const FlatPlan plan = ws.banded || ws.rows_even ? FlatPlan{0, 0, 0} : sddmm_flat_plan(dev, M, K, nnz, D);
    SddmmShape plain = shape;
    if (plan.chunk == 0) sddmm_few_rows_pieces(dev, plain, M, nnz);
    const hipError_t e = plan.chunk > 0 ? sddmm_flat_launch(args, shape, plan.chunk, st) : sddmm_launch(args, plain, st);
    return e == hipSuccess ? DLSPM_OK : fail_hip(e);
}

int fused_sddmm_spmm_f32(int M, int K, int D, int nnz, const int* row_offsets, const int* col_indices, const float* Q,
                         const float* Kmat, const float* V, float scale, float* O, void* workspace,
                         size_t workspace_bytes, void* stream)
{
    if (M < 0 || K < 0 || D < 0 || nnz < 0) return DLSPM_E_INVALID_ARG;
    if ((long long)nnz > (long long)M * K) return DLSPM_E_INVALID_ARG;
    const WorkspaceArg ws = workspace_arg(workspace, workspace_bytes);
    if (ws.bad_hint) return DLSPM_E_INVALID_ARG;
    if (ws.row_plan && ws.mem && ws.bytes < row_plan_bytes(M)) return DLSPM_E_WORKSPACE;
    if (M == 0 || D == 0) return DLSPM_OK;
    if (!row_offsets || !O) return DLSPM_E_INVALID_ARG;
    if (nnz > 0 && (!col_indices || !Q || !Kmat || !V)) return DLSPM_E_INVALID_ARG;
    const DeviceInfo& dev = device_info();
    if (const int st = require_device(dev)) return st;
    const bool vec4 = D >= 4;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const FusedArgs args{M, K, D, nnz, row_offsets, col_indices, Q, Kmat, V, scale, O, ws.banded ? 1 : 0};
    hipError_t e;
    if (ws.cut_plan && ws.mem) {
        const CutPlan cp = cut_plan_layout(M, D, dev.cus);
        if (cp.bytes == 0 || ws.bytes < cp.bytes) return DLSPM_E_WORKSPACE;
        FusedShape shape = fused_choose(dev, M, D, nnz, vec4);
        e = fused_cut_plan_applies(dev, shape, M, D, nnz) ? fused_pieces_launch(args, shape, cp, ws.mem, st) : fused_launch(args, shape, st);
        return e == hipSuccess ? DLSPM_OK : fail_hip(e);
    }
    if (ws.row_plan && ws.mem) {
        FusedShape shape = fused_choose(dev, M, D, nnz, vec4);
        e = fused_plan_applies(dev, shape, M, D, nnz, ws.skewed) ? fused_planned_launch(args, shape, static_cast<const int*>(ws.mem), st)
                                                 : fused_launch(args, shape, st);
        return e == hipSuccess ? DLSPM_OK : fail_hip(e);
    }
    const FusedShape shape = fused_choose(dev, M, D, nnz, vec4, ws.rows_even ? kRowsEven : ws.skewed ? kRowsSkewed : kRowsUnknown, K);
    if (!ws.rows_even && !ws.banded && ws.mem) {
        const SlicePlan sliced = fused_slice_plan(dev, M, K, D, nnz, shape);
        const FlatPlan plan = sliced.slices > 0 ? FlatPlan{0, 0, 0} : flat_plan(dev, M, nnz, D, shape.G);
        if (ws.bytes < (sliced.slices > 0 ? sliced.bytes : plan.bytes)) return DLSPM_E_WORKSPACE;
        if (sliced.slices > 0)
            e = fused_sliced_launch(args, shape, sliced, ws.mem, st);
        else if (plan.chunk > 0)
            e = fused_flat_launch(args, shape, plan, static_cast<float*>(ws.mem), st);
        else
            e = fused_launch(args, shape, st);
    } else {
        e = fused_launch(args, shape, st);
    }
    return e == hipSuccess ? DLSPM_OK : fail_hip(e);
}

size_t dlspm_workspace_bytes(int op, int M, int K, int N_or_D, int nnz)
{
    const DeviceInfo& dev = device_info();
    // The workgroup-per-row-block schedule splits the work from row_offsets alone and keeps partial sums in LDS: no
    // scratch. Where flat_plan's rule selects the flat schedule for SpMM or the fused op, its partial rows live in the
    // workspace; a call without workspace runs the row-block schedule instead.
    if (M <= 0 || N_or_D <= 0 || nnz <= 0) return 0;
    if (op == DLSPM_OP_SPMM) {
        const SpmmShape s = spmm_choose(dev, M, K, N_or_D, nnz, N_or_D >= 4, false, false);  // a call with memory
        const SlicePlan sliced = spmm_slice_plan(dev, M, K, N_or_D, nnz, s);
        return sliced.slices > 0 ? sliced.bytes : flat_plan(dev, M, nnz, N_or_D, s.G).bytes;
    }
    if (op == DLSPM_OP_FUSED) {
        const FusedShape s = fused_choose(dev, M, N_or_D, nnz, N_or_D >= 4);
        const SlicePlan sliced = fused_slice_plan(dev, M, K, N_or_D, nnz, s);
        return sliced.slices > 0 ? sliced.bytes : flat_plan(dev, M, nnz, N_or_D, s.G).bytes;
    }
    if (op == DLSPM_OP_SDDMM) {  // every result goes into its own CSR slot: only the slice boundaries need memory
        const SddmmShape s = sddmm_choose(dev, M, N_or_D, nnz, N_or_D >= 4);
        return sddmm_slice_plan(dev, M, K, N_or_D, nnz, s).bytes;
    }
    return 0;
}

int dlspm_csr_check(int M, int K, int nnz, const int* row_offsets, const int* col_indices, void* stream)
{
    if (M < 0 || K < 0 || nnz < 0) return DLSPM_E_INVALID_ARG;
    if ((long long)nnz > (long long)M * K) return DLSPM_E_INVALID_CSR;
    if (!row_offsets) return DLSPM_E_INVALID_ARG;
    if (nnz > 0 && !col_indices) return DLSPM_E_INVALID_ARG;
    const DeviceInfo& dev = device_info();
    if (const int st = require_device(dev)) return st;
    hipStream_t s = static_cast<hipStream_t>(stream);
    int* d_flags = nullptr;
    hipError_t e = hipMalloc(&d_flags, sizeof(int));
    if (e != hipSuccess) return fail_hip(e);
    int h_flags = 0;
    e = hipMemsetAsync(d_flags, 0, sizeof(int), s);
    if (e == hipSuccess) {
        const long long work = (long long)(M > nnz ? M : nnz);
        int blocks = (int)ceil_div(work, 256);
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
        const DeviceInfo& dev = device_info();
    if (const int st = require_device(dev)) return st;
        hipStream_t s = static_cast<hipStream_t>(stream);
        int* d = nullptr;
        hipError_t e = hipMalloc(&d, 2 * sizeof(int));
        if (e != hipSuccess) return fail_hip(e);
        e = hipMemsetAsync(d, 0, 2 * sizeof(int), s);
        if (e == hipSuccess) {
            int blocks = (int)std::min<long long>(ceil_div(M, 256), 1024);
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
    const DeviceInfo& dev = device_info();
    if (passing != DLSPM_PASS_NULL && passing != DLSPM_PASS_ROWS_EVEN && passing != DLSPM_PASS_WORKSPACE && passing != DLSPM_PASS_ROWS_SKEWED)
        return DLSPM_E_INVALID_ARG;
    const bool even = passing == DLSPM_PASS_ROWS_EVEN;
    const int rows = even ? kRowsEven : passing == DLSPM_PASS_ROWS_SKEWED ? kRowsSkewed : kRowsUnknown;
    const bool memory = passing == DLSPM_PASS_WORKSPACE;
    if (!shape || M < 0 || N_or_D < 0 || nnz < 0) return DLSPM_E_INVALID_ARG;
    const int n = N_or_D;
    const bool vec4 = n >= 4;
    for (int i = 0; i < 10; ++i) shape[i] = 0;
    if (op == DLSPM_OP_SPMM) {
        const SpmmShape s = spmm_choose(dev, M, K, n, nnz, vec4, rows, !memory, false, !memory);
        const int tw = s.G * s.vec * s.V;
        shape[0] = s.vec; shape[1] = s.G; shape[2] = s.V; shape[5] = s.W; shape[6] = s.R; shape[7] = (int)ceil_div(n, tw);
        const FlatPlan fp = flat_plan(dev, M, nnz, n, s.G);
        shape[8] = fp.chunk; shape[9] = fp.units;
    } else if (op == DLSPM_OP_SDDMM) {
        SddmmShape s = sddmm_choose(dev, M, n, nnz, vec4, rows);
        const FlatPlan fp = even ? FlatPlan{0, 0, 0} : sddmm_flat_plan(dev, M, K, nnz, n);  // as sddmm_csr_f32 decides
        if (!memory && fp.chunk == 0) sddmm_few_rows_pieces(dev, s, M, nnz);
        // ([7]: the workgroups that share a row -- SDDMM has no column tiles)
        shape[0] = s.vec; shape[3] = s.G1; shape[4] = s.DS; shape[5] = s.W; shape[6] = s.R; shape[7] = 1 << s.pieces_lg;
        shape[8] = fp.chunk; shape[9] = fp.units;
    } else if (op == DLSPM_OP_FUSED) {
        const FusedShape s = fused_choose(dev, M, n, nnz, vec4, rows, K);
        const int tw = s.G * s.vec * s.V;
        shape[0] = s.vec; shape[1] = s.G; shape[2] = s.V; shape[3] = s.G1; shape[4] = s.DS; shape[5] = s.W; shape[6] = s.R;
        shape[7] = (int)ceil_div(n, tw);
        const FlatPlan fp = flat_plan(dev, M, nnz, n, s.G);
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
    const DeviceInfo& dev = device_info();
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
        const SpmmShape without = spmm_choose(dev, M, K, N_or_D, nnz, N_or_D >= 4, false, true);
        const SpmmShape with = spmm_choose(dev, M, K, N_or_D, nnz, N_or_D >= 4, false, false);
        if (without.tile_major && without.G * without.V < with.G * with.V) sliced = false;
    }
    if (sliced || (uneven && want > 0 && slices == 0)) return DLSPM_PASS_WORKSPACE;
    return even ? DLSPM_PASS_ROWS_EVEN : DLSPM_PASS_NULL;
}

int dlspm_describe_slices(int op, int M, int K, int N_or_D, int nnz, int* slices, int* rows_per_workgroup)
{
    const DeviceInfo& dev = device_info();
    if (M < 0 || K < 0 || N_or_D < 0 || nnz < 0) return DLSPM_E_INVALID_ARG;
    SlicePlan p{0, 1, 0, 0};
    if (op == DLSPM_OP_SPMM) p = spmm_slice_plan(dev, M, K, N_or_D, nnz, spmm_choose(dev, M, K, N_or_D, nnz, N_or_D >= 4, false, false));
    else if (op == DLSPM_OP_FUSED) p = fused_slice_plan(dev, M, K, N_or_D, nnz, fused_choose(dev, M, N_or_D, nnz, N_or_D >= 4));
    else if (op == DLSPM_OP_SDDMM) p = sddmm_slice_plan(dev, M, K, N_or_D, nnz, sddmm_choose(dev, M, N_or_D, nnz, N_or_D >= 4));
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

const char* dlspm_version(void) { return "dlspm_hip 0.3 gfx950"; }

}  // extern "C"
