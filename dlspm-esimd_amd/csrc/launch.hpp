// Argument bundles and launch-shape records shared by the kernel files and the C ABI layer.
#pragma once

#include <hip/hip_runtime.h>

#include <tuple>

namespace dlspm {

// ---- the shapes the kernels are built for, as compile-time tables, and the run-time dispatch onto them ---------------
// One table per kind of shape; a kernel family instantiates itself for every entry of the tables it is launched over
// (dispatch below calls `launch` with each entry type), and the size rules choose among the same entries, so a shape is
// added in one place.
template <int W_, int R_> struct Split { static constexpr int W = W_, R = R_; };  // waves, consecutive rows per workgroup
using Splits = std::tuple<Split<4, 16>, Split<4, 8>, Split<4, 4>, Split<4, 2>, Split<4, 1>, Split<8, 4>, Split<8, 2>, Split<8, 1>,
                          Split<16, 1>>;
template <int R_> struct Rows { static constexpr int R = R_; };  // rows per four-wave workgroup of the column-sliced kernels
using SlicedRows = std::tuple<Rows<1>, Rows<2>, Rows<4>, Rows<8>, Rows<16>>;
// SpMM: floats per lane and access, lanes per dense row, accesses per lane (the last entry: widths below 4)
template <int VEC_, int G_, int V_> struct RowLanes { static constexpr int VEC = VEC_, G = G_, V = V_; };
using SpmmLayouts = std::tuple<RowLanes<4, 64, 2>, RowLanes<4, 64, 1>, RowLanes<4, 32, 1>, RowLanes<4, 16, 1>, RowLanes<4, 8, 1>,
                               RowLanes<1, 8, 1>>;
// SDDMM: floats per lane and access, lanes per dot product, accesses per lane (0: a run-time loop)
template <int VEC_, int G1_, int DS_> struct DotLanes { static constexpr int VEC = VEC_, G1 = G1_, DS = DS_; };
using SddmmLayouts = std::tuple<DotLanes<4, 4, 1>, DotLanes<4, 8, 1>, DotLanes<4, 8, 2>, DotLanes<4, 8, 3>, DotLanes<4, 8, 4>,
                                DotLanes<4, 8, 6>, DotLanes<4, 8, 8>, DotLanes<4, 8, 12>, DotLanes<4, 8, 16>, DotLanes<4, 8, 0>,
                                DotLanes<1, 4, 1>>;
// fused: both stages
template <int VEC_, int G1_, int DS_, int G_, int V_> struct FusedLanes {
    static constexpr int VEC = VEC_, G1 = G1_, DS = DS_, G = G_, V = V_;
};
using FusedLayouts = std::tuple<FusedLanes<4, 4, 1, 8, 1>, FusedLanes<4, 8, 1, 8, 1>, FusedLanes<4, 8, 2, 16, 1>, FusedLanes<4, 8, 3, 32, 1>,
                                FusedLanes<4, 8, 4, 32, 1>, FusedLanes<4, 8, 6, 64, 1>, FusedLanes<4, 8, 8, 64, 1>, FusedLanes<4, 8, 12, 64, 2>,
                                FusedLanes<4, 8, 16, 64, 2>, FusedLanes<4, 8, 0, 64, 4>, FusedLanes<1, 4, 1, 8, 1>>;

// launch(entry) for the first entry of Table that `match` accepts; hipErrorInvalidValue if there is none
template <typename Table, typename Match, typename Launch> hipError_t dispatch(Match&& match, Launch&& launch)
{
    hipError_t e = hipErrorInvalidValue;
    bool found = false;
    auto one = [&](auto entry) {
        if (!found && match(entry)) {
            found = true;
            e = launch(entry);
        }
    };
    std::apply([&](auto... entry) { (one(entry), ...); }, Table{});
    return e;
}
template <typename Launch> hipError_t dispatch_split(int W, int R, Launch&& launch)
{
    return dispatch<Splits>([&](auto s) { return s.W == W && s.R == R; }, launch);
}
template <typename Launch> hipError_t dispatch_sliced_rows(int R, Launch&& launch)
{
    return dispatch<SlicedRows>([&](auto r) { return r.R == R; }, launch);
}
inline bool split_is_built(int W, int R, int max_w)
{
    return dispatch_split(W, R, [&](auto s) { return s.W <= max_w ? hipSuccess : hipErrorInvalidValue; }) == hipSuccess;
}

// ceil(a / b) without the overflow of (a + b - 1) for a near INT_MAX
inline long long ceil_div(long long a, long long b) { return (a + b - 1) / b; }

// A dense operand of `rows` x `width` floats can be read through a buffer descriptor (32-bit byte offsets)
// and through 24-bit multiplies of (row, row pitch in bytes)
inline bool dense_fits_buffer(long long rows, long long width)
{
    return rows * width * 4 < (1ll << 32) && rows < (1 << 24) && width * 4 < (1 << 24);
}

// DLSPM_E_LAUNCH, after noting e as the calling thread's last HIP error (dlspm_last_hip_error)
int fail_hip(hipError_t e);

// The device the calling thread has current, as far as the launch rules need it: compute units and the size of one
// L2. Read from hipDeviceProp_t once per device and cached; without a device (host-only queries on a machine that has
// none) the figures of a whole MI355X: 256 compute units, 4 MiB.
struct DeviceInfo {
    int cus;
    long long l2_bytes;
    bool present;  // a HIP device is current
    bool gfx950;   // ... and it is the architecture the kernels are built for
};
const DeviceInfo& device_info();  // one look-up per entry-point call; everything below takes the result as `dev`

// Overrides of the launch rules for tuning sweeps and tests (dlspm_set_tuning; one set per host thread, initialised from
// the environment once per process). The fields and their "follow the rule" values are those of dlspm_tuning.
struct Tuning {
    int split_w = 0, split_r = 0;
    int flat = -1, flat_chunk = 0;
    int slices = -1;
    int tile_major = -1, tile_width = 0;
    int plan_order = 0;
    int xcd_contiguous = 0;
    int stream_results = -1;
    int cut_piece_pct = 0, cut_longest_pct = 0;
    int rules_off = 0;  // DLSPM_RULE_* bits: size rules switched off, to measure what each is worth
    int compute_units = 0;  // > 0: device_info() reports this many compute units instead of the device's own
};
// (the values of DLSPM_RULE_* in the header)
constexpr int kRuleEightWavesFewRows = 1, kRuleSixteenWavesTallLongRows = 2, kRuleMoreWavesFewLongRows = 4, kRuleGroupRows = 8,
              kRuleRowAlignedSplit = 16, kRulePlanUngroups = 32, kRuleExactWidthKernels = 64, kRuleCutRowsByColumns = 128,
              kRuleFinerColumnTiles = 256, kRuleRowPiecesFewRows = 512, kRuleMaskByRange = 1024;

const Tuning& tuning();
inline bool rule_on(int rule) { return (tuning().rules_off & rule) == 0; }

// What a row-block kernel is told about its launch in one int: bit 0 = deal the row blocks to the XCDs in contiguous
// runs (DLSPM_HINT_BANDED or the tuning knob), bits 1-2 = results with the non-temporal hint: 0 by the size rule,
// 1 never, 2 wherever the rule could say so (dlspm_tuning.stream_results).
// bit 3 = never take the row-aligned split (DLSPM_RULE_ROW_ALIGNED_SPLIT switched off); bit 4 (SDDMM, one row per
// workgroup) = the waves of a row take whole passes of 64 nonzeros in turn (sddmm_row_interleaved).
constexpr int kFlagXcdContiguous = 1, kFlagStreamShift = 1, kFlagStreamNever = 1, kFlagStreamAlways = 2, kFlagNoAlignedSplit = 8,
              kFlagFullPasses = 16, kFlagPiecesShift = 8, kFlagPiecesMask = 7, kFlagTileOrderShift = 12;  // (bits 8-10: log2 of the workgroups that share a row, SDDMM; bits 12-13: SpmmShape::tile_major of a planned SpMM launch)
inline int launch_flags(int xcd_contiguous_hint)
{
    const Tuning& t = tuning();
    const int stream = t.stream_results < 0 ? 0 : t.stream_results == 0 ? kFlagStreamNever : kFlagStreamAlways;
    return ((xcd_contiguous_hint | t.xcd_contiguous) ? kFlagXcdContiguous : 0) | (stream << kFlagStreamShift) |
           ((t.rules_off & 16) ? kFlagNoAlignedSplit : 0);
}

// Lane layout and work split of one launch.
//   vec : floats per lane per access (4 = dwordx4 when the dense width is at least 4, else 1 = dword)
//   G   : lanes covering one dense row (SpMM / fused stage 2)          V  : accesses per lane per dense row
//   G1  : lanes covering one dot product (SDDMM / fused stage 1)        DS : accesses per lane per dot
//         product (0 = run-time loop, lhs row re-read instead of kept in registers)
//   W   : waves per workgroup                                           R  : consecutive rows per workgroup
// what the caller said about the rows (`rows` of the *_choose functions): nothing, DLSPM_HINT_ROWS_EVEN, or DLSPM_HINT_ROWS_SKEWED
// without a plan (long rows lie next to each other: fewer rows per workgroup)
constexpr int kRowsUnknown = 0, kRowsEven = 1, kRowsSkewed = 2;
constexpr int kTilesPerXcd = 2, kTilesPerXcdTileMajor = 3;  // SpmmShape::tile_major: 0 row-major, 1 tile-major, 2 / 3 each XCD on its own tiles (row- / tile-major within it)
struct SpmmShape { int vec, G, V, W, R, tile_major; };  // tile_major: column tiles one after the other (else row blocks)
struct SddmmShape { int vec, G1, DS, W, R, pieces_lg; };  // pieces_lg: 2^pieces_lg workgroups share each row (sddmm_few_rows_pieces)
struct FusedShape { int vec, G1, DS, G, V, W, R; };

struct SpmmArgs {
    int M, K, N, nnz;
    const int* row_offsets;
    const int* col_indices;
    const float* values;
    const float* B;
    float* C;
    int xcd_contiguous = 0;  // deal the row blocks to the XCDs in contiguous runs (DLSPM_HINT_BANDED)
};
struct SddmmArgs {
    int M, K, D, nnz;
    const int* row_offsets;
    const int* col_indices;
    const float* lhs;
    const float* rhs;
    float* out;
    int xcd_contiguous = 0;
    long long l2_bytes = 4ll << 20;  // of the device the call runs on (DeviceInfo::l2_bytes): results beyond it are streamed
    int cus = 256;                   // ... and its compute units
};
struct FusedArgs {
    int M, K, D, nnz;
    const int* row_offsets;
    const int* col_indices;
    const float* Q;
    const float* Kmat;
    const float* V;
    float scale;
    float* O;
    int xcd_contiguous = 0;
};

// Flat schedule: `units` waves of `chunk` consecutive nonzeros each; `bytes` of device workspace for the partial
// rows (units x 2 x width floats). chunk == 0: not used for this problem.
constexpr int kSlicedMinNnz = 1 << 19;  // the column-sliced schedule (two more launches) only from this many nonzeros on
constexpr long long kSlicedMinRowsPerCu = 4;  // ... and from this many rows per compute unit on (one slice's workgroups must fill the device)
constexpr int kFlatWaves = 4;  // waves per workgroup of the flat kernels (the waves are independent)
struct FlatPlan {
    int chunk;
    int units;
    size_t bytes;
};
FlatPlan flat_plan(const DeviceInfo& dev, int M, int nnz, int width, int G);
hipError_t row_fixup_launch(int M, int N, int chunk, const int* row_offsets, const float* partial, float* out,
                            hipStream_t stream);

// Column-sliced schedule: the columns of the sparse matrix (the rows of the gathered dense operands) are cut into
// `slices` equal ranges which the device works through one after the other, `R` rows per four-wave workgroup; the
// workspace holds the (slices + 1) x M slice boundaries of the rows, then slices x M x width partial rows (SpMM, fused).
// slices == 0: not used for this problem.
struct SlicePlan {
    int slices;
    int R;
    size_t bounds_bytes;
    size_t bytes;
};
// `operands`: dense operands gathered per nonzero (1 SpMM and SDDMM, 2 fused); `partial_width`: floats of a partial
// row that `bytes` accounts for (0: SDDMM has none, SpMM adds its own); `partial_rows`: the op writes partial rows at
// all (its slices are then a third larger); G, slots: the op's lane layout
SlicePlan slice_plan(const DeviceInfo& dev, int M, int K, int width, int nnz, int operands, int partial_width, int G, bool partial_rows,
                     int slots, int blocks_per_cu);
hipError_t slice_bounds_launch(int M, int K, int slices, const int* row_offsets, const int* col_indices, int* bounds,
                               hipStream_t stream);
hipError_t slice_sum_launch(long long count, int slices, const float* partial, float* out, hipStream_t stream);

// narrow_tiles: the call passes no workspace memory (column tiles below 128 columns are then allowed)
SpmmShape spmm_choose(const DeviceInfo& dev, int M, int K, int N, int nnz, bool vec4, int rows, bool narrow_tiles, bool banded = false,
                      bool plain = false);
hipError_t spmm_launch(const SpmmArgs& x, const SpmmShape& s, hipStream_t stream);
// Row plan (3 x M ints on the device: first nonzero, end and row number of the row that workgroup i works on): only for
// shapes of one row per four-wave workgroup and one column tile
hipError_t row_plan_build_launch(int M, const int* row_offsets, int* plan, int bins, int order, hipStream_t stream);
size_t row_plan_bytes(int M);
bool plan_ungroups(const DeviceInfo& dev, int M, int width, int nnz);  // SpMM: rows long enough that a plan runs them one per workgroup against the size rule
bool plan_ungroups_dots(const DeviceInfo& dev, int M, int D, int nnz);  // the same for SDDMM and the fused op
bool spmm_plan_applies(const DeviceInfo& dev, SpmmShape& s, int M, int N, int nnz);  // true: s is the shape of the planned launch (R = 1)
hipError_t spmm_planned_launch(const SpmmArgs& x, const SpmmShape& s, const int* plan, hipStream_t stream);
hipError_t spmm_flat_launch(const SpmmArgs& x, const SpmmShape& s, const FlatPlan& plan, float* partial,
                            hipStream_t stream);
hipError_t spmm_sliced_launch(const SpmmArgs& x, const SpmmShape& s, const SlicePlan& plan, void* workspace,
                              hipStream_t stream);

SddmmShape sddmm_choose(const DeviceInfo& dev, int M, int D, int nnz, bool vec4, int rows = kRowsUnknown);
void sddmm_few_rows_pieces(const DeviceInfo& dev, SddmmShape& s, int M, int nnz);  // a call without plan or memory: sets s.pieces_lg (and W = 4)
hipError_t sddmm_launch(const SddmmArgs& x, const SddmmShape& s, hipStream_t stream);
hipError_t sddmm_flat_launch(const SddmmArgs& x, const SddmmShape& s, int chunk, hipStream_t stream);
hipError_t sddmm_sliced_launch(const SddmmArgs& x, const SddmmShape& s, const SlicePlan& plan, void* workspace,
                               hipStream_t stream);

// K > 0: the height of Kmat and V is known and may count (operands beyond one L2 group long rows as under the even-rows hint)
FusedShape fused_choose(const DeviceInfo& dev, int M, int D, int nnz, bool vec4, int rows = kRowsUnknown, int K = 0);
hipError_t fused_launch(const FusedArgs& x, const FusedShape& s, hipStream_t stream);
hipError_t fused_flat_launch(const FusedArgs& x, const FusedShape& s, const FlatPlan& plan, float* partial,
                             hipStream_t stream);
hipError_t fused_sliced_launch(const FusedArgs& x, const FusedShape& s, const SlicePlan& plan, void* workspace,
                               hipStream_t stream);

// Picks (W, R), W <= max_w: waves per workgroup from the number of rows, rows per workgroup as large as keeps
// `blocks_per_cu` workgroups per compute unit in the grid. `slots` = nonzeros of a row a wave works on at once (64 / G); `more_waves_long_rows`:
// the op gains from more waves per row where rows are very long (SpMM only, see choose_split); `w8_few_rows_avg`: see below. `rows_even`: the caller knows that no
// row is much longer than the mean. Only the pairs the kernels are instantiated for are returned.
struct SplitRule {
    int blocks_per_cu;
    int max_w;
    int slots;
    bool more_waves_long_rows;
    int w8_few_rows_avg = 0;  // > 0: eight waves per row from this many nonzeros per row on where there are few rows
    int even_rows_avg = 128;  // rows known to be even are grouped four to a workgroup from this many nonzeros per row on
    int skewed_rows_cap = 4;  // rows per workgroup at most where long rows are known to lie next to each other
};
void choose_split(const DeviceInfo& dev, int M, long long col_tiles, int nnz, const SplitRule& rule, int rows, int& W, int& R);

// Row plan with cut rows ("cut plan"): rows longer than `longest_pct` per cent of a share (a share = the nonzeros of the
// matrix over the compute units) are cut into pieces of at most `piece_pct` per cent of a share, and the plan hands out
// `entries` = M + extra entries, each a whole row, a piece of a row, or nothing (no matrix can need more: see plan.hip).
// All offsets are bytes from the start of the plan's memory; the launches read the first 4 x entries ints (first
// nonzero, end, row, slot) and, SpMM and the fused op, the partial rows of the pieces and the list of cut rows.
constexpr int kCutPlanMaxRows = 1 << 20;  // a cut plan is built by one workgroup: not for taller matrices
// The rule (dlspm_tuning.cut_piece_pct / .cut_longest_pct override it): rows above one share in pieces of at most three
// quarters of a share. Against pieces of a share for rows above one and a half (every fourth of the 302 long-row files of
// the reference's data set, geometric means): SpMM at N = 256 4.95 -> 4.83 us, SDDMM at D = 128 3.54 -> 3.45 us, the fused
// op at D = 64 5.59 -> 5.62 us; 512 x 2048 with a row of 4.7 shares: SpMM 5.59 -> 5.18 us. Half a share (and 75 %): 4.90 /
// 3.54 / 5.68 us.
constexpr int kCutPiecePct = 75, kCutLongestPct = 100;
constexpr int kCutAdvicePct = 150;  // a cut plan is advised from a longest row of this many per cent of a share on
struct CutPlan {
    int entries;      // M + ceil(bins x 100 / piece_pct)
    int bins;         // compute units the plan was sized for (at most 256)
    int piece_pct, longest_pct;
    int slots;        // partial rows the plan has room for (more than the pieces of any matrix)
    int max_cut;      // rows that can be cut (ceil(bins x 100 / longest_pct): more than any matrix has above the limit)
    size_t off_keys;      // sort keys of the build (2 x entries 64-bit words; only beyond 2048 entries)
    size_t off_virtual;   // the rows and pieces in matrix order: entries + 1 offsets, entries rows, entries slots
    size_t off_cut;       // [0] number of cut rows, [1] share, [2] entries in use, [3] unused; then max_cut records of (row, first slot, pieces, in use)
    size_t off_pieces;    // slots x width floats
    size_t bytes;
};
CutPlan cut_plan_layout(int M, int width, int cus);
hipError_t cut_plan_build_launch(int M, const int* row_offsets, const CutPlan& cp, void* plan, int order, hipStream_t stream);
hipError_t cut_rows_sum_launch(int M, int width, const CutPlan& cp, const void* plan, float* out, hipStream_t stream);
hipError_t spmm_pieces_launch(const SpmmArgs& x, const SpmmShape& s, const CutPlan& cp, void* plan, hipStream_t stream);
bool spmm_cut_by_columns(const SpmmShape& s, int N);  // the pieces of a cut row share its columns: one kernel, no partial rows

// the same plan for the other two ops (16 < D <= 512, one row per four-wave workgroup)
// skewed (DLSPM_HINT_ROWS_SKEWED): the caller knows that the longest row is at least twenty times the mean
bool plan_ungroups_skewed(const DeviceInfo& dev, int M, int nnz);
bool sddmm_plan_applies(const DeviceInfo& dev, SddmmShape& s, int M, int D, int nnz, bool skewed = false);
bool sddmm_cut_plan_applies(const DeviceInfo& dev, SddmmShape& s, int M, int D, int nnz);  // also few rows of eight waves each
hipError_t sddmm_planned_launch(const SddmmArgs& x, const SddmmShape& s, const int* plan, hipStream_t stream);
bool fused_plan_applies(const DeviceInfo& dev, FusedShape& s, int M, int D, int nnz, bool skewed = false);
bool fused_cut_plan_applies(const DeviceInfo& dev, FusedShape& s, int M, int D, int nnz);  // ... of a launch with a cut plan (also few rows)
hipError_t fused_planned_launch(const FusedArgs& x, const FusedShape& s, const int* plan, hipStream_t stream);
// with a cut plan: SDDMM needs neither partial rows nor a second kernel (every piece writes its own CSR slots)
hipError_t sddmm_pieces_launch(const SddmmArgs& x, const SddmmShape& s, const CutPlan& cp, const void* plan, hipStream_t stream);
hipError_t fused_pieces_launch(const FusedArgs& x, const FusedShape& s, const CutPlan& cp, void* plan, hipStream_t stream);

}  // namespace dlspm
