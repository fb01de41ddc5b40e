// CSR-sampled SDDMM, out[j] = <lhs[i, :], rhs[col[j], :]> for every slot j of CSR row i, fp32, gfx950.
//
// Computes what the reference's CPU loop Sddmm (SDDMM/sddmm-esimd-fromfile.cpp:18-36) computes and
// takes the place of its ESIMD kernels (SDDMM/sddmm-esimd-fromfile.hpp:59-131 and the small-K variant
// SDDMM/sddmm-esimd-fromfile_v4.hpp:102-177, which adds partial dot products with float atomics).
// Here:
//   * a workgroup of W waves owns R consecutive rows and splits their nonzeros evenly over its waves;
//   * a wave keeps the lhs row of its current segment in registers (DS accesses of VEC floats per
//     lane), reads 64 column indices with one coalesced load, and works on 64/G1 nonzeros at a time:
//     G1 lanes read one rhs row (a full 128-byte line per group and access when G1 = 8, VEC = 4),
//     multiply, and reduce with DPP inside their 16-lane row;
//   * after up to G1 such rounds every lane holds one finished dot product; one ds_bpermute puts them
//     in CSR order and one coalesced store writes 64 results straight into the sampled slots.
// Every slot is written exactly once and no atomics are used, so the output needs no zeroing and is
// deterministic. The CSR index arrays are only read.
#include "common.hpp"
#include "launch.hpp"

namespace dlspm {

// Where the results go. Results of more than one and a half times what one L2 holds (6 MiB on an MI355X) are stored with
// the non-temporal hint: ordinary stores are held in the L2 as dirty lines and written back later, hinted ones drain as
// they are issued. (The L2's hit rate and the bytes fetched do not change by it; the time does.) Measured with both
// kinds of store in one process, D = 32 / 128: 24576 x 8192 at density 0.3 (230 MiB of results) 443 -> 297 us /
// 1287 -> 1089 us; 8192 x 2048 at 0.3 (19 MiB) 32.5 -> 28.1 us / 90.6 -> 88.3 us; 6144 x 2048 at 0.2 (9.6 MiB) -3.5 % /
// -4.4 %; 6.4 MiB -1.2 % / -1.8 %; 4.8 MiB +0.4 ... +2.2 % / equal. Small results lose by the hint -- neighbouring waves
// share cache lines here, and a kernel ends when its stores have reached memory -- (2048 x 2048 at 5 %, 0.8 MiB: +8 % /
// +4 %) and keep ordinary stores.
struct SampledOut {
    float* __restrict__ at;
    int streaming;
    __device__ __forceinline__ void store(int j, float v) const
    {
        // (wave-uniform) The hinted store is written out as an instruction: __builtin_nontemporal_store on one side of
        // this branch and a plain store on the other are merged into one store by the compiler, and the hint is lost.
        // (A vector store like any other; the wait counts that the compiler inserts can only become stricter by it.)
        if (streaming) asm volatile("global_store_dword %0, %1, off nt" : : "v"(at + j), "v"(v) : "memory");
        else at[j] = v;
    }
};
static inline SampledOut sampled_out(const SddmmArgs& x)
{
    const int forced = tuning().stream_results;  // -1: the size rule (sweeps and tests switch it off or on)
    const long long l2 = x.l2_bytes;
    const bool by_rule = (long long)x.nnz * (long long)sizeof(float) > l2 + l2 / 2;
    return SampledOut{x.out, (forced < 0 ? by_rule : forced != 0) ? 1 : 0};
}

// out[j] = <lhs_row, rhs[col_indices[j]]> for the nonzeros j in [p, q) of one row (p < q, wave-uniform).
template <int VEC, int G1, int DS, int MASKED>
__device__ __forceinline__ void sddmm_segment(int p, int q, int D, const int* __restrict__ col_indices,
                                              const float* __restrict__ lhs_row, const float* __restrict__ rhs,
                                              SampledOut out, int lane)
{
    using VecT = Vec<VEC>;
    const int g = lane % G1;
    VecT lq[DS > 0 ? DS : 1];
    if constexpr (DS > 0) {
#pragma unroll
        for (int s = 0; s < DS; ++s) {
            const int d = (s * G1 + g) * VEC;
            if constexpr (MASKED) lq[s] = d < D ? VecT::gload_clip(lhs_row, d, D) : VecT::zero();
            else lq[s] = VecT::gload(lhs_row + d);
        }
    }
    // 64 column indices per pass, one per lane; the next 64 are requested (index clamped, no condition) before
    // the rhs rows of the current ones
    int c_nxt = col_indices[min(p + lane, q - 1)];
    for (int base = p; base < q; base += kWave) {
        const int c = base + lane < q ? c_nxt : 0;
        c_nxt = col_indices[min(base + kWave + lane, q - 1)];
        const int cnt = min(kWave, q - base);
        const float o = sddmm_chunk<VEC, G1, DS, MASKED>(D, lane, cnt, c, lhs_row, lq, rhs);
        if (base + lane < q) out.store(base + lane, o);
    }
}

// The same for one row shared by the W waves of a workgroup: the row is gone through in passes of `chunk` nonzeros, wave w
// taking the passes w, w + W, ... -- so that the waves go through the row's (ascending) columns together, and so that no
// wave is left with a nearly empty pass of its own (an even split of 300 nonzeros over four waves is 64 + 11 each: two
// passes; here it is two passes of 40). `chunk` is the row's length over the fewest passes per wave that passes of 64
// would need, rounded up to the eight nonzeros a wave works on at once: all waves get the same number of rounds.
// Every result is one nonzero's own dot product, so which wave computes it changes no bit.
// Measured (D = 128, in a graph, even split -> this): lognormal rows with a row plan, 2048 x 2048 8.6 -> 7.9 us, 16384 x 4096
// 39.4 -> 32.9 us; 2048 x 512 with 51 per row 4.95 -> 4.16 us.
template <int VEC, int G1, int DS, int MASKED>
__device__ __forceinline__ void sddmm_row_interleaved(int p, int q, int w, int W, int D, const int* __restrict__ col_indices,
                                                      const float* __restrict__ lhs_row, const float* __restrict__ rhs,
                                                      SampledOut out, int lane, bool full_passes)
{
    using VecT = Vec<VEC>;
    constexpr int kRound = kWave / G1;  // nonzeros a wave works on at once
    const int T = q - p;
    if (T <= 0) return;
    int chunk = kWave;
    if (!full_passes) {
        const int passes = (T + W * kWave - 1) / (W * kWave);  // per wave
        chunk = min(kWave, ((T + W * passes - 1) / (W * passes) + kRound - 1) / kRound * kRound);
    }
    if (p + w * chunk >= q) return;
    const int g = lane % G1;
    VecT lq[DS > 0 ? DS : 1];
    if constexpr (DS > 0) {
#pragma unroll
        for (int s = 0; s < DS; ++s) {
            const int d = (s * G1 + g) * VEC;
            if constexpr (MASKED) lq[s] = d < D ? VecT::gload_clip(lhs_row, d, D) : VecT::zero();
            else lq[s] = VecT::gload(lhs_row + d);
        }
    }
    int c_nxt = col_indices[min(p + w * chunk + lane, q - 1)];
    for (int base = p + w * chunk; base < q; base += W * chunk) {
        const int cnt = min(chunk, q - base);
        const int c = lane < cnt ? c_nxt : 0;
        c_nxt = col_indices[min(base + W * chunk + lane, q - 1)];
        const float o = sddmm_chunk<VEC, G1, DS, MASKED>(D, lane, cnt, c, lhs_row, lq, rhs);
        if (lane < cnt) out.store(base + lane, o);
    }
}

// The work of workgroup `bid` (RowBlock in common.hpp explains SLICED and PLANNED; a segment's results go where its
// nonzeros lie, so a sliced or planned launch writes the same slots as any other). This kernel has neither LDS nor a
// barrier.
template <int VEC, int G1, int DS, int MASKED, int W, int R, bool SLICED, int PLANNED = kPlanNone>
__device__ __forceinline__ void sddmm_block(int bid, int M, int D, const int* __restrict__ row_offsets,
                                            const int* __restrict__ row_ends, const int* __restrict__ col_indices,
                                            const float* __restrict__ lhs, const float* __restrict__ rhs,
                                            SampledOut out, const int* __restrict__ row_ids = nullptr, int nnz = 0,
                                            int flags = 0, const int* __restrict__ row_slots = nullptr, int slots = 0)
{
    RowBlock<W, R, SLICED, PLANNED> blk;
    const int lg = !SLICED && !PLANNED && R == 1 && W > 1 ? (flags >> kFlagPiecesShift) & kFlagPiecesMask : 0;
    blk.load(bid >> lg, M, nnz, row_offsets, row_ends, row_ids, [&]() { fetch_args_now(col_indices, lhs, rhs, out.at); }, flags,
             row_slots, slots);
    if constexpr (R == 1 && W > 1) {
        const int first = blk.T0 + blk.shift(0);
        int w = blk.w, waves = W;
        if constexpr (!SLICED && !PLANNED) {  // 2^lg workgroups share the row: their waves take its passes in turn like one workgroup's
            w += (bid & ((1 << lg) - 1)) * W;
            waves = W << lg;
        }
        sddmm_row_interleaved<VEC, G1, DS, MASKED>(first, first + blk.T, w, waves, D, col_indices, lhs + (size_t)blk.row0 * D, rhs,
                                                   out, blk.lane, (flags & kFlagFullPasses) != 0);
    } else {
        blk.for_each_segment([&](int r, int p, int q, int, int) {
            const float* lhs_row = lhs + (size_t)(blk.row0 + r) * D;
            const int shift = blk.shift(r);
            sddmm_segment<VEC, G1, DS, MASKED>(p + shift, q + shift, D, col_indices, lhs_row, rhs, out, blk.lane);
        });
    }
}

// Five and more accesses per lane and row of rhs (D = 129 ... 512): the compiler, aiming at eight waves per SIMD and their 64
// registers, would issue the accesses of a round two or three at a time and wait for each group; told that four waves
// per SIMD are enough (three from twelve accesses on), it issues all of them before the first wait (D = 256: 78 registers,
// six waves per SIMD; D = 384: 110; D = 512: four waves). In a graph, before -> after:
// D = 256, Bernoulli rows 1024 x 2304 12.3 -> 10.7 us, 8192 x 2048 21.5 -> 20.5 us, lognormal rows 1024 x 2304 44.2 -> 26.0 us,
// 4096 x 4096 120 -> 70 us; one row per workgroup on rows of 100 nonzeros loses 6-10 % (2048 x 512 under a row plan 9.5 ->
// 10.4 us). D = 512: lognormal rows 0.58-1.03 of the time (0.84 in the mean), Bernoulli rows 0.92-1.12 (0.99; 4096 x 4096 of
// 200 per row, rhs of twice the L2, 81 -> 91 us). D = 384 with twelve accesses at the compiler's own choice took longer
// than D = 512 where rhs exceeds the L2 (512 x 4608 of 1380 per row: 69 against 57 us; with all twelve in flight 39 us).
// (W: waves per workgroup. The least number of waves per SIMD that the attribute names must not be below what one workgroup
// puts there, or the compiler drops the attribute -- eight-wave workgroups, lognormal rows on 448 rows, D = 256 ... 512: 12-19 %
// faster with it kept --; and the largest not below the least.)
#define DLSPM_SDDMM_WAVES_PER_SIMD(DS, W) \
    __attribute__((amdgpu_waves_per_eu(waves_per_simd_least(W), waves_per_simd_most(W, (DS) > 4 && (DS) <= 8 ? 4 : (DS) >= 12 ? 3 : 8))))

// MASKED = false: D == G1 * VEC * DS exactly, every access of every lane falls inside the row.
template <int VEC, int G1, int DS, int MASKED, int W, int R>
__global__ __launch_bounds__(W * 64) DLSPM_SDDMM_WAVES_PER_SIMD(DS, W) void sddmm_kernel(int M, int D, int flags, const int* __restrict__ row_offsets,
                                                       const int* __restrict__ col_indices,
                                                       const float* __restrict__ lhs, const float* __restrict__ rhs,
                                                       SampledOut out)
{
    sddmm_block<VEC, G1, DS, MASKED, W, R, false>((int)blockIdx.x, M, D, row_offsets, nullptr, col_indices, lhs, rhs, out,
                                                  nullptr, 0, flags);
}

// Column-sliced schedule (see spmm_sliced_kernel): the row blocks once per slice of columns, slice after slice, so that
// the rows of rhs gathered at any time come from one slice. Every result still goes to its own CSR slot: no partial
// rows, no second pass, and the same bits as under any other schedule.
template <int VEC, int G1, int DS, int MASKED, int R>
__global__ __launch_bounds__(4 * 64) DLSPM_SDDMM_WAVES_PER_SIMD(DS, 4) void sddmm_sliced_kernel(int M, int D, int slice_blocks,
                                                              const int* __restrict__ bounds,
                                                              const int* __restrict__ col_indices,
                                                              const float* __restrict__ lhs,
                                                              const float* __restrict__ rhs, SampledOut out)
{
    const int sl = (int)(blockIdx.x / (unsigned)slice_blocks);
    const int bid = (int)blockIdx.x - sl * slice_blocks;
    sddmm_block<VEC, G1, DS, MASKED, 4, R, true>(bid, M, D, bounds + (size_t)sl * M, bounds + (size_t)(sl + 1) * M,
                                                 col_indices, lhs, rhs, out);
}

// ---- host side --------------------------------------------------------------------------------------

// Row plan: workgroup i works on the whole row rows[i] = [starts[i], ends[i]) (one row per four-wave workgroup).
template <int VEC, int G1, int DS, int MASKED>
__global__ __launch_bounds__(4 * 64) DLSPM_SDDMM_WAVES_PER_SIMD(DS, 4) void sddmm_planned_kernel(int M, int D, int nnz, int flags, const int* __restrict__ starts,
                                                               const int* __restrict__ ends, const int* __restrict__ rows,
                                                               const int* __restrict__ col_indices,
                                                               const float* __restrict__ lhs, const float* __restrict__ rhs,
                                                               SampledOut out)
{
    sddmm_block<VEC, G1, DS, MASKED, 4, 1, true, kPlanRows>((int)blockIdx.x, M, D, starts, ends, col_indices, lhs, rhs, out, rows,
                                                            nnz, flags);
}

// Row plan with cut rows: entry i is a whole row (slot_of[i] == -1), a piece of one -- entered with its row's whole range,
// slot_of[i] says which piece of how many: that share of the row's nonzeros, whose results go to their own CSR slots like
// any others -- or nothing (an empty range).
template <int VEC, int G1, int DS, int MASKED>
__global__ __launch_bounds__(4 * 64) DLSPM_SDDMM_WAVES_PER_SIMD(DS, 4) void sddmm_pieces_kernel(int M, int D, int nnz, int flags, int slots, const int* __restrict__ starts,
                                                              const int* __restrict__ ends, const int* __restrict__ rows,
                                                              const int* __restrict__ slot_of,
                                                              const int* __restrict__ col_indices,
                                                              const float* __restrict__ lhs, const float* __restrict__ rhs,
                                                              SampledOut out)
{
    sddmm_block<VEC, G1, DS, MASKED, 4, 1, true, kPlanPieces>((int)blockIdx.x, M, D, starts, ends, col_indices, lhs, rhs, out, rows,
                                                              nnz, flags, slot_of, slots);
}

// Whole passes of 64 in turn where the device has rows to spare (from two rows per compute unit on: fewer waves at work per
// row, each with a full pass -- lognormal rows 8-17 % faster than passes sized to occupy all waves); below that every wave
// of a row gets its share (64 x 576 with 400 per row: 0.95 of the time against 1.05).
static int sddmm_flags(const SddmmArgs& x, long long entries)
{
    return launch_flags(x.xcd_contiguous) | (entries >= 2ll * x.cus ? kFlagFullPasses : 0);
}

// Whether the kernels that mask by the range of a buffer apply (sddmm_rounds_load): D a multiple of four, rhs within the
// window. Against the kernels that mask by selects (Bernoulli / lognormal rows, 20 shapes of 128 ... 16384 rows, geometric
// means): D = 80 0.96 / 0.92 of the time, D = 100 0.89 / 0.80, D = 160 0.95 / 0.91, D = 224 0.94 / 0.90, D = 320 0.90 / 0.88; with
// sixteen accesses (D = 400 ... 496, twelve shapes, plain calls and planned ones) 0.78-0.82 and 0.75-0.77, 0.58 ... 1.13: the
// select kernel needs 172 registers there, two waves per SIMD, the range kernel 122. The fused op's kernels mask by
// selects at every width.
template <int DS> static bool masked_by_range(int K, int D)
{
    return DS >= 1 && DS <= 16 && D % 4 == 0 && K < (1 << 24) &&
           (long long)K * D * (long long)sizeof(float) <= (long long)kRangeWindowBytes && rule_on(kRuleMaskByRange);
}
// (the kind to instantiate: no range kernels for the run-time loop of D > 512)
template <int DS> constexpr int masked_kind(bool by_range) { return by_range && DS >= 1 && DS <= 16 ? kMaskedByRange : kMaskedBySelect; }

template <int VEC, int G1, int DS, int W, int R>
static hipError_t launch_one(const SddmmArgs& x, int pieces_lg, hipStream_t stream)
{
    if (R != 1 || W == 1) pieces_lg = 0;
    const int blocks = (int)ceil_div(x.M, R) << pieces_lg;
    if (blocks <= 0) return hipSuccess;
    // (row pieces: the workgroups of a row must stay neighbours, so no XCD-contiguous runs of row blocks)
    const int flags = pieces_lg > 0 ? (sddmm_flags(x, x.M) & ~kFlagXcdContiguous) | (pieces_lg << kFlagPiecesShift) : sddmm_flags(x, x.M);
    if constexpr (DS > 0) {
        if (x.D == G1 * VEC * DS && rule_on(kRuleExactWidthKernels)) {
            hipLaunchKernelGGL((sddmm_kernel<VEC, G1, DS, kExactWidth, W, R>), dim3(blocks), dim3(W * 64), 0, stream, x.M,
                               x.D, flags, x.row_offsets, x.col_indices, x.lhs, x.rhs, sampled_out(x));
            return hipGetLastError();
        }
    }
    if constexpr (VEC == 4 && G1 == 8 && DS >= 1 && DS <= 16) {
        if (masked_by_range<DS>(x.K, x.D)) {
            hipLaunchKernelGGL((sddmm_kernel<VEC, G1, DS, kMaskedByRange, W, R>), dim3(blocks), dim3(W * 64), 0, stream, x.M, x.D,
                               flags, x.row_offsets, x.col_indices, x.lhs, x.rhs, sampled_out(x));
            return hipGetLastError();
        }
    }
    hipLaunchKernelGGL((sddmm_kernel<VEC, G1, DS, kMaskedBySelect, W, R>), dim3(blocks), dim3(W * 64), 0, stream, x.M, x.D,
                       flags, x.row_offsets, x.col_indices, x.lhs, x.rhs, sampled_out(x));
    return hipGetLastError();
}

// the layout of shape s among SddmmLayouts
template <typename Launch> static hipError_t dispatch_layout(const SddmmShape& s, Launch&& launch)
{
    return dispatch<SddmmLayouts>([&](auto l) { return l.VEC == s.vec && l.G1 == s.G1 && l.DS == s.DS; }, launch);
}

SddmmShape sddmm_choose(const DeviceInfo& dev, int M, int D, int nnz, bool vec4, int rows)
{
    SddmmShape s{};
    s.vec = vec4 ? 4 : 1;
    if (vec4) {
        if (D <= 16) { s.G1 = 4; s.DS = 1; }
        else {
            s.G1 = 8;
            // accesses of 32 floats per dot product: powers of two and the steps half-way between them (an access
            // that lies past D is issued like the others)
            s.DS = D <= 32 ? 1 : D <= 64 ? 2 : D <= 96 ? 3 : D <= 128 ? 4 : D <= 192 ? 6 : D <= 256 ? 8 : D <= 384 ? 12 : D <= 512 ? 16 : 0;
        }
    } else {  // D < 4: one float per lane
        s.G1 = 4;
        s.DS = 1;
    }
    choose_split(dev, M, 1, nnz, SplitRule{2, 16, kWave / s.G1, false, 96}, rows, s.W, s.R);
    // Rows of unknown lengths are grouped only where the launch is many times what the device holds at once: from 128
    // rows per compute unit on, and from 64 at D <= 32. Below that one row per workgroup, whose four waves take the row's passes
    // in turn, is the shorter way through the launch even where three of the four waves find nothing to do (rows per
    // workgroup by the size rule against one, K = 2048, rows of 8 ... 128 nonzeros, D = 32 / 64 / 128 / 256, geometric means:
    // Bernoulli rows 1.01 / 1.12 / 1.09 / 1.03 of the time, lognormal rows 1.21 / 1.21 / 1.13 / 1.05, up to 1.9; 2048 x 2048
    // of 8 per row, D = 64: 3.42 -> 2.78 us; 8192 x 2048 of 16, lognormal, D = 64: 7.68 -> 4.76 us. At 32768 rows the groups
    // win 5-30 % on Bernoulli rows and at D = 32, at 16384 rows at D = 32 only: 16384 x 2048 of 32 per row 6.4 against 8.7 us.)
    // Rows known to be even keep their groups of four -- one whole row per wave -- where rows and dot products are long (128
    // nonzeros, 128 floats: 0.91-1.03 of the time of one row per workgroup at 2048 ... 8192 rows), and lose the others
    // (Bernoulli rows of 8 ... 64 nonzeros on 1024 ... 8192 rows, the hint's groups against none: 1.05-1.31 of the time).
    const bool many_rows = (long long)M >= 128ll * dev.cus || ((long long)M >= 64ll * dev.cus && D <= 32);
    const bool even_long_rows = rows == kRowsEven && (long long)nnz >= 128ll * M && D >= 128;
    if (s.R > 1 && tuning().split_w == 0 && !many_rows && !even_long_rows) s.R = 1;
    return s;
}

// Few rows in a call without plan or memory: 2^lg four-wave workgroups share each row, so that the device gets two
// workgroups per compute unit where one row per workgroup -- with eight waves -- leaves most of it idle. Their waves take the
// row's passes in turn exactly as the waves of one workgroup do (sddmm_row_interleaved), every result is still one
// nonzero's own dot product, and nothing else changes: no plan, no second kernel, the same bits. Up to three quarters of
// a compute unit's count of rows, rows of 128 nonzeros and more on average, and a workgroup keeps at least 32 of a mean row.
// Measured (us inside a graph, rule off / on / with a cut plan; Bernoulli rows, geometric means over four shapes of 230 ...
// 1380 nonzeros per row): D = 128: 16 rows 4.04 / 2.60 / 2.63, 64 rows 4.14 / 3.09 / 3.08, 128 rows 4.22 / 3.69 / 3.65,
// 192 rows 4.30 / 4.49 / 4.43; D = 256: 5.81 / 3.00 / 2.83, 6.38 / 3.91 / 4.07, 6.45 / 5.05 / 5.07, 6.48 / 6.47 / 6.63;
// lognormal rows (sigma 0.8), D = 128: 6.36 / 2.84 / 2.64, 7.60 / 3.72 / 3.16, 8.05 / 4.84 / 3.72, 8.14 / 5.83 / 4.27
// (a cut plan still cuts the longest rows finer); the reference's 128-row ResNet-50 layers (26 files): 3.80 / 3.28 / 3.31.
// Between three quarters and one and a half of a compute unit's count of rows two four-wave workgroups share a row, which
// fills the device evenly where one eight-wave workgroup per row leaves the last compute units with one row and the
// others with two (four workgroups per row lose 3 ... 23 % on Bernoulli rows there): 256 rows, D = 128, 4.61 / 4.74 / 5.20 and
// lognormal 8.76 / 7.82 / 4.94; 384 rows 6.54 / 5.95 / 6.17 and 11.37 / 9.06 / 6.09; D = 256: 1.02 and 0.86 of the time, lognormal 0.86 and 0.78.
void sddmm_few_rows_pieces(const DeviceInfo& dev, SddmmShape& s, int M, int nnz)
{
    s.pieces_lg = 0;
    if (!rule_on(kRuleRowPiecesFewRows) || s.R != 1 || s.W == 1 || tuning().split_w > 0 || M <= 0) return;
    if (2ll * M > 3ll * dev.cus || (long long)nnz < 128ll * M) return;
    int lg = 0;
    while (lg < kFlagPiecesMask && ((long long)M << lg) < 2ll * dev.cus && (long long)nnz >= (64ll << lg) * M) ++lg;
    if (4ll * M > 3ll * dev.cus) lg = 1;
    if (lg == 0) return;
    s.pieces_lg = lg;
    s.W = 4;
}

hipError_t sddmm_launch(const SddmmArgs& x, const SddmmShape& s, hipStream_t stream)
{
    return dispatch_layout(s, [&](auto l) {
        using L = decltype(l);
        return dispatch_split(s.W, s.R, [&](auto split) {
            using S = decltype(split);
            return launch_one<L::VEC, L::G1, L::DS, S::W, S::R>(x, s.pieces_lg, stream);
        });
    });
}

// ---- flat schedule: every wave owns `chunk` consecutive nonzeros of the mask, whatever rows they belong to ---------
// (see spmm.hip; here every result goes to its own CSR slot, so there is nothing to combine and no workspace)
template <int VEC, int G1, int DS, int MASKED>
__global__ __launch_bounds__(kFlatWaves * 64) DLSPM_SDDMM_WAVES_PER_SIMD(DS, kFlatWaves) void sddmm_flat_kernel(int M, int D, int nnz, int chunk,
                                                                      const int* __restrict__ row_offsets,
                                                                      const int* __restrict__ col_indices,
                                                                      const float* __restrict__ lhs,
                                                                      const float* __restrict__ rhs, SampledOut out)
{
    fetch_args_now(row_offsets, col_indices, lhs, rhs, out.at);
    const int lane = threadIdx.x & 63;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const long long a64 = ((long long)blockIdx.x * kFlatWaves + w) * chunk;
    if (a64 >= nnz) return;  // wave-uniform
    const int a = (int)a64;
    const int b = (int)min((long long)nnz, a64 + chunk);
    int r = find_row(row_offsets, M, a, lane);
    int rbase = r;
    int win = window_load(row_offsets, M, rbase, lane);
    int pos = a;
    while (true) {
        if (r - rbase >= kWinRows) {
            rbase = r;
            win = window_load(row_offsets, M, rbase, lane);
        }
        const int re = window_get(win, r - rbase + 1);
        const int q = min(re, b);
        sddmm_segment<VEC, G1, DS, MASKED>(pos, q, D, col_indices, lhs + (size_t)r * D, rhs, out, lane);
        pos = q;
        if (pos >= b) break;
        r = window_next_row(row_offsets, M, pos, lane, win, rbase);
    }
}

template <int VEC, int G1, int DS>
static hipError_t launch_flat(const SddmmArgs& x, int chunk, hipStream_t stream)
{
    const long long units = ((long long)x.nnz + chunk - 1) / chunk;
    const unsigned blocks = (unsigned)((units + kFlatWaves - 1) / kFlatWaves);
    if constexpr (DS > 0) {
        if (x.D == G1 * VEC * DS && rule_on(kRuleExactWidthKernels)) {
            hipLaunchKernelGGL((sddmm_flat_kernel<VEC, G1, DS, kExactWidth>), dim3(blocks), dim3(kFlatWaves * 64), 0, stream, x.M,
                               x.D, x.nnz, chunk, x.row_offsets, x.col_indices, x.lhs, x.rhs, sampled_out(x));
            return hipGetLastError();
        }
    }
    if constexpr (VEC == 4 && G1 == 8 && DS >= 1 && DS <= 16) {
        if (masked_by_range<DS>(x.K, x.D)) {
            hipLaunchKernelGGL((sddmm_flat_kernel<VEC, G1, DS, kMaskedByRange>), dim3(blocks), dim3(kFlatWaves * 64), 0, stream, x.M,
                               x.D, x.nnz, chunk, x.row_offsets, x.col_indices, x.lhs, x.rhs, sampled_out(x));
            return hipGetLastError();
        }
    }
    hipLaunchKernelGGL((sddmm_flat_kernel<VEC, G1, DS, kMaskedBySelect>), dim3(blocks), dim3(kFlatWaves * 64), 0, stream, x.M, x.D,
                       x.nnz, chunk, x.row_offsets, x.col_indices, x.lhs, x.rhs, sampled_out(x));
    return hipGetLastError();
}

hipError_t sddmm_flat_launch(const SddmmArgs& x, const SddmmShape& s, int chunk, hipStream_t stream)
{
    return dispatch_layout(s, [&](auto l) {
        using L = decltype(l);
        return launch_flat<L::VEC, L::G1, L::DS>(x, chunk, stream);
    });
}

// ---- column-sliced schedule ------------------------------------------------------------------------

template <int VEC, int G1, int DS, int R>
static hipError_t launch_sliced_r(const SddmmArgs& x, const SlicePlan& plan, const int* bounds, hipStream_t stream)
{
    const long long slice_blocks = ceil_div(x.M, R);
    const long long blocks = slice_blocks * plan.slices;
    if (blocks <= 0) return hipSuccess;
    if (blocks > 0x7fffffffLL) return hipErrorInvalidConfiguration;
    if (x.D == G1 * VEC * DS)
        hipLaunchKernelGGL((sddmm_sliced_kernel<VEC, G1, DS, kExactWidth, R>), dim3((unsigned)blocks), dim3(4 * 64), 0, stream,
                           x.M, x.D, (int)slice_blocks, bounds, x.col_indices, x.lhs, x.rhs, sampled_out(x));
    else if (masked_by_range<DS>(x.K, x.D))
        hipLaunchKernelGGL((sddmm_sliced_kernel<VEC, G1, DS, masked_kind<DS>(true), R>), dim3((unsigned)blocks), dim3(4 * 64), 0, stream,
                           x.M, x.D, (int)slice_blocks, bounds, x.col_indices, x.lhs, x.rhs, sampled_out(x));
    else
        hipLaunchKernelGGL((sddmm_sliced_kernel<VEC, G1, DS, kMaskedBySelect, R>), dim3((unsigned)blocks), dim3(4 * 64), 0, stream,
                           x.M, x.D, (int)slice_blocks, bounds, x.col_indices, x.lhs, x.rhs, sampled_out(x));
    return hipGetLastError();
}

template <int VEC, int G1, int DS>
static hipError_t launch_sliced(const SddmmArgs& x, const SlicePlan& plan, const int* bounds, hipStream_t stream)
{
    return dispatch_sliced_rows(plan.R, [&](auto r) { return launch_sliced_r<VEC, G1, DS, decltype(r)::R>(x, plan, bounds, stream); });
}

// built for 16 < D <= 512 (G1 = 8 with 1 to 16 accesses per lane)
hipError_t sddmm_sliced_launch(const SddmmArgs& x, const SddmmShape& s, const SlicePlan& plan, void* workspace,
                               hipStream_t stream)
{
    int* bounds = static_cast<int*>(workspace);
    const hipError_t e = slice_bounds_launch(x.M, x.K, plan.slices, x.row_offsets, x.col_indices, bounds, stream);
    if (e != hipSuccess) return e;
    return dispatch_layout(s, [&](auto l) {
        using L = decltype(l);
        if constexpr (L::VEC == 4 && L::G1 == 8 && L::DS >= 1) return launch_sliced<4, 8, L::DS>(x, plan, bounds, stream);
        else return hipErrorInvalidValue;
    });
}

// ---- row plan ---------------------------------------------------------------------------------------

bool sddmm_plan_applies(const DeviceInfo& dev, SddmmShape& s, int M, int D, int nnz, bool skewed)
{
    if (s.vec != 4 || s.G1 != 8 || s.DS < 1 || s.W != 4) return false;  // built for 16 < D <= 512
    if (s.R == 1) return true;
    if (!plan_ungroups_dots(dev, M, D, nnz) && !(skewed && plan_ungroups_skewed(dev, M, nnz))) return false;
    s.R = 1;
    return true;
}

// `entries` workgroups: M for a plan over whole rows; a cut plan's M + bins, each a row, a piece of a row (its results go
// to its own CSR slots like any others: no partial rows, no second kernel, the same bits) or nothing (first nonzero ==
// end, which writes nothing)
// A cut plan also serves masks of fewer rows than compute units, which the size rule runs with eight waves per row and
// which a plan over whole rows cannot help (every row has a compute unit to itself, half of the device idles): cut, the
// pieces of the rows fill the device, at no cost to SDDMM, whose pieces write their own CSR slots. Measured on the
// reference's ResNet-50 layers of 64 and 128 rows (36 ... 900 nonzeros per row, D = 128, in a graph): 0.74 ... 0.93 of the
// time (64 x 576 with 499 per row: 4.30 -> 3.20 us; 128 x 1152 with 231: 3.78 -> 3.15 us); with 256 rows 0.93 ... 1.06 on
// those layers, whose longest rows hold two to three shares, and 0.66 where one holds three and a half (256 x 2304,
// lognormal rows of 200 on average): from as many rows as compute units on, the advice asks for a longer row.
bool sddmm_cut_plan_applies(const DeviceInfo& dev, SddmmShape& s, int M, int D, int nnz)
{
    if (s.vec == 4 && s.G1 == 8 && s.DS >= 1 && s.W == 8 && M < 2 * dev.cus) {
        s.W = 4;
        s.R = 1;
        return true;
    }
    return sddmm_plan_applies(dev, s, M, D, nnz);
}

template <int DS>
static hipError_t launch_planned(const SddmmArgs& x, const int* plan, int entries, int slots, hipStream_t stream)
{
    const int *starts = plan, *ends = plan + entries, *rows = plan + 2 * (size_t)entries, *slot_of = plan + 3 * (size_t)entries;
    const bool by_range = masked_by_range<DS>(x.K, x.D);
    if (slots > 0) {  // a cut plan
        if (x.D == 8 * 4 * DS)
            hipLaunchKernelGGL((sddmm_pieces_kernel<4, 8, DS, kExactWidth>), dim3((unsigned)entries), dim3(4 * 64), 0, stream, x.M, x.D,
                               x.nnz, sddmm_flags(x, x.M), slots, starts, ends, rows, slot_of, x.col_indices, x.lhs, x.rhs, sampled_out(x));
        else if (by_range)
            hipLaunchKernelGGL((sddmm_pieces_kernel<4, 8, DS, masked_kind<DS>(true)>), dim3((unsigned)entries), dim3(4 * 64), 0, stream, x.M, x.D,
                               x.nnz, sddmm_flags(x, x.M), slots, starts, ends, rows, slot_of, x.col_indices, x.lhs, x.rhs, sampled_out(x));
        else
            hipLaunchKernelGGL((sddmm_pieces_kernel<4, 8, DS, kMaskedBySelect>), dim3((unsigned)entries), dim3(4 * 64), 0, stream, x.M, x.D,
                               x.nnz, sddmm_flags(x, x.M), slots, starts, ends, rows, slot_of, x.col_indices, x.lhs, x.rhs, sampled_out(x));
        return hipGetLastError();
    }
    if (x.D == 8 * 4 * DS)
        hipLaunchKernelGGL((sddmm_planned_kernel<4, 8, DS, kExactWidth>), dim3((unsigned)entries), dim3(4 * 64), 0, stream, x.M, x.D,
                           x.nnz, sddmm_flags(x, x.M), starts, ends, rows, x.col_indices, x.lhs, x.rhs, sampled_out(x));
    else if (by_range)
        hipLaunchKernelGGL((sddmm_planned_kernel<4, 8, DS, masked_kind<DS>(true)>), dim3((unsigned)entries), dim3(4 * 64), 0, stream, x.M, x.D,
                           x.nnz, sddmm_flags(x, x.M), starts, ends, rows, x.col_indices, x.lhs, x.rhs, sampled_out(x));
    else
        hipLaunchKernelGGL((sddmm_planned_kernel<4, 8, DS, kMaskedBySelect>), dim3((unsigned)entries), dim3(4 * 64), 0, stream, x.M, x.D,
                           x.nnz, sddmm_flags(x, x.M), starts, ends, rows, x.col_indices, x.lhs, x.rhs, sampled_out(x));
    return hipGetLastError();
}

static hipError_t launch_planned_ds(const SddmmArgs& x, const SddmmShape& s, const int* plan, int entries, int slots,
                                    hipStream_t stream)
{
    if (x.M <= 0) return hipSuccess;
    return dispatch_layout(s, [&](auto l) {
        using L = decltype(l);
        if constexpr (L::VEC == 4 && L::G1 == 8 && L::DS >= 1) return launch_planned<L::DS>(x, plan, entries, slots, stream);
        else return hipErrorInvalidValue;
    });
}

hipError_t sddmm_planned_launch(const SddmmArgs& x, const SddmmShape& s, const int* plan, hipStream_t stream)
{
    return launch_planned_ds(x, s, plan, x.M, 0, stream);
}

hipError_t sddmm_pieces_launch(const SddmmArgs& x, const SddmmShape& s, const CutPlan& cp, const void* plan, hipStream_t stream)
{
    return launch_planned_ds(x, s, static_cast<const int*>(plan), cp.entries, cp.slots, stream);
}

}  // namespace dlspm
