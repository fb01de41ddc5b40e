// Fused SDDMM -> SpMM, O[M x D] = (S .* (Q * Kmat^T) * scale) * V with S given as a CSR pattern, fp32, gfx950.
//
// Computes what Sddmm followed by Spmm compute in the reference's FUSED/fused.cpp:47-89 (with scale = 1)
// and takes the place of its ESIMD kernel FusedEsimd (FUSED/fused-esimd_cb.cpp:100-189), which handles
// one row per hardware thread and keeps 32 scores in a register vector between its two inner loops.
// Here, per chunk of up to 64 nonzeros of a row segment:
//   stage 1  the wave computes the 64 sampled scores exactly as the SDDMM kernel does (G1 lanes per dot
//            product, DPP reduction, one transpose) and multiplies them by `scale`: lane l then holds the
//            score and the column index of nonzero l in registers;
//   stage 2  the same wave consumes them as the A-values of an SpMM step against V: G lanes cover one row
//            of V with VEC*V2 floats each and the 64/G lane groups take different nonzeros, fetching score
//            and column index from the owning lane by ds_bpermute.
// The scores never leave the register file, so nothing of size nnz is written to or read from memory.
// Work split, partial-sum handling for rows shared by several waves, and zero rows are as in the SpMM
// kernel (per-wave partial sums in LDS, added in wave order after one barrier).
#include "common.hpp"
#include "launch.hpp"

namespace dlspm {

// acc[v] = sum over the nonzeros [p, q) of one mask row (p < q, wave-uniform) of scale * <q_row, Kmat[column]> *
// Vmat[column, colv[v] ..], summed over the wave's slots so that every lane ends with the total.
template <int VEC, int G1, int DS, int MASKED, int G, int V2>
__device__ __forceinline__ void fused_segment(Vec<VEC>* acc, int p, int q, int D, float scale,
                                              const int* __restrict__ col_indices, const float* __restrict__ q_row,
                                              const float* __restrict__ Kmat, const float* __restrict__ Vmat,
                                              const int* colv, int lane)
{
    using VecT = Vec<VEC>;
    const int g1 = lane % G1;
    VecT lq[DS > 0 ? DS : 1];
    if constexpr (DS > 0) {
#pragma unroll
        for (int s = 0; s < DS; ++s) {
            const int d = (s * G1 + g1) * VEC;
            if constexpr (MASKED) lq[s] = d < D ? VecT::gload_clip(q_row, d, D) : VecT::zero();
            else lq[s] = VecT::gload(q_row + d);
        }
    }
#pragma unroll
    for (int v = 0; v < V2; ++v) acc[v] = VecT::zero();

    int c_nxt = col_indices[min(p + lane, q - 1)];  // next pass's columns are requested one pass ahead
    for (int base = p; base < q; base += kWave) {
        const int c = base + lane < q ? c_nxt : 0;
        c_nxt = col_indices[min(base + kWave + lane, q - 1)];
        const int cnt = min(kWave, q - base);
        // stage 1: lane l <- score of nonzero base + l (fp32, as between the reference's two loops)
        float score = sddmm_chunk<VEC, G1, DS, MASKED>(D, lane, cnt, c, q_row, lq, Kmat);
        score = base + lane < q ? score * scale : 0.f;
        // stage 2: acc += score_j * V[col_j, :]
        dense_rows_fma<VEC, G, V2>(acc, c, score, cnt, Vmat, D, colv, lane);
    }
    if constexpr (kWave / G > 1) slots_sum<VEC, G, V2>(acc, lane);
}

// The work of workgroup `bid` (RowBlock in common.hpp explains SLICED and PLANNED: with PLANNED workgroup i works on row
// row_ids[i] of Q, O and the mask). Column tiles (D > 1024) tile-major, as in spmm_block; no division in the usual
// case of one tile.
template <int VEC, int G1, int DS, int MASKED, int G, int V2, int W, int R, bool SLICED, int PLANNED = kPlanNone>
__device__ __forceinline__ void fused_block(int bid, int M, int D, int col_tiles, float scale,
                                            const int* __restrict__ row_offsets, const int* __restrict__ row_ends,
                                            const int* __restrict__ col_indices, const float* __restrict__ Q,
                                            const float* __restrict__ Kmat, const float* __restrict__ Vmat,
                                            float* __restrict__ O, const int* __restrict__ row_ids = nullptr, int nnz = 0,
                                            int flags = 0, const int* __restrict__ row_slots = nullptr,
                                            float* __restrict__ pieces = nullptr, int slots = 0)
{
    const int row_blocks = (M - 1) / R + 1;  // (planned launches have one column tile)
    const int ct = col_tiles == 1 ? 0 : bid / row_blocks;
    const int rb = bid - ct * row_blocks;
    RowBlock<W, R, SLICED, PLANNED> blk;
    blk.load(rb, M, nnz, row_offsets, row_ends, row_ids, [&]() { fetch_args_now(col_indices, Q, Kmat, Vmat, O); },
             col_tiles == 1 ? flags : flags & ~1, row_slots, slots);
    dense_rows_block<VEC, G, V2>(
        blk, ct, D, O,
        [&](Vec<VEC>* acc, int r, int p, int q, const int* colv) {
            const float* q_row = Q + (size_t)(blk.row0 + r) * D;
            fused_segment<VEC, G1, DS, MASKED, G, V2>(acc, p, q, D, scale, col_indices, q_row, Kmat, Vmat, colv, blk.lane);
        },
        pieces);
}

// (No register budget beyond the compiler's own for twelve and sixteen stage-1 accesses, unlike sddmm.hip's kernels: with all of
// them in flight -- three waves per SIMD -- Bernoulli rows lost 6 % at D = 384 and up to 23 % at D = 512 (1024 x 2304 of 230 per
// row: 47.5 -> 57.6 us), lognormal rows gained 0-11 %.)
// MASKED = false: D == G1 * VEC * DS exactly, every stage-1 access of every lane falls inside the row.
template <int VEC, int G1, int DS, int MASKED, int G, int V2, int W, int R>
__global__ __launch_bounds__(W * 64) void fused_kernel(int M, int D, int col_tiles, int flags, float scale,
                                                       const int* __restrict__ row_offsets,
                                                       const int* __restrict__ col_indices,
                                                       const float* __restrict__ Q, const float* __restrict__ Kmat,
                                                       const float* __restrict__ Vmat, float* __restrict__ O)
{
    fused_block<VEC, G1, DS, MASKED, G, V2, W, R, false>((int)blockIdx.x, M, D, col_tiles, scale, row_offsets, nullptr,
                                                         col_indices, Q, Kmat, Vmat, O, nullptr, 0, flags);
}

// Column-sliced schedule (see spmm_sliced_kernel): the row blocks once per slice of columns, slice after slice, so
// that the rows of Kmat and V gathered at any time come from one slice; partial[s][i][:] is row i's share of slice s.
template <int VEC, int G1, int DS, int MASKED, int G, int V2, int R>
__global__ __launch_bounds__(4 * 64) void fused_sliced_kernel(int M, int D, int col_tiles, int slice_blocks, float scale,
                                                              const int* __restrict__ bounds,
                                                              const int* __restrict__ col_indices,
                                                              const float* __restrict__ Q,
                                                              const float* __restrict__ Kmat,
                                                              const float* __restrict__ Vmat,
                                                              float* __restrict__ partial)
{
    const int sl = (int)(blockIdx.x / (unsigned)slice_blocks);
    const int bid = (int)blockIdx.x - sl * slice_blocks;
    fused_block<VEC, G1, DS, MASKED, G, V2, 4, R, true>(bid, M, D, col_tiles, scale, bounds + (size_t)sl * M,
                                                        bounds + (size_t)(sl + 1) * M, col_indices, Q, Kmat, Vmat,
                                                        partial + (size_t)sl * M * D);
}

// Row plan: workgroup i works on the whole row rows[i] = [starts[i], ends[i]) (one row per four-wave workgroup, one
// column tile).
template <int VEC, int G1, int DS, int MASKED, int G, int V2>
__global__ __launch_bounds__(4 * 64) void fused_planned_kernel(int M, int D, int nnz, int flags, float scale,
                                                               const int* __restrict__ starts, const int* __restrict__ ends,
                                                               const int* __restrict__ rows,
                                                               const int* __restrict__ col_indices,
                                                               const float* __restrict__ Q, const float* __restrict__ Kmat,
                                                               const float* __restrict__ Vmat, float* __restrict__ O)
{
    fused_block<VEC, G1, DS, MASKED, G, V2, 4, 1, true, kPlanRows>((int)blockIdx.x, M, D, 1, scale, starts, ends, col_indices,
                                                                   Q, Kmat, Vmat, O, rows, nnz, flags);
}

// Row plan with cut rows (see spmm_pieces_kernel): entry i is the whole row rows[i], a piece of it whose partial row of O
// goes to pieces[slot_of[i]], or nothing.
template <int VEC, int G1, int DS, int MASKED, int G, int V2>
__global__ __launch_bounds__(4 * 64) void fused_pieces_kernel(int M, int D, int nnz, int flags, int slots, float scale,
                                                              const int* __restrict__ starts, const int* __restrict__ ends,
                                                              const int* __restrict__ rows, const int* __restrict__ slot_of,
                                                              const int* __restrict__ col_indices,
                                                              const float* __restrict__ Q, const float* __restrict__ Kmat,
                                                              const float* __restrict__ Vmat, float* __restrict__ O,
                                                              float* __restrict__ pieces)
{
    fused_block<VEC, G1, DS, MASKED, G, V2, 4, 1, true, kPlanPieces>((int)blockIdx.x, M, D, 1, scale, starts, ends, col_indices,
                                                                     Q, Kmat, Vmat, O, rows, nnz, flags, slot_of, pieces, slots);
}

// ---- host side --------------------------------------------------------------------------------------

// Whether stage 1 masks the lanes past D by the range check of a buffer load (sddmm_rounds_load), in the row-block, planned and
// cut-plan kernels of twelve stage-1 accesses (D = 257 ... 383, a multiple of four, Kmat within the window): 0.92-0.93 of the
// time of the kernels that mask by selects over nine shapes (0.86 ... 0.97), the same bits. With sixteen accesses 0.99-1.00
// (0.73 ... 1.14), and below 257 the masks are a few per cent of a kernel that stage 2 dominates: those keep the selects.
template <int DS> static bool stage1_masked_by_range(int K, int D)
{
    return DS == 12 && D % 4 == 0 && K < (1 << 24) && (long long)K * D * (long long)sizeof(float) <= (long long)kRangeWindowBytes &&
           rule_on(kRuleMaskByRange);
}
template <int DS> constexpr int stage1_masked_kind(bool by_range) { return by_range && DS == 12 ? kMaskedByRange : kMaskedBySelect; }

template <int VEC, int G1, int DS, int G, int V2, int W, int R>
static hipError_t launch_one(const FusedArgs& x, hipStream_t stream)
{
    constexpr int TW = G * VEC * V2;
    const int col_tiles = (int)ceil_div(x.D, TW);
    const long long blocks = ceil_div(x.M, R) * col_tiles;
    if (blocks <= 0) return hipSuccess;
    if (blocks > 0x7fffffffLL) return hipErrorInvalidConfiguration;
    if constexpr (DS > 0) {
        if (x.D == G1 * VEC * DS && rule_on(kRuleExactWidthKernels)) {
            hipLaunchKernelGGL((fused_kernel<VEC, G1, DS, false, G, V2, W, R>), dim3((unsigned)blocks), dim3(W * 64),
                               0, stream, x.M, x.D, col_tiles, launch_flags(x.xcd_contiguous), x.scale, x.row_offsets, x.col_indices,
                               x.Q, x.Kmat, x.V, x.O);
            return hipGetLastError();
        }
    }
    if constexpr (VEC == 4 && G1 == 8 && DS == 12) {
        if (stage1_masked_by_range<DS>(x.K, x.D)) {
            hipLaunchKernelGGL((fused_kernel<VEC, G1, DS, kMaskedByRange, G, V2, W, R>), dim3((unsigned)blocks), dim3(W * 64), 0, stream,
                               x.M, x.D, col_tiles, launch_flags(x.xcd_contiguous), x.scale, x.row_offsets, x.col_indices, x.Q, x.Kmat,
                               x.V, x.O);
            return hipGetLastError();
        }
    }
    hipLaunchKernelGGL((fused_kernel<VEC, G1, DS, kMaskedBySelect, G, V2, W, R>), dim3((unsigned)blocks), dim3(W * 64), 0, stream,
                       x.M, x.D, col_tiles, launch_flags(x.xcd_contiguous), x.scale, x.row_offsets, x.col_indices, x.Q, x.Kmat, x.V,
                       x.O);
    return hipGetLastError();
}

// the layout of shape s among FusedLayouts
template <typename Launch> static hipError_t dispatch_layout(const FusedShape& s, Launch&& launch)
{
    return dispatch<FusedLayouts>(
        [&](auto l) { return l.VEC == s.vec && l.G1 == s.G1 && l.DS == s.DS && l.G == s.G && l.V == s.V; }, launch);
}
// the layouts the column-sliced and planned kernels are built for: 16 < D <= 512 in one column tile
template <typename L> constexpr bool kOneTileLayout = L::VEC == 4 && L::G1 == 8 && L::DS >= 1;

FusedShape fused_choose(const DeviceInfo& dev, int M, int D, int nnz, bool vec4, int rows, int K)
{
    FusedShape s{};
    s.vec = vec4 ? 4 : 1;
    if (vec4) {
        if (D <= 16) { s.G1 = 4; s.DS = 1; s.G = 8; s.V = 1; }
        else if (D <= 32) { s.G1 = 8; s.DS = 1; s.G = 8; s.V = 1; }
        else if (D <= 64) { s.G1 = 8; s.DS = 2; s.G = 16; s.V = 1; }
        else if (D <= 96) { s.G1 = 8; s.DS = 3; s.G = 32; s.V = 1; }
        else if (D <= 128) { s.G1 = 8; s.DS = 4; s.G = 32; s.V = 1; }
        else if (D <= 192) { s.G1 = 8; s.DS = 6; s.G = 64; s.V = 1; }
        else if (D <= 256) { s.G1 = 8; s.DS = 8; s.G = 64; s.V = 1; }
        else if (D <= 384) { s.G1 = 8; s.DS = 12; s.G = 64; s.V = 2; }
        else if (D <= 512) { s.G1 = 8; s.DS = 16; s.G = 64; s.V = 2; }
        else { s.G1 = 8; s.DS = 0; s.G = 64; s.V = 4; }  // wider D: column tiles of 1024, scores recomputed per tile
    } else {  // D < 4: one float per lane
        s.G1 = 4; s.DS = 1; s.G = 8; s.V = 1;
    }
    const int tw = s.G * s.vec * s.V;
    // rows are grouped while the grid keeps three workgroups per compute unit (lognormal rows of 8 ... 40 nonzeros, D = 64,
    // rows per workgroup 1 / 2 / 4 / 8 / 16: 1024 rows 3.3 / 4.4 / 5.5 / 6.9 / 10.9 us; 2048 rows 4.8 / 4.9 / 6.1 / 7.8 /
    // 11.7 us; 4096 rows 7.3 / 7.2 / 6.5 / 8.0 / 11.6 us; 8192 rows 12.1 / 10.4 / 8.3 / 7.2 / 9.2 us; 16384 rows: sixteen;
    // 3072 rows of 102, even: two per workgroup 8.5 us, four 7.2 us)
    // Kmat and V beyond one L2 (K known: a plain call or one with the even-rows hint): long rows are grouped four to a
    // workgroup, one whole row per wave, as under the even-rows hint, whatever the caller said. Waves that live for a whole row
    // and start together sweep the sorted columns together, so the rows of Kmat and V they gather are in L2 at the same
    // time: even rows (Bernoulli patterns, D = 128 / 256) 8192 x 8192 398 -> 243 us and 1159 -> 638 us, 16384 x 8192 462 ->
    // 283 us, 4096 x 16384 300 -> 144 us; lognormal rows (sigma 0.3 ... 1.0) lose nothing to 8 % (8192 x 8192: 470 -> 475,
    // 486 -> 514, 545 -> 577 us), which is what a caller with such rows gets back several times over from a row plan or the
    // column slices. Within one L2 the same grouping gains 6 % on even rows and loses 7 % on uneven ones: only on the hint.
    const bool beyond_l2 = K > 0 && 2.0 * (double)K * (double)D * sizeof(float) > (double)dev.l2_bytes;
    choose_split(dev, M, ceil_div(D, tw), nnz, SplitRule{3, tw >= 1024 ? 4 : 16, kWave / s.G, false, 96, 128, 8}, rows == kRowsUnknown && beyond_l2 ? kRowsEven : rows, s.W,
                 s.R);
    return s;
}

hipError_t fused_launch(const FusedArgs& x, const FusedShape& s, hipStream_t stream)
{
    return dispatch_layout(s, [&](auto l) {
        using L = decltype(l);
        return dispatch_split(s.W, s.R, [&](auto split) {
            using S = decltype(split);
            // column tiles of 1024: the per-wave partial sums of 8 or 16 waves do not fit in LDS
            if constexpr (S::W > 4 && L::G * L::VEC * L::V >= 1024) return hipErrorInvalidValue;
            else return launch_one<L::VEC, L::G1, L::DS, L::G, L::V, S::W, S::R>(x, stream);
        });
    });
}

// ---- flat schedule (see spmm.hip): every wave owns `chunk` consecutive nonzeros of the mask ------------------------
template <int VEC, int G1, int DS, int MASKED, int G, int V2>
__global__ __launch_bounds__(kFlatWaves * 64) void fused_flat_kernel(int M, int D, int nnz, int chunk, int col_tiles,
                                                                      float scale, const int* __restrict__ row_offsets,
                                                                      const int* __restrict__ col_indices,
                                                                      const float* __restrict__ Q,
                                                                      const float* __restrict__ Kmat,
                                                                      const float* __restrict__ Vmat, float* __restrict__ O,
                                                                      float* __restrict__ partial)
{
    fetch_args_now(row_offsets, col_indices, Q, Kmat, Vmat, O, partial);
    constexpr int TW = G * VEC * V2;
    using VecT = Vec<VEC>;
    const int lane = threadIdx.x & 63;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int g = lane % G;
    const int slot = lane / G;
    const long long id = (long long)blockIdx.x * kFlatWaves + w;
    // column tiles tile-major, as in the row-block kernel: all units of tile 0, then of tile 1, ...
    const int units = (int)(((long long)nnz + chunk - 1) / chunk);
    const int ct = col_tiles == 1 ? 0 : (int)(id / units);
    const int unit = (int)(id - (long long)ct * units);
    const long long a64 = (long long)unit * chunk;
    if (ct >= col_tiles || a64 >= nnz) return;  // wave-uniform
    const int a = (int)a64;
    const int b = (int)min((long long)nnz, a64 + chunk);

    int colv[V2];
    bool act[V2];
#pragma unroll
    for (int v = 0; v < V2; ++v) {
        const int col = ct * TW + (v * G + g) * VEC;
        act[v] = col < D;
        colv[v] = act[v] ? min(col, D - VEC) : 0;
    }

    int r = find_row(row_offsets, M, a, lane);
    int rbase = r;
    int win = window_load(row_offsets, M, rbase, lane);
    int pos = a;
    while (true) {
        if (r - rbase >= kWinRows) {
            rbase = r;
            win = window_load(row_offsets, M, rbase, lane);
        }
        const int rs = window_get(win, r - rbase);
        const int re = window_get(win, r - rbase + 1);
        const int p = pos;
        const int q = min(re, b);

        VecT acc[V2];
        fused_segment<VEC, G1, DS, MASKED, G, V2>(acc, p, q, D, scale, col_indices, Q + (size_t)r * D, Kmat, Vmat, colv,
                                                  lane);
        if (slot == 0) {
            float* dst = (p == rs && q == re) ? O + (size_t)r * D : partial + ((size_t)unit * 2 + (p == a ? 0 : 1)) * D;
#pragma unroll
            for (int v = 0; v < V2; ++v)
                if (act[v]) acc[v].gstore(dst + colv[v]);
        }
        pos = q;
        if (pos >= b) break;
        r = window_next_row(row_offsets, M, pos, lane, win, rbase);
    }
}

template <int VEC, int G1, int DS, int G, int V2>
static hipError_t launch_flat(const FusedArgs& x, const FlatPlan& plan, float* partial, hipStream_t stream)
{
    constexpr int TW = G * VEC * V2;
    const int col_tiles = (int)ceil_div(x.D, TW);
    const long long waves = (long long)plan.units * col_tiles;
    const long long blocks = (waves + kFlatWaves - 1) / kFlatWaves;
    if (blocks > 0x7fffffffLL) return hipErrorInvalidConfiguration;
    bool exact = false;
    if constexpr (DS > 0) exact = x.D == G1 * VEC * DS;
    if constexpr (DS > 0) {
        if (exact)
            hipLaunchKernelGGL((fused_flat_kernel<VEC, G1, DS, false, G, V2>), dim3((unsigned)blocks), dim3(kFlatWaves * 64),
                               0, stream, x.M, x.D, x.nnz, plan.chunk, col_tiles, x.scale, x.row_offsets, x.col_indices, x.Q,
                               x.Kmat, x.V, x.O, partial);
    }
    if (!exact)
        hipLaunchKernelGGL((fused_flat_kernel<VEC, G1, DS, true, G, V2>), dim3((unsigned)blocks), dim3(kFlatWaves * 64), 0,
                           stream, x.M, x.D, x.nnz, plan.chunk, col_tiles, x.scale, x.row_offsets, x.col_indices, x.Q,
                           x.Kmat, x.V, x.O, partial);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    return row_fixup_launch(x.M, x.D, plan.chunk, x.row_offsets, partial, x.O, stream);
}

hipError_t fused_flat_launch(const FusedArgs& x, const FusedShape& s, const FlatPlan& plan, float* partial,
                             hipStream_t stream)
{
    return dispatch_layout(s, [&](auto l) {
        using L = decltype(l);
        return launch_flat<L::VEC, L::G1, L::DS, L::G, L::V>(x, plan, partial, stream);
    });
}

// ---- column-sliced schedule ------------------------------------------------------------------------

template <int VEC, int G1, int DS, int G, int V2, int R>
static hipError_t launch_sliced_r(const FusedArgs& x, const SlicePlan& plan, const int* bounds, float* partial,
                                  hipStream_t stream)
{
    constexpr int TW = G * VEC * V2;
    const int col_tiles = (int)ceil_div(x.D, TW);
    const long long slice_blocks = ceil_div(x.M, R) * col_tiles;
    const long long blocks = slice_blocks * plan.slices;
    if (blocks <= 0) return hipSuccess;
    if (blocks > 0x7fffffffLL) return hipErrorInvalidConfiguration;
    if constexpr (DS > 0) {
        if (x.D == G1 * VEC * DS && rule_on(kRuleExactWidthKernels)) {
            hipLaunchKernelGGL((fused_sliced_kernel<VEC, G1, DS, false, G, V2, R>), dim3((unsigned)blocks), dim3(4 * 64), 0,
                               stream, x.M, x.D, col_tiles, (int)slice_blocks, x.scale, bounds, x.col_indices, x.Q, x.Kmat,
                               x.V, partial);
            return hipGetLastError();
        }
    }
    hipLaunchKernelGGL((fused_sliced_kernel<VEC, G1, DS, true, G, V2, R>), dim3((unsigned)blocks), dim3(4 * 64), 0, stream,
                       x.M, x.D, col_tiles, (int)slice_blocks, x.scale, bounds, x.col_indices, x.Q, x.Kmat, x.V, partial);
    return hipGetLastError();
}

template <int VEC, int G1, int DS, int G, int V2>
static hipError_t launch_sliced(const FusedArgs& x, const SlicePlan& plan, const int* bounds, float* partial,
                                hipStream_t stream)
{
    return dispatch_sliced_rows(plan.R, [&](auto r) {
        return launch_sliced_r<VEC, G1, DS, G, V2, decltype(r)::R>(x, plan, bounds, partial, stream);
    });
}

hipError_t fused_sliced_launch(const FusedArgs& x, const FusedShape& s, const SlicePlan& plan, void* workspace,
                               hipStream_t stream)
{
    int* bounds = static_cast<int*>(workspace);
    float* partial = reinterpret_cast<float*>(static_cast<char*>(workspace) + plan.bounds_bytes);
    hipError_t e = slice_bounds_launch(x.M, x.K, plan.slices, x.row_offsets, x.col_indices, bounds, stream);
    if (e != hipSuccess) return e;
    e = dispatch_layout(s, [&](auto l) {
        using L = decltype(l);
        if constexpr (kOneTileLayout<L>) return launch_sliced<4, 8, L::DS, L::G, L::V>(x, plan, bounds, partial, stream);
        else return hipErrorInvalidValue;
    });
    if (e != hipSuccess) return e;
    return slice_sum_launch((long long)x.M * x.D, plan.slices, partial, x.O, stream);
}

// ---- row plan ---------------------------------------------------------------------------------------

bool fused_plan_applies(const DeviceInfo& dev, FusedShape& s, int M, int D, int nnz, bool skewed)
{
    // built for 16 < D <= 512 (the shapes of the column-sliced kernels): one column tile
    if (s.vec != 4 || s.G1 != 8 || s.DS < 1 || s.W != 4 || s.G * s.vec * s.V < D) return false;
    if (s.R == 1) return true;
    if (!plan_ungroups_dots(dev, M, D, nnz) && !(skewed && plan_ungroups_skewed(dev, M, nnz))) return false;
    s.R = 1;
    return true;
}

// A cut plan also serves masks of fewer rows than two per compute unit, which the size rule runs with eight waves per row:
// cut, the pieces of the rows fill the device (four waves each), at the price of the kernel that adds the partial rows.
bool fused_cut_plan_applies(const DeviceInfo& dev, FusedShape& s, int M, int D, int nnz)
{
    if (s.vec == 4 && s.G1 == 8 && s.DS >= 1 && s.G * s.vec * s.V >= D && s.W == 8 && M < 2 * dev.cus) {
        s.W = 4;
        s.R = 1;
        return true;
    }
    return fused_plan_applies(dev, s, M, D, nnz);
}

template <int DS, int G, int V2>
static hipError_t launch_planned(const FusedArgs& x, const int* plan, hipStream_t stream)
{
    const int *starts = plan, *ends = plan + x.M, *rows = plan + 2 * (size_t)x.M;
    if (x.D == 8 * 4 * DS)
        hipLaunchKernelGGL((fused_planned_kernel<4, 8, DS, false, G, V2>), dim3((unsigned)x.M), dim3(4 * 64), 0, stream, x.M,
                           x.D, x.nnz, launch_flags(0), x.scale, starts, ends, rows, x.col_indices, x.Q, x.Kmat, x.V, x.O);
    else if (stage1_masked_by_range<DS>(x.K, x.D))
        hipLaunchKernelGGL((fused_planned_kernel<4, 8, DS, stage1_masked_kind<DS>(true), G, V2>), dim3((unsigned)x.M), dim3(4 * 64), 0, stream, x.M,
                           x.D, x.nnz, launch_flags(0), x.scale, starts, ends, rows, x.col_indices, x.Q, x.Kmat, x.V, x.O);
    else
        hipLaunchKernelGGL((fused_planned_kernel<4, 8, DS, kMaskedBySelect, G, V2>), dim3((unsigned)x.M), dim3(4 * 64), 0, stream, x.M,
                           x.D, x.nnz, launch_flags(0), x.scale, starts, ends, rows, x.col_indices, x.Q, x.Kmat, x.V, x.O);
    return hipGetLastError();
}

template <int DS, int G, int V2>
static hipError_t launch_pieces(const FusedArgs& x, const CutPlan& cp, void* plan, hipStream_t stream)
{
    const int* base = static_cast<const int*>(plan);
    const int *starts = base, *ends = base + cp.entries, *rows = base + 2 * (size_t)cp.entries,
              *slot_of = base + 3 * (size_t)cp.entries;
    float* pieces = reinterpret_cast<float*>(static_cast<char*>(plan) + cp.off_pieces);
    if (x.D == 8 * 4 * DS)
        hipLaunchKernelGGL((fused_pieces_kernel<4, 8, DS, false, G, V2>), dim3((unsigned)cp.entries), dim3(4 * 64), 0, stream,
                           x.M, x.D, x.nnz, launch_flags(0), cp.slots, x.scale, starts, ends, rows, slot_of, x.col_indices, x.Q,
                           x.Kmat, x.V, x.O, pieces);
    else if (stage1_masked_by_range<DS>(x.K, x.D))
        hipLaunchKernelGGL((fused_pieces_kernel<4, 8, DS, stage1_masked_kind<DS>(true), G, V2>), dim3((unsigned)cp.entries), dim3(4 * 64), 0, stream,
                           x.M, x.D, x.nnz, launch_flags(0), cp.slots, x.scale, starts, ends, rows, slot_of, x.col_indices, x.Q,
                           x.Kmat, x.V, x.O, pieces);
    else
        hipLaunchKernelGGL((fused_pieces_kernel<4, 8, DS, kMaskedBySelect, G, V2>), dim3((unsigned)cp.entries), dim3(4 * 64), 0, stream,
                           x.M, x.D, x.nnz, launch_flags(0), cp.slots, x.scale, starts, ends, rows, slot_of, x.col_indices, x.Q,
                           x.Kmat, x.V, x.O, pieces);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    return cut_rows_sum_launch(x.M, x.D, cp, plan, x.O, stream);
}

hipError_t fused_pieces_launch(const FusedArgs& x, const FusedShape& s, const CutPlan& cp, void* plan, hipStream_t stream)
{
    if (x.M <= 0) return hipSuccess;
    return dispatch_layout(s, [&](auto l) {
        using L = decltype(l);
        if constexpr (kOneTileLayout<L>) return launch_pieces<L::DS, L::G, L::V>(x, cp, plan, stream);
        else return hipErrorInvalidValue;
    });
}

hipError_t fused_planned_launch(const FusedArgs& x, const FusedShape& s, const int* plan, hipStream_t stream)
{
    if (x.M <= 0) return hipSuccess;
    return dispatch_layout(s, [&](auto l) {
        using L = decltype(l);
        if constexpr (kOneTileLayout<L>) return launch_planned<L::DS, L::G, L::V>(x, plan, stream);
        else return hipErrorInvalidValue;
    });
}

}  // namespace dlspm
