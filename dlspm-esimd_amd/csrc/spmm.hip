// CSR SpMM, C[M x N] = A_csr[M x K] * B[K x N], fp32, for gfx950.
//
// Computes what the reference's CPU loop Spmm (SPMM/spmm-esimd-fromfile2.cpp:63-83) computes and takes
// the place of its ESIMD kernel SpmmEsimd<CH> (SPMM/spmmesimd2.hpp:63-147). The decomposition is not
// the reference's (one hardware thread per (row, CH-wide column slice), sized by an occupancy
// heuristic): here
//   * a workgroup of W waves owns R consecutive rows and splits the nonzeros of those rows evenly
//     over its waves regardless of row boundaries (a merge-path split inside the row block), so a long
//     row is shared by several waves and several short rows share one wave;
//   * inside a wave, G lanes cover one row of B with VEC*V floats each (dwordx4 loads when VEC = 4),
//     and the 64/G lane groups ("slots") work on different nonzeros of the same row segment at once;
//   * a wave reads 64 (column, value) pairs with one coalesced load each and hands them out by
//     v_readlane (G = 64) or ds_bpermute (G < 64), so the CSR arrays are read exactly once per column tile;
//   * rows finished inside one wave are stored straight to C; rows shared by several waves leave
//     per-wave partial sums in LDS which are added in wave order after one barrier, so the result does
//     not depend on timing (no atomics, no pre-zeroed output); rows without nonzeros are written as 0.
// Two more schedules reuse these pieces when the caller passes a workspace: the flat schedule (every wave
// owns a fixed run of nonzeros of the whole matrix; for very uneven rows) and the column-sliced schedule
// (the same workgroups on one range of columns of A after the other; for a B larger than one L2), and a
// B larger than one L2 is always cut into column tiles that the grid works through one after the other.
#include "common.hpp"
#include "launch.hpp"

namespace dlspm {

// acc[v] = sum over the nonzeros [p, q) of one row (p < q, wave-uniform) of value * B[column, colv[v] ..], summed over
// the wave's S = 64/G slots, so that every lane (slot 0 in particular) ends with the total.
template <int VEC, int G, int V, bool BUF = false>
__device__ __forceinline__ void spmm_segment(Vec<VEC>* acc, int p, int q, const int* __restrict__ col_indices,
                                             const float* __restrict__ values, const float* __restrict__ B, int N,
                                             const int* colv, int lane)
{
    using VecT = Vec<VEC>;
#pragma unroll
    for (int v = 0; v < V; ++v) acc[v] = VecT::zero();
    // 64 (column, value) pairs per pass, one per lane; the next 64 are requested (index clamped, so the
    // loads carry no condition) before the rows of B for the current ones, and arrive behind them. Narrow rows of B
    // (lane groups of 8 or fewer: a pass is at most 8 row loads) request two passes ahead: CSR arrays beyond the
    // Infinity Cache come from HBM, and one such pass does not cover that (24576 x 8192 at density 0.3, N = 32:
    // 382 -> 335 us; lane groups of 16: 604 -> 627 us; of 32 and 64: -2 % and -1 %; matrices within the cache: equal).
    const int first = min(p + lane, q - 1);
    int c_nxt = col_indices[first];
    float a_nxt = values[first];
    if constexpr (G <= 8) {
        const int second = min(p + kWave + lane, q - 1);
        int c_far = col_indices[second];
        float a_far = values[second];
        for (int base = p; base < q; base += kWave) {
            const bool mine = base + lane < q;
            const int c = mine ? c_nxt : 0;
            const float av = mine ? a_nxt : 0.f;
            c_nxt = c_far;
            a_nxt = a_far;
            const int ahead = min(base + 2 * kWave + lane, q - 1);
            c_far = col_indices[ahead];
            a_far = values[ahead];
            dense_rows_fma<VEC, G, V, BUF>(acc, c, av, min(kWave, q - base), B, N, colv, lane);
        }
    } else {
        for (int base = p; base < q; base += kWave) {
            const bool mine = base + lane < q;
            const int c = mine ? c_nxt : 0;
            const float av = mine ? a_nxt : 0.f;
            const int ahead = min(base + kWave + lane, q - 1);
            c_nxt = col_indices[ahead];
            a_nxt = values[ahead];
            dense_rows_fma<VEC, G, V, BUF>(acc, c, av, min(kWave, q - base), B, N, colv, lane);
        }
    }
    if constexpr (kWave / G > 1) slots_sum<VEC, G, V>(acc, lane);
}

// The work of workgroup `bid` (RowBlock in common.hpp explains SLICED and PLANNED; `row_ends` and `row_ids` belong to
// them). Column tiles (dense rows wider than one wave covers): row-major order (the tiles of a row block next to each
// other, so the CSR arrays are read from memory once) while all of B fits one L2; tile-major order (all row blocks of
// tile 0, then of tile 1, ...) when it does not, so that the device gathers from one K x TW slab of B at a time.
// Measured on 512 x 4608, N = 3136 (B: 55 MiB): 708 -> 239 us tile-major; on 2048 x 1024, N = 784 (3 MiB), lognormal
// rows: 81 us row-major, 93 us tile-major. No division in the usual case of one tile.
template <int VEC, int G, int V, int W, int R, bool SLICED, int PLANNED = kPlanNone, bool BUF = false>
__device__ __forceinline__ void spmm_block(int bid, int M, int N, int col_tiles, int tile_major,
                                           const int* __restrict__ row_offsets,
                                           const int* __restrict__ row_ends, const int* __restrict__ col_indices,
                                           const float* __restrict__ values, const float* __restrict__ B,
                                           float* __restrict__ C, const int* __restrict__ row_ids = nullptr, int nnz = 0,
                                           int flags = 0, int row_blocks = 0, const int* __restrict__ row_slots = nullptr,
                                           float* __restrict__ pieces = nullptr, int slots = 0)
{
    int ct = 0, rb = bid;
    if (col_tiles != 1) {
        if (tile_major >= kTilesPerXcd) {
            // Each XCD works on its own run of column tiles (workgroup 8 j + x runs on XCD x, as the hardware deals them): the
            // eight L2s then fetch B once between them, not once each. XCD x owns the q = T / 8 tiles from x q on; the T mod 8
            // tiles left over come last and are shared by all XCDs like the tiles of the other orders, so every XCD gets
            // the same number of workgroups. Inside an XCD's part (and in the shared part) the order is row-major or tile-major.
            if constexpr (!PLANNED) row_blocks = (M - 1) / R + 1;
            const int q = col_tiles >> 3, owned = 8 * q * row_blocks;
            const bool tiles_first = tile_major == kTilesPerXcdTileMajor;
            if (bid < owned) {
                const int x = bid & 7, j = bid >> 3;
                int local;
                if (tiles_first) {
                    local = j / row_blocks;
                    rb = j - local * row_blocks;
                } else {
                    rb = j / q;
                    local = j - rb * q;
                }
                ct = x * q + local;
            } else {
                const int rest = col_tiles - 8 * q, j = bid - owned;
                if (tiles_first) {
                    const int local = j / row_blocks;
                    rb = j - local * row_blocks;
                    ct = 8 * q + local;
                } else {
                    rb = j / rest;
                    ct = 8 * q + j - rb * rest;
                }
            }
        } else if (tile_major) {
            if constexpr (!PLANNED) row_blocks = (M - 1) / R + 1;  // (a plan has as many entries as its launch says)
            ct = bid / row_blocks;
            rb = bid - ct * row_blocks;
        } else {
            rb = bid / col_tiles;
            ct = bid - rb * col_tiles;
        }
    }
    RowBlock<W, R, SLICED, PLANNED> blk;
    blk.load(rb, M, nnz, row_offsets, row_ends, row_ids, [&]() { fetch_args_now(col_indices, values, B, C); },
             col_tiles == 1 ? flags : flags & ~1, row_slots, slots);
    dense_rows_block<VEC, G, V>(
        blk, ct, N, C,
        [&](Vec<VEC>* acc, int, int p, int q, const int* colv) {
            spmm_segment<VEC, G, V, BUF>(acc, p, q, col_indices, values, B, N, colv, blk.lane);
        },
        pieces);
}

// BUF: B is read through a buffer descriptor (B below 4 GiB: see dense_rows_fma)
template <int VEC, int G, int V, int W, int R, bool BUF>
__global__ __launch_bounds__(W * 64) void spmm_kernel(int M, int N, int col_tiles, int tile_major, int flags,
                                                      const int* __restrict__ row_offsets,
                                                      const int* __restrict__ col_indices,
                                                      const float* __restrict__ values,
                                                      const float* __restrict__ B, float* __restrict__ C)
{
    spmm_block<VEC, G, V, W, R, false, false, BUF>((int)blockIdx.x, M, N, col_tiles, tile_major, row_offsets, nullptr,
                                                   col_indices, values, B, C, nullptr, 0, flags);
}

// Column-sliced schedule: the grid holds the row blocks once per slice of columns, slice after slice, so that at
// any time the device gathers rows of B from one slice only (a dense operand larger than one L2 is then read at L2
// speed). Slice s of row i is [bounds[s][i], bounds[s + 1][i]); its partial row goes to partial[s][i][:].
template <int VEC, int G, int V, int R>
__global__ __launch_bounds__(4 * 64) void spmm_sliced_kernel(int M, int N, int col_tiles, int tile_major,
                                                             int slice_blocks, const int* __restrict__ bounds,
                                                             const int* __restrict__ col_indices,
                                                             const float* __restrict__ values,
                                                             const float* __restrict__ B, float* __restrict__ partial)
{
    const int sl = (int)(blockIdx.x / (unsigned)slice_blocks);
    const int bid = (int)blockIdx.x - sl * slice_blocks;
    spmm_block<VEC, G, V, 4, R, true>(bid, M, N, col_tiles, tile_major, bounds + (size_t)sl * M,
                                      bounds + (size_t)(sl + 1) * M, col_indices, values, B, partial + (size_t)sl * M * N);
}

// the order of the column tiles in a planned launch (launch flags, bits 12-13): tile after tile for all XCDs, or every
// XCD on its own tiles (tile after tile inside it)
__device__ __forceinline__ int planned_tile_order(int flags)
{
    const int order = (flags >> kFlagTileOrderShift) & 3;
    return order >= kTilesPerXcd ? kTilesPerXcdTileMajor : 1;
}

// Row plan: workgroup i works on the whole row rows[i] = [starts[i], ends[i]) of the CSR matrix (one row per four-wave
// workgroup); with column tiles the plan is gone through once per tile, tile after tile.
template <int VEC, int G, int V, bool BUF>
__global__ __launch_bounds__(4 * 64) void spmm_planned_kernel(int M, int N, int nnz, int col_tiles, int flags,
                                                              const int* __restrict__ starts,
                                                              const int* __restrict__ ends, const int* __restrict__ rows,
                                                              const int* __restrict__ col_indices,
                                                              const float* __restrict__ values,
                                                              const float* __restrict__ B, float* __restrict__ C)
{
    spmm_block<VEC, G, V, 4, 1, true, kPlanRows, BUF>((int)blockIdx.x, M, N, col_tiles, planned_tile_order(flags), starts, ends,
                                                      col_indices, values, B, C, rows, nnz, flags, M);
}

// Row plan with cut rows: `entries` workgroups per column tile, entry i = the nonzeros [starts[i], ends[i]) of row rows[i],
// which is the whole row (slot_of[i] == -1: stored to C), a piece of it (slot_of[i] = s >= 0: the piece's sum goes to
// pieces[s][0 .. N) and cut_rows_sum_kernel adds the pieces of each cut row afterwards), or nothing (below -1).
template <int VEC, int G, int V, bool BUF>
__global__ __launch_bounds__(4 * 64) void spmm_pieces_kernel(int M, int N, int nnz, int col_tiles, int flags, int entries,
                                                             int slots, const int* __restrict__ starts,
                                                             const int* __restrict__ ends, const int* __restrict__ rows,
                                                             const int* __restrict__ slot_of,
                                                             const int* __restrict__ col_indices,
                                                             const float* __restrict__ values,
                                                             const float* __restrict__ B, float* __restrict__ C,
                                                             float* __restrict__ pieces)
{
    spmm_block<VEC, G, V, 4, 1, true, kPlanPieces, BUF>((int)blockIdx.x, M, N, col_tiles, planned_tile_order(flags), starts, ends, col_indices, values,
                                                        B, C, rows, nnz, flags, entries, slot_of, pieces, slots);
}

// The same plan with the cut rows shared out by COLUMNS instead (widths that one wave covers with lane groups of 16 to 64,
// 33 ... 512 columns): an entry that is piece k of a row cut into c works on ALL nonzeros of the row -- the plan enters a piece with
// its whole row's range -- and on the k-th of c equal shares of the columns (a multiple of four each), and stores to C
// directly: no partial rows, no second kernel. The share is gone through in passes of GW x 4 columns with GW lanes per
// dense row, GW = 32, 16 or 8 for shares of more than 64, more than 32, and fewer columns: a pass then costs the piece
// as many load instructions as its share of the nonzeros would have (64 / GW nonzeros per instruction instead of
// one; c is a power of two, so 256 columns are shared out exactly down to 32 per piece). Every share of a row is summed in
// the same order (that of a row in the GW layout), so the result does not depend on the plan.
template <int VEC, int GW, bool BUF, typename Block>
__device__ __forceinline__ void spmm_share_passes(const Block& blk, int col0, int col_end, int N,
                                                  const int* __restrict__ col_indices, const float* __restrict__ values,
                                                  const float* __restrict__ B, float* __restrict__ C)
{
    constexpr int TWW = GW * VEC;
    for (int c0 = col0; c0 < col_end; c0 += TWW) {
        dense_rows_window<VEC, GW, 1>(blk, c0, min(col_end, c0 + TWW), N, C,
                                      [&](Vec<VEC>* acc, int, int p, int q, const int* colv) {
                                          spmm_segment<VEC, GW, 1, BUF>(acc, p, q, col_indices, values, B, N, colv, blk.lane);
                                      });
        if (c0 + TWW < col_end) __syncthreads();  // the partial sums in LDS are written again by the next pass
    }
}

template <int VEC, int G, int V, bool BUF>
__global__ __launch_bounds__(4 * 64) void spmm_shares_kernel(int M, int N, int nnz, int flags, int entries,
                                                             const int* __restrict__ starts, const int* __restrict__ ends,
                                                             const int* __restrict__ rows, const int* __restrict__ slot_of,
                                                             const int* __restrict__ col_indices,
                                                             const float* __restrict__ values,
                                                             const float* __restrict__ B, float* __restrict__ C)
{
    // (the word is asked for together with the rest of the entry: looking at it first would put one more round trip to
    // memory in front of every workgroup's work)
    const int word = slot_of[blockIdx.x];
    RowBlock<4, 1, true, kPlanRows> blk;
    blk.load((int)blockIdx.x, M, nnz, starts, ends, rows, [&]() { fetch_args_now(col_indices, values, B, C); }, flags);
    if (word < -1) return;  // an entry that holds nothing
    if (word < 0) {  // a whole row
        dense_rows_block<VEC, G, V>(blk, 0, N, C, [&](Vec<VEC>* acc, int, int p, int q, const int* colv) {
            spmm_segment<VEC, G, V, BUF>(acc, p, q, col_indices, values, B, N, colv, blk.lane);
        });
        return;
    }
    const int k = (word >> kPieceNumberShift) & kPieceNumberMask, lg = (word >> kPieceCountShift) & kPieceCountMask;
    const int share = max((((N + (1 << lg) - 1) >> lg) + 3) & ~3, 4);
    const int col0 = k * share, col_end = min(N, col0 + share);
    if (col0 >= N) return;  // more pieces than the width has shares of four columns
    // (a width that is no multiple of four: the last share's lanes move back to end with the width, as everywhere; where
    // that takes them into the share before, they store what its own piece stores there)
    if (share > 64) spmm_share_passes<VEC, 32, BUF>(blk, col0, col_end, N, col_indices, values, B, C);
    else if (share > 32) spmm_share_passes<VEC, 16, BUF>(blk, col0, col_end, N, col_indices, values, B, C);
    else spmm_share_passes<VEC, 8, BUF>(blk, col0, col_end, N, col_indices, values, B, C);
}

// ---- host side --------------------------------------------------------------------------------------

template <int VEC, int G, int V, int W, int R>
static hipError_t launch_one(const SpmmArgs& x, int tile_major, hipStream_t stream)
{
    constexpr int TW = G * VEC * V;
    const int col_tiles = (int)ceil_div(x.N, TW);
    const long long blocks = ceil_div(x.M, R) * col_tiles;
    if (blocks <= 0) return hipSuccess;
    if (blocks > 0x7fffffffLL) return hipErrorInvalidConfiguration;
    {
        if (dense_fits_buffer(x.K, x.N)) {
            hipLaunchKernelGGL((spmm_kernel<VEC, G, V, W, R, true>), dim3((unsigned)blocks), dim3(W * 64), 0, stream, x.M, x.N,
                               col_tiles, tile_major, launch_flags(x.xcd_contiguous), x.row_offsets, x.col_indices, x.values, x.B, x.C);
            return hipGetLastError();
        }
    }
    hipLaunchKernelGGL((spmm_kernel<VEC, G, V, W, R, false>), dim3((unsigned)blocks), dim3(W * 64), 0, stream, x.M, x.N,
                       col_tiles, tile_major, launch_flags(x.xcd_contiguous), x.row_offsets, x.col_indices, x.values, x.B, x.C);
    return hipGetLastError();
}

// the layout of shape s among SpmmLayouts
template <typename Launch> static hipError_t dispatch_layout(const SpmmShape& s, Launch&& launch)
{
    return dispatch<SpmmLayouts>([&](auto l) { return l.VEC == s.vec && l.G == s.G && l.V == s.V; }, launch);
}

// Width of the column tiles of B that the grid works through one after the other (tile-major order), or 0: one tile
// if a wave can cover N, else tiles of 512 in row-major order.
// A B that does not fit one XCD's 4 MiB L2 is cut into tiles, each the widest of 512 ... 32 columns whose K x tile
// slab still fits (measured on 8192 x 4096, N = 1024: 1460 us with tiles of 512, 930 us with 256; on 512 x 4608,
// N = 3136: 309 us against 273 us); also where one wave could cover the whole width (N <= 512). Not for grids the
// device holds all at once: there the order cannot help, and 64 x 147 at N = 12544 lost 4 us.
// Tiles narrower than 128 columns (lane groups of 16 or 8 per dense row) only for a call without workspace memory
// (`narrow_tiles`): with it, slicing the columns of A keeps wider, more efficient dense rows (8192 x 65536, N = 128:
// 330 us untiled, 236 us in tiles of 32, 137 us in 16 slices of the full width).
// More tiles than a wave needs to cover N cost every row its start-up once more per tile: the tile is narrowed only
// for rows of at least 32 nonzeros on average, and only while the slab is at most twice the L2 (measured on graph-
// like shapes, K = 262144 ... 1048576, 8 nonzeros per row: tiles of 32 up to 2x slower than one tile; 32 per row:
// equal; K = 65536, slab 8 MiB, 655 per row: 330 -> 236 us).
// dlspm_tuning.tile_major = 0|1 and .tile_width = 512|...|32 override the rule for tuning sweeps (tile_major = 0 with a
// width: tiles of that width in row-major order). "The L2" is the device's own figure for one of them (4 MiB on MI355X),
// "all at once" eight workgroups on each compute unit.
//
// Finer tiles for a call without memory or plan (`plain`; kRuleFinerColumnTiles, rows of 16 nonzeros and more on average).
// Such a call does not know how even the rows are; finer tiles cost even rows little and spread a long row over
// several compute units. Times in us inside a graph, rule off / on:
//  * few rows (up to three quarters of a compute unit's worth of row x tile pairs): the widest tile that gives two pairs
//    per compute unit, row-major. Bernoulli rows, M = 16 / 64 / 128, mean over six shapes: N = 128: 4.20 / 3.40, 4.3 / 3.5,
//    4.38 / 3.80; N = 256: 4.89 / 3.44, 5.0 / 3.7, 5.28 / 4.50; N = 512: 6.93 / 3.51, 7.3 / 4.6, 7.59 / 5.74; lognormal
//    rows (sigma 0.8): times 0.35 ... 0.9; at 160 and 192 rows even rows gain nothing (0.96 ... 1.13, the losses at widths
//    that are not a multiple of the tile) and lognormal ones 10-40 %. The reference's 128 x 1152 and 128 x 512 ResNet-50
//    layers at N = 256 (26 files): 6.08 / 4.80; at N = 512: 8.81 / 6.51.
//  * N above 512 and up to eight rows per compute unit: row-major tiles of 256 instead of 512 (200 x 2304, N = 784:
//    12.2 / 11.5 even, 42.1 / 19.7 lognormal; 1500 x 512, N = 600: 24.8 / 19.3 and 34.4 / 25.6; taller matrices lose:
//    8192 x 512, N = 784: 57.4 / 62.0).
//  * B beyond the L2 and N above 512 (rows of 32 nonzeros and more; planned launches too, and N from 449 on in matrices of up to
//    sixteen rows per compute unit): every XCD works on its own tiles of B (spmm_block), in
//    tile-major order inside the XCD, in tiles of 128 where that gives each XCD two tiles and more, else of 64, and never
//    wider than the slab that fits the L2. The eight L2s then fetch B once between them instead of once each, the finer
//    tiles spread long rows, and the slab in use per XCD stays small. Against the widest fitting tile in one tile-major
//    order for all XCDs (and row-major tiles of 512 on small grids), even / lognormal rows: 64 x 576, N = 3136: 10.4 -> 6.8 and
//    14.3 -> 14.4; 64 x 147, N = 12544: 22.3 -> 12.7 and 19.3 -> 12.8; 256 x 2304, N = 3136: 86.8 -> ~40 and 134 -> ~90;
//    1024 x 1152, N = 12544: 212 -> 197 and 645 -> 200; 2048 x 2304, N = 3136: 225 -> 200 and 404 -> 202; 4096 x 4096,
//    N = 3136: 453 -> 350 and 679 -> 370; 8192 x 4096, N = 1024: 122 -> 120 and 134 -> 129 (tiles of 64).
//    With tiles dealt to the XCDs in whole numbers only (49 tiles: 7 to one XCD, 6 to the others) the uneven load cost what
//    the fetches saved (4096 x 4096: 394 us): hence the shared rest.
//  Rows below 16 nonzeros pay the start of a row once more per tile: 256 x 64 with 3 ... 13 per row at N = 3136 lost 13-33 %
//  to tiles of 256, 512 x 128 with 6 per row at N = 784 10-18 %.
struct TileChoice { int width, major; };  // width 0: no tiles narrower than a wave covers (or than 512)

// widest tile that one wave covers N with: what a launch without tiles works in
static int spmm_one_wave_tile(int N) { return N > 256 ? 512 : N > 128 ? 256 : N > 64 ? 128 : N > 32 ? 64 : 32; }

static TileChoice spmm_tile_width(const DeviceInfo& dev, int M, int K, int N, int nnz, bool narrow_tiles, bool plain)
{
    const long long l2 = dev.l2_bytes;
    const int min_tile = narrow_tiles ? 32 : 128;
    if (N <= min_tile) return {0, 0};
    const auto valid = [&](int t) { return (t == 512 || t == 256 || t == 128 || t == 64 || t == 32) && t >= min_tile; };
    const bool finer = plain && narrow_tiles && rule_on(kRuleFinerColumnTiles);
    const bool beyond_l2 = (double)K * (double)N * (double)sizeof(float) > (double)l2;
    const int one = spmm_one_wave_tile(N);
    const bool few_rows = finer && (long long)nnz >= 16ll * M && 4ll * M * ceil_div(N, one) <= 3ll * dev.cus;
    // B beyond the L2 under dense rows of eight tiles of 64 floats and more, rows of 32 nonzeros and more: every XCD on its own tiles
    // (N = 512, tiles of 128 for all XCDs -> of 64, each XCD on its own: 2048 x 8192: 80.5 -> 64.0 us even, 137 -> 74.9 us lognormal; 8192 x
    // 8192: 513 -> 505 and 631 -> 510 us; 1024 x 2304: 21.4 -> 20.7 and 64.1 -> 26.0 us; up to sixteen rows per compute unit: 8192 x
    // 2304 of 100 per row lost 17 %; at N = 256 eight tiles of 32 lose up to 25 %)
    // (calls without schedule memory: plain ones and planned ones alike, so that a plan keeps what the plain call has)
    const bool per_xcd = narrow_tiles && rule_on(kRuleFinerColumnTiles) && !few_rows && beyond_l2 && (long long)nnz >= 32ll * M &&
                         (N > 512 || (N > 448 && M <= 16ll * dev.cus));
    bool on = beyond_l2 && ((long long)M * ceil_div(N, 512) >= 8ll * dev.cus || per_xcd);
    if (tuning().tile_major >= 0) on = tuning().tile_major != 0;
    if (tuning().tile_major >= kTilesPerXcd && narrow_tiles)  // tuning: tiles of this width, each XCD on its own run of them (not with schedule memory)
        return valid(tuning().tile_width) && tuning().tile_width < N ? TileChoice{tuning().tile_width, tuning().tile_major} : TileChoice{0, 0};
    if (!on) {
        const int t = tuning().tile_width;
        if (tuning().tile_major == 0)  // tuning: tiles of this width in row-major order
            return valid(t) && t < N ? TileChoice{t, 0} : TileChoice{0, 0};
        if (!finer || (long long)nnz < 16ll * M) return {0, 0};
        if (few_rows) {
            int tile = one;
            while (tile > 32 && (long long)M * ceil_div(N, tile) < 2ll * dev.cus) tile /= 2;
            if (2 * (N - (int)(ceil_div(N, tile) - 1) * tile) < tile) tile *= 2;  // a last tile less than half full: wider tiles
            if (tile >= one || tile >= N) return {0, 0};
            return {tile, beyond_l2 && ceil_div(N, tile) >= 8 ? kTilesPerXcd : 0};
        }
        return N > 512 && M <= 8ll * dev.cus ? TileChoice{256, 0} : TileChoice{0, 0};
    }
    int tile = min_tile;
    for (int t = 512; t > min_tile; t /= 2)
        if ((long long)K * t * (long long)sizeof(float) <= l2) {
            tile = t;
            break;
        }
    // with workspace memory the column-sliced schedule cuts a taller slab along K as well, from two slices of 32
    // nonzeros per row on (8192 x 32768, N = 1024: 925 us in tiles of 32 without memory, 807 us in 16 slices of tiles
    // of 512, 533 us in 8 slices of tiles of 128; 2048 x 131072, N = 512: 384 / 324 / 250 us)
    const bool sliced_too = !narrow_tiles && nnz >= kSlicedMinNnz && (long long)nnz >= 64ll * M && (long long)M >= kSlicedMinRowsPerCu * dev.cus;
    const bool narrow_ok =
        (long long)nnz >= 32ll * M && ((long long)K * tile * (long long)sizeof(float) <= 2 * l2 || sliced_too);
    int major = 1;
    if (!narrow_ok) tile = 512;
    else if (per_xcd && tuning().tile_major < 0) {
        int t = ceil_div(N, 128) >= 16 ? 128 : 64;  // two tiles of 128 per XCD and more, else tiles of 64
        if (!plain && (long long)M >= 4ll * dev.cus) {
            // a planned launch runs one row per workgroup whatever the rows' lengths (a plain one groups short rows): from four
            // rows per compute unit on, the finest tile that still gives a workgroup 20 000 products of a mean row, 64 ... 256
            // columns (lognormal rows, sigma 0.5, tiles of 256 / 128 / 64: 8192 x 4096 of 100 per row, N = 1024: 124 / 127 /
            // 185 us; 2048 x 2304 of 230, N = 3136: 206 / 197 / 215 us; 4096 x 8192 of 400, N = 1024: 407 / 253 / 236 us;
            // fewer rows want the finer tiles of the plain call, which shorten the tail: 300 x 1152 of 115: 23.5 / 19.7 / 24.0 us)
            const long long avg = std::max<long long>(nnz / std::max(M, 1), 1);
            const int by_work = avg * 64 >= 20000 ? 64 : avg * 128 >= 20000 ? 128 : 256;
            if (by_work > t) t = by_work;
        }
        if (t > tile) t = tile;
        if (ceil_div(N, t) >= 8) {
            tile = t;
            major = kTilesPerXcdTileMajor;
        } else if (!plain) {
            tile = t;  // fewer than eight tiles: one after the other for all XCDs
        } else if (tile > 64) {
            tile = 64;
        }
    }
    {
        const int t = tuning().tile_width;
        if (valid(t)) tile = t;
    }
    return tile < N ? TileChoice{tile, major} : TileChoice{0, 0};  // a single tile: nothing to order
}

// Chooses the lane layout from N (and the height of B) and the (W, R) split from the mean row length.
SpmmShape spmm_choose(const DeviceInfo& dev, int M, int K, int N, int nnz, bool vec4, int rows, bool narrow_tiles, bool banded,
                      bool plain)
{
    SpmmShape s{};
    s.vec = vec4 ? 4 : 1;
    // banded (DLSPM_HINT_BANDED): no L2-sized column tiles, each XCD gathers from its own part of B anyway
    const TileChoice tiles = vec4 && !banded ? spmm_tile_width(dev, M, K, N, nnz, narrow_tiles, plain) : TileChoice{0, 0};
    const int tile = tiles.width;
    s.tile_major = tiles.major;
    if (vec4) {
        if (tile == 512) { s.G = 64; s.V = 2; }
        else if (tile == 256) { s.G = 64; s.V = 1; }
        else if (tile == 128) { s.G = 32; s.V = 1; }
        else if (tile == 64) { s.G = 16; s.V = 1; }
        else if (tile == 32) { s.G = 8; s.V = 1; }
        else if (N > 256) { s.G = 64; s.V = 2; }
        else if (N > 128) { s.G = 64; s.V = 1; }
        else if (N > 64) { s.G = 32; s.V = 1; }
        else if (N > 32) { s.G = 16; s.V = 1; }
        else { s.G = 8; s.V = 1; }
    } else {  // N < 4: one float per lane, eight nonzeros per access
        s.G = 8;
        s.V = 1;
    }
    const int tw = s.G * s.vec * s.V;
    choose_split(dev, M, ceil_div(N, tw), nnz, SplitRule{8, 16, kWave / s.G, true, 0, s.G == kWave ? 96 : 128}, rows, s.W, s.R);
    return s;
}

hipError_t spmm_launch(const SpmmArgs& x, const SpmmShape& s, hipStream_t stream)
{
    return dispatch_layout(s, [&](auto l) {
        using L = decltype(l);
        return dispatch_split(s.W, s.R, [&](auto split) {
            using S = decltype(split);
            return launch_one<L::VEC, L::G, L::V, S::W, S::R>(x, s.tile_major, stream);
        });
    });
}

// ---- flat schedule ----------------------------------------------------------------------------------
// Every wave owns `chunk` consecutive nonzeros of the whole matrix (and one column tile), whatever rows they
// belong to, so the time of a wave does not depend on how the nonzeros are spread over the rows: one row of a
// million nonzeros is shared by thousands of waves. A wave finds its first row by search, walks the rows of its
// range with a register window of row offsets, stores rows that lie wholly inside its range straight to C, and
// leaves at most two partial rows (the one that began before its range, the one that continues after it) in
// `partial[unit][0 or 1][N]`. row_fixup_kernel then adds the partial rows in unit order and writes rows without
// nonzeros as zeros, so the result is deterministic. No LDS, no barrier, no atomics.
template <int VEC, int G, int V>
__global__ __launch_bounds__(kFlatWaves * 64) void spmm_flat_kernel(int M, int N, int nnz, int chunk, int col_tiles,
                                                                     int tile_major,
                                                                     const int* __restrict__ row_offsets,
                                                                     const int* __restrict__ col_indices,
                                                                     const float* __restrict__ values,
                                                                     const float* __restrict__ B, float* __restrict__ C,
                                                                     float* __restrict__ partial)
{
    fetch_args_now(row_offsets, col_indices, values, B, C, partial);
    constexpr int TW = G * VEC * V;
    using VecT = Vec<VEC>;
    const int lane = threadIdx.x & 63;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int g = lane % G;
    const int slot = lane / G;
    const long long id = (long long)blockIdx.x * kFlatWaves + w;
    // column tiles in the order the row-block kernel uses (tile-major: all units of tile 0, then of tile 1, ...)
    int ct = 0, unit = (int)id;
    if (col_tiles != 1) {
        if (tile_major) {
            const int units = (int)(((long long)nnz + chunk - 1) / chunk);
            ct = (int)(id / units);
            unit = (int)(id - (long long)ct * units);
        } else {
            unit = (int)(id / col_tiles);
            ct = (int)(id - (long long)unit * col_tiles);
        }
    }
    const long long a64 = (long long)unit * chunk;
    if (ct >= col_tiles || a64 >= nnz) return;  // wave-uniform
    const int a = (int)a64;
    const int b = (int)min((long long)nnz, a64 + chunk);

    int colv[V];
    bool act[V];
#pragma unroll
    for (int v = 0; v < V; ++v) {
        const int col = ct * TW + (v * G + g) * VEC;
        act[v] = col < N;
        colv[v] = act[v] ? min(col, N - VEC) : 0;
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

        VecT acc[V];
        spmm_segment<VEC, G, V>(acc, p, q, col_indices, values, B, N, colv, lane);

        if (slot == 0) {
            float* dst = (p == rs && q == re) ? C + (size_t)r * N : partial + ((size_t)unit * 2 + (p == a ? 0 : 1)) * N;
#pragma unroll
            for (int v = 0; v < V; ++v)
                if (act[v]) acc[v].gstore(dst + colv[v]);
        }
        pos = q;
        if (pos >= b) break;
        r = window_next_row(row_offsets, M, pos, lane, win, rbase);
    }
}

template <int VEC, int G, int V>
static hipError_t launch_flat(const SpmmArgs& x, const FlatPlan& plan, int tile_major, float* partial, hipStream_t stream)
{
    constexpr int TW = G * VEC * V;
    const int col_tiles = (int)ceil_div(x.N, TW);
    const long long waves = (long long)plan.units * col_tiles;
    const long long blocks = (waves + kFlatWaves - 1) / kFlatWaves;
    if (blocks > 0x7fffffffLL) return hipErrorInvalidConfiguration;
    hipLaunchKernelGGL((spmm_flat_kernel<VEC, G, V>), dim3((unsigned)blocks), dim3(kFlatWaves * 64), 0, stream, x.M, x.N,
                       x.nnz, plan.chunk, col_tiles, tile_major, x.row_offsets, x.col_indices, x.values, x.B, x.C, partial);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    return row_fixup_launch(x.M, x.N, plan.chunk, x.row_offsets, partial, x.C, stream);
}

hipError_t spmm_flat_launch(const SpmmArgs& x, const SpmmShape& s, const FlatPlan& plan, float* partial,
                            hipStream_t stream)
{
    return dispatch_layout(s, [&](auto l) {
        using L = decltype(l);
        return launch_flat<L::VEC, L::G, L::V>(x, plan, s.tile_major, partial, stream);
    });
}

// ---- column-sliced schedule ------------------------------------------------------------------------

template <int VEC, int G, int V, int R>
static hipError_t launch_sliced_r(const SpmmArgs& x, const SlicePlan& plan, int tile_major, const int* bounds,
                                  float* partial, hipStream_t stream)
{
    constexpr int TW = G * VEC * V;
    const int col_tiles = (int)ceil_div(x.N, TW);
    const long long slice_blocks = ceil_div(x.M, R) * col_tiles;
    const long long blocks = slice_blocks * plan.slices;
    if (blocks <= 0) return hipSuccess;
    if (blocks > 0x7fffffffLL) return hipErrorInvalidConfiguration;
    hipLaunchKernelGGL((spmm_sliced_kernel<VEC, G, V, R>), dim3((unsigned)blocks), dim3(4 * 64), 0, stream, x.M, x.N,
                       col_tiles, tile_major, (int)slice_blocks, bounds, x.col_indices, x.values, x.B, partial);
    return hipGetLastError();
}

template <int VEC, int G, int V>
static hipError_t launch_sliced(const SpmmArgs& x, const SlicePlan& plan, int tile_major, const int* bounds,
                                float* partial, hipStream_t stream)
{
    return dispatch_sliced_rows(plan.R, [&](auto r) {
        return launch_sliced_r<VEC, G, V, decltype(r)::R>(x, plan, tile_major, bounds, partial, stream);
    });
}

hipError_t spmm_sliced_launch(const SpmmArgs& x, const SpmmShape& s, const SlicePlan& plan, void* workspace,
                              hipStream_t stream)
{
    int* bounds = static_cast<int*>(workspace);
    float* partial = reinterpret_cast<float*>(static_cast<char*>(workspace) + plan.bounds_bytes);
    hipError_t e = slice_bounds_launch(x.M, x.K, plan.slices, x.row_offsets, x.col_indices, bounds, stream);
    if (e != hipSuccess) return e;
    // built for every dwordx4 layout spmm_choose gives (N >= 4)
    e = dispatch_layout(s, [&](auto l) {
        using L = decltype(l);
        if constexpr (L::VEC == 4) return launch_sliced<4, L::G, L::V>(x, plan, s.tile_major, bounds, partial, stream);
        else return hipErrorInvalidValue;
    });
    if (e != hipSuccess) return e;
    return slice_sum_launch((long long)x.M * x.N, plan.slices, partial, x.C, stream);
}

// ---- row plan ---------------------------------------------------------------------------------------

// A planned launch runs one row per four-wave workgroup in one column tile. Where the size rule groups several rows
// per workgroup (it was measured on even rows), a plan ungroups them if the rows are long enough: on lognormal rows
// (sigma 0.6 ... 1.2) one row per workgroup in plan order against the rule's grouping: 4096 x 1024, 99 per row, N = 256:
// 18.3 against 24.6 us; 8192 x 2048, 199 per row, N = 128: 29.1 against 37.5 us; 16384 x 512, 51 per row, N = 256: 31.4
// against 35.3 us; 65536 x 2048, 197 per row, N = 128: 223 against 232 us; but 32768 x 1024, 32 per row, N = 256: 46.6
// against 43.9 us; 16384 x 2048, 101 per row, N = 32: 17.7 against 14.2 us; rows below 32 nonzeros lose everywhere.
bool plan_ungroups(const DeviceInfo& dev, int M, int width, int nnz)
{
    const long long avg32 = 32ll * M, avg48 = 48ll * M, avg128 = 128ll * M;
    const long long cus = dev.cus;  // measured on 256 compute units: 4096, 8192 and 16384 rows
    if (!rule_on(kRulePlanUngroups)) return false;
    return nnz >= avg32 && (M <= 16 * cus || (width >= 128 && (M <= 32 * cus || (nnz >= avg48 && M <= 64 * cus) || nnz >= avg128)));
}

// The same question for SDDMM and the fused op, which gain less from one row per workgroup: lognormal rows, sigma 0.6, rule's
// grouping against one row per workgroup in plan order: mask 2048 x 2048, D = 64, 100 per row: fused 12.5 -> 8.6 us;
// 4096 x 1024: 14.2 -> 11.7 us; 8192 x 2048, D = 128, 197 per row: 76.9 -> 58.1 us; but 16384 x 2048, D = 128, 60 per row: 44.9 ->
// 55.8 us; 32768 x 4096, D = 64, 100 per row: 68.8 -> 88.1 us; 8192 x 8192, D = 64, 100 per row: equal (SDDMM alike).
// Up to eight rows per compute unit the plan's order wins whatever the length of the rows (lognormal rows, sigma 0.8,
// D = 64 / 128, rule's grouping against one row per workgroup in plan order: 2048 x 1024, 8 per row: fused 4.86 -> 4.44 us,
// SDDMM 3.71 -> 3.57 us; 24 per row: 6.04 -> 4.97 us, 4.26 -> 4.03 us; from 4096 rows on short rows lose).
bool plan_ungroups_dots(const DeviceInfo& dev, int M, int D, int nnz)
{
    const long long cus = dev.cus;  // measured on 256 compute units: 2048, 4096 and 8192 rows
    if (!rule_on(kRulePlanUngroups)) return false;
    if (M <= 8 * cus) return true;
    return (long long)nnz >= 32ll * M && (M <= 16 * cus || (D >= 128 && M <= 32 * cus && (long long)nnz >= 128ll * M));
}

// Very uneven rows (the longest at least twenty times the mean: lognormal row lengths from sigma = 1 on) in masks of 16 to
// 64 rows per compute unit: SDDMM and the fused op, which the size rule runs several rows per workgroup there, take
// 0.63 ... 0.93 of the time with one row per workgroup in plan order (8192 x 2048, 60 per row, sigma = 1: fused at D = 64
// 27.3 -> 17.5 us, SDDMM at D = 128 24.0 -> 17.6 us; 16384 x 4096, sigma = 1.5: 58.8 -> 44.1 and 59.2 -> 41.3 us); at
// sigma <= 0.6, or from 128 rows per compute unit on, the same choice loses 4 ... 100 %. The sizes cannot tell the two
// apart, so this applies on the caller's word only (DLSPM_HINT_ROWS_SKEWED; dlspm_advise says it from the longest row).
bool plan_ungroups_skewed(const DeviceInfo& dev, int M, int nnz)
{
    const long long cus = dev.cus;  // measured on 256 compute units: 8192 and 16384 rows
    return M > 16 * cus && M <= 64 * cus && (long long)nnz >= 32ll * M;
}

bool spmm_plan_applies(const DeviceInfo& dev, SpmmShape& s, int M, int N, int nnz)
{
    // one column tile, or tiles in tile-major order (a B beyond one L2): there the workgroups of one tile are consecutive,
    // as the plan's packing assumes; tiles in row-major order (B within the L2) keep the matrix order
    if (s.vec != 4 || s.W != 4 || (s.G * s.vec * s.V < N && !s.tile_major)) return false;
    if (s.R == 1) return true;
    if (!plan_ungroups(dev, M, N, nnz)) return false;
    s.R = 1;
    return true;
}

hipError_t spmm_planned_launch(const SpmmArgs& x, const SpmmShape& s, const int* plan, hipStream_t stream)
{
    if (x.M <= 0) return hipSuccess;
    const int *starts = plan, *ends = plan + x.M, *rows = plan + 2 * (size_t)x.M;
    return dispatch_layout(s, [&](auto l) {
        using L = decltype(l);
        if constexpr (L::VEC != 4) {
            return hipErrorInvalidValue;
        } else {
            const int col_tiles = (int)ceil_div(x.N, L::G * 4 * L::V);
            const long long blocks = (long long)x.M * col_tiles;
            if (blocks > 0x7fffffffLL) return hipErrorInvalidConfiguration;
            if (dense_fits_buffer(x.K, x.N))
                hipLaunchKernelGGL((spmm_planned_kernel<4, L::G, L::V, true>), dim3((unsigned)blocks), dim3(4 * 64), 0, stream, x.M,
                                   x.N, x.nnz, col_tiles, launch_flags(0) | (s.tile_major << kFlagTileOrderShift), starts, ends, rows, x.col_indices, x.values, x.B, x.C);
            else
                hipLaunchKernelGGL((spmm_planned_kernel<4, L::G, L::V, false>), dim3((unsigned)blocks), dim3(4 * 64), 0, stream, x.M,
                                   x.N, x.nnz, col_tiles, launch_flags(0) | (s.tile_major << kFlagTileOrderShift), starts, ends, rows, x.col_indices, x.values, x.B, x.C);
            return hipGetLastError();
        }
    });
}

// The same with a cut plan (CutPlan, launch.hpp): one workgroup per entry and column tile, then the kernel that adds the
// pieces of the cut rows in piece order.
// Cut rows are shared out by columns (spmm_shares_kernel) where one wave covers the width with lane groups of 16 to 64
// (33 ... 512 columns).
bool spmm_cut_by_columns(const SpmmShape& s, int N)
{
    return rule_on(kRuleCutRowsByColumns) && s.vec == 4 && s.G >= 16 && N <= s.G * 4 * s.V;
}

hipError_t spmm_pieces_launch(const SpmmArgs& x, const SpmmShape& s, const CutPlan& cp, void* plan, hipStream_t stream)
{
    if (x.M <= 0) return hipSuccess;
    const int* base = static_cast<const int*>(plan);
    const int *starts = base, *ends = base + cp.entries, *rows = base + 2 * (size_t)cp.entries,
              *slot_of = base + 3 * (size_t)cp.entries;
    float* pieces = reinterpret_cast<float*>(static_cast<char*>(plan) + cp.off_pieces);
    const bool by_columns = spmm_cut_by_columns(s, x.N);
    const hipError_t e = dispatch_layout(s, [&](auto l) {
        using L = decltype(l);
        if constexpr (L::VEC != 4) {
            return hipErrorInvalidValue;
        } else {
            const int col_tiles = (int)ceil_div(x.N, L::G * 4 * L::V);
            const long long blocks = (long long)cp.entries * col_tiles;
            if (blocks > 0x7fffffffLL) return hipErrorInvalidConfiguration;
            if constexpr (L::G >= 16) {
                if (by_columns) {
                    if (dense_fits_buffer(x.K, x.N))
                        hipLaunchKernelGGL((spmm_shares_kernel<4, L::G, L::V, true>), dim3((unsigned)cp.entries), dim3(4 * 64), 0,
                                           stream, x.M, x.N, x.nnz, launch_flags(0), cp.entries, starts, ends, rows, slot_of,
                                           x.col_indices, x.values, x.B, x.C);
                    else
                        hipLaunchKernelGGL((spmm_shares_kernel<4, L::G, L::V, false>), dim3((unsigned)cp.entries), dim3(4 * 64), 0,
                                           stream, x.M, x.N, x.nnz, launch_flags(0), cp.entries, starts, ends, rows, slot_of,
                                           x.col_indices, x.values, x.B, x.C);
                    return hipGetLastError();
                }
            }
            if (dense_fits_buffer(x.K, x.N))
                hipLaunchKernelGGL((spmm_pieces_kernel<4, L::G, L::V, true>), dim3((unsigned)blocks), dim3(4 * 64), 0, stream, x.M,
                                   x.N, x.nnz, col_tiles, launch_flags(0) | (s.tile_major << kFlagTileOrderShift), cp.entries, cp.slots, starts, ends, rows, slot_of,
                                   x.col_indices, x.values, x.B, x.C, pieces);
            else
                hipLaunchKernelGGL((spmm_pieces_kernel<4, L::G, L::V, false>), dim3((unsigned)blocks), dim3(4 * 64), 0, stream, x.M,
                                   x.N, x.nnz, col_tiles, launch_flags(0) | (s.tile_major << kFlagTileOrderShift), cp.entries, cp.slots, starts, ends, rows, slot_of,
                                   x.col_indices, x.values, x.B, x.C, pieces);
            return hipGetLastError();
        }
    });
    if (e != hipSuccess || by_columns) return e;
    return cut_rows_sum_launch(x.M, x.N, cp, plan, x.C, stream);
}

}  // namespace dlspm
