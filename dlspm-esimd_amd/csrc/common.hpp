// Shared device helpers for the gfx950 sparse kernels: vector load/store types, cross-lane moves
// (DPP inside 16-lane rows, ds_bpermute across rows) and the work split used by every kernel.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace dlspm {

constexpr int kWave = 64;

// ---- VEC floats per lane: dwordx4 (VEC = 4) or dword (VEC = 1) global accesses --------------------
template <int VEC> struct Vec;
// four floats that need only 4-byte alignment: global_load/store_dwordx4 accept any dword address
typedef float float4_dword_aligned __attribute__((ext_vector_type(4), aligned(4)));
template <> struct Vec<4> {
    float4 v;
    __device__ __forceinline__ static Vec zero() { return Vec{make_float4(0.f, 0.f, 0.f, 0.f)}; }
    // 16-byte aligned address (LDS)
    __device__ __forceinline__ static Vec load(const float* p) { return Vec{*reinterpret_cast<const float4*>(p)}; }
    __device__ __forceinline__ void store(float* p) const { *reinterpret_cast<float4*>(p) = v; }
    // any float address (global memory): rows of a dense operand whose width is not a multiple of 4 floats
    __device__ __forceinline__ static Vec gload(const float* p)
    {
        const float4_dword_aligned t = *reinterpret_cast<const float4_dword_aligned*>(p);
        return Vec{make_float4(t.x, t.y, t.z, t.w)};
    }
    // the same through a buffer descriptor: base + per-lane byte offset + wave-uniform byte offset, all 32-bit, summed
    // by the load itself (no address arithmetic in the wave's instruction stream)
    __device__ __forceinline__ static Vec bload(__amdgpu_buffer_rsrc_t rsrc, unsigned lane_bytes, unsigned row_bytes)
    {
        typedef unsigned u4 __attribute__((ext_vector_type(4)));
        const u4 t = __builtin_amdgcn_raw_buffer_load_b128(rsrc, lane_bytes, row_bytes, 0);
        return Vec{make_float4(__uint_as_float(t.x), __uint_as_float(t.y), __uint_as_float(t.z), __uint_as_float(t.w))};
    }
    __device__ __forceinline__ void gstore(float* p) const
    {
        float4_dword_aligned t = {v.x, v.y, v.z, v.w};
        *reinterpret_cast<float4_dword_aligned*>(p) = t;
    }
    // The same with the non-temporal hint where `streaming` (wave-uniform) says so. Written out as an instruction: a
    // hinted store on one side of a branch and a plain one on the other are merged into one plain store by the
    // compiler. (A vector store like any other; the wait counts the compiler inserts can only become stricter by it.)
    __device__ __forceinline__ void gstore(float* p, bool streaming) const
    {
        if (streaming) {
            typedef float f4 __attribute__((ext_vector_type(4)));
            const f4 t = {v.x, v.y, v.z, v.w};
            // s_nop 1: on the gfx940 family a vector-memory store of more than 8 bytes still reads its data registers for
            // two wait states after it issues, and a VALU write of those registers must not come earlier (the "VMEM store
            // of more than 64 bits, then a write of the VGPRs holding its data" row of the ISA guide's table of wait
            // states the program must insert; the compiler keeps two independent instructions or `s_nop 1` there for its
            // own dwordx4 stores). It cannot see that this asm is such a store, so the two wait states are spent here,
            // whatever it schedules behind. (The dword store below reads its data as it issues and needs none.)
            asm volatile("global_store_dwordx4 %0, %1, off nt\n\ts_nop 1" : : "v"(p), "v"(t) : "memory");
        } else {
            gstore(p);
        }
    }
    // elements [d, d+4) of a row of D >= 4 floats, d < D, for sums over the row: a lane whose four elements
    // would run past D reads the last four instead and zeroes the ones its left neighbour already covers
    __device__ __forceinline__ static Vec gload_clip(const float* row, int d, int D)
    {
        const int dl = min(d, D - 4);
        Vec t = gload(row + dl);
        const int ov = d - dl;
        t.v.x = ov > 0 ? 0.f : t.v.x;
        t.v.y = ov > 1 ? 0.f : t.v.y;
        t.v.z = ov > 2 ? 0.f : t.v.z;
        return t;
    }
    // zeroes the first `n` of the four elements (n >= 4: all of them), one select each and no branch
    __device__ __forceinline__ void zero_first(int n)
    {
        v.x = n > 0 ? 0.f : v.x;
        v.y = n > 1 ? 0.f : v.y;
        v.z = n > 2 ? 0.f : v.z;
        v.w = n > 3 ? 0.f : v.w;
    }
    __device__ __forceinline__ void fma(float a, const Vec& b)
    {
        v.x = fmaf(a, b.v.x, v.x); v.y = fmaf(a, b.v.y, v.y); v.z = fmaf(a, b.v.z, v.z); v.w = fmaf(a, b.v.w, v.w);
    }
    __device__ __forceinline__ void add(const Vec& b) { v.x += b.v.x; v.y += b.v.y; v.z += b.v.z; v.w += b.v.w; }
    __device__ __forceinline__ float dot(const Vec& b, float acc) const
    {
        acc = fmaf(v.x, b.v.x, acc); acc = fmaf(v.y, b.v.y, acc); acc = fmaf(v.z, b.v.z, acc); acc = fmaf(v.w, b.v.w, acc);
        return acc;
    }
};
template <> struct Vec<1> {
    float v;
    __device__ __forceinline__ static Vec zero() { return Vec{0.f}; }
    __device__ __forceinline__ static Vec load(const float* p) { return Vec{*p}; }
    __device__ __forceinline__ void store(float* p) const { *p = v; }
    __device__ __forceinline__ static Vec gload(const float* p) { return Vec{*p}; }
    __device__ __forceinline__ static Vec bload(__amdgpu_buffer_rsrc_t rsrc, unsigned lane_bytes, unsigned row_bytes)
    {
        return Vec{__uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(rsrc, lane_bytes, row_bytes, 0))};
    }
    __device__ __forceinline__ void gstore(float* p) const { *p = v; }
    __device__ __forceinline__ void gstore(float* p, bool streaming) const
    {
        if (streaming) asm volatile("global_store_dword %0, %1, off nt" : : "v"(p), "v"(v) : "memory");
        else *p = v;
    }
    __device__ __forceinline__ static Vec gload_clip(const float* row, int d, int) { return Vec{row[d]}; }
    __device__ __forceinline__ void zero_first(int n) { v = n > 0 ? 0.f : v; }
    __device__ __forceinline__ void fma(float a, const Vec& b) { v = fmaf(a, b.v, v); }
    __device__ __forceinline__ void add(const Vec& b) { v += b.v; }
    __device__ __forceinline__ float dot(const Vec& b, float acc) const { return fmaf(v, b.v, acc); }
};

// arguments of amdgpu_waves_per_eu for a kernel of `waves` waves per workgroup (four SIMDs per compute unit)
constexpr int waves_per_simd_least(int waves) { return waves > 4 ? (waves + 3) / 4 : 1; }
constexpr int waves_per_simd_most(int waves, int wanted) { return wanted > waves_per_simd_least(waves) ? wanted : waves_per_simd_least(waves); }

// ---- cross-lane ---------------------------------------------------------------------------------
// value of `x` in lane `src` (any lane of the wave), through the LDS crossbar (ds_bpermute_b32)
__device__ __forceinline__ int lane_get(int x, int src) { return __builtin_amdgcn_ds_bpermute(src << 2, x); }
__device__ __forceinline__ float lane_get(float x, int src)
{
    return __int_as_float(__builtin_amdgcn_ds_bpermute(src << 2, __float_as_int(x)));
}
// wave-uniform source lane: v_readlane_b32 into an SGPR
__device__ __forceinline__ int lane_bcast(int x, int src) { return __builtin_amdgcn_readlane(x, src); }
__device__ __forceinline__ float lane_bcast(float x, int src)
{
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(x), src));
}

// DPP move inside a 16-lane row; CTRL is the dpp_ctrl immediate
template <int CTRL> __device__ __forceinline__ float dpp_move(float x)
{
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xF, 0xF, true));
}
constexpr int kDppQuadSwap1 = 0xB1;      // quad_perm [1,0,3,2]: lane ^ 1
constexpr int kDppQuadSwap2 = 0x4E;      // quad_perm [2,3,0,1]: lane ^ 2
constexpr int kDppRowHalfMirror = 0x141; // lane i <-> 7 - i inside each group of 8
constexpr int kDppRowMirror = 0x140;     // lane i <-> 15 - i inside each row of 16

// x[lane] + x[lane ^ 8 | 16 | 32] in every lane, without touching LDS: a DPP row rotate for 8, and the gfx950
// v_permlane16_swap / v_permlane32_swap (which exchange the odd 16- or 32-lane blocks of one register with the
// even blocks of another; applied to two copies of x they leave (even, even) and (odd, odd) copies to add).
constexpr int kDppRowRor8 = 0x128;
__device__ __forceinline__ float add_xor8(float x) { return x + dpp_move<kDppRowRor8>(x); }
__device__ __forceinline__ float add_xor16(float x)
{
    const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float add_xor32(float x)
{
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
template <int STEP> __device__ __forceinline__ float add_xor(float x)
{
    static_assert(STEP == 8 || STEP == 16 || STEP == 32, "cross-group sums start at 8 lanes");
    if constexpr (STEP == 8) return add_xor8(x);
    else if constexpr (STEP == 16) return add_xor16(x);
    else return add_xor32(x);
}

// Sum of x over aligned groups of G lanes, result in every lane of the group. G in {1,2,4,8,16,32,64}.
// Must be called with all lanes of the wave active.
template <int G> __device__ __forceinline__ float group_sum(float x)
{
    if constexpr (G >= 2) x += dpp_move<kDppQuadSwap1>(x);
    if constexpr (G >= 4) x += dpp_move<kDppQuadSwap2>(x);
    if constexpr (G >= 8) x += dpp_move<kDppRowHalfMirror>(x);  // quads already uniform: mirror pairs quad 0 with quad 1
    if constexpr (G >= 16) x += dpp_move<kDppRowMirror>(x);     // halves already uniform: mirror pairs the two halves
    if constexpr (G >= 32) x = add_xor16(x);
    if constexpr (G >= 64) x = add_xor32(x);
    return x;
}

// Asks for kernel arguments now: the compiler otherwise fetches a pointer from the argument segment only where it
// is first used, and that scalar load then sits in the middle of the kernel's chain of dependent memory accesses
// (row offsets -> column indices -> dense rows). Fetched together at entry, they cost one round trip in all.
template <typename P> __device__ __forceinline__ void fetch_arg_now(P p) { asm volatile("" : : "s"(p)); }
template <typename... P> __device__ __forceinline__ void fetch_args_now(P... p) { (fetch_arg_now(p), ...); }

// ---- work split -----------------------------------------------------------------------------------
// A workgroup of W waves owns a block of consecutive rows holding T nonzeros in all; wave w takes the
// contiguous nonzero range [w*per, (w+1)*per) of them (clipped to T) regardless of row boundaries.
__host__ __device__ __forceinline__ int split_per_wave(int T, int W)
{
    int per = (T + W - 1) / W;
    return per < 1 ? 1 : per;
}

// Lane i <- sum of x over the lanes below i, for i < 32 (five rounds through the LDS crossbar; the whole wave calls it).
__device__ __forceinline__ int lanes_exclusive_sum32(int x, int lane)
{
    int inc = x;
#pragma unroll
    for (int d = 1; d < 32; d *= 2) {
        const int y = lane_get(inc, lane >= d ? lane - d : lane);
        inc += lane >= d ? y : 0;
    }
    return inc - x;
}

// Row-aligned variant of that split, used when it is nearly as even: with R = k*W rows per workgroup wave w takes the
// k rows w*k .. w*k+k-1 whole; with W = m*R waves per row the m waves of a row take equal parts of it. A wave then
// never works on the tail of one row and the head of the next (two dependent chains of memory accesses in sequence),
// whole rows are stored without a partial sum, and a matrix of even rows loses nothing in balance (measured on
// 2048x2048, 102-103 nonzeros per row, D = 128: 6.2 -> 5.7 us). It is taken when no wave would get more than 5/4 of
// the even share `per`; every wave of the workgroup evaluates the same test on the same offsets. `off(i)` returns
// row offset i of the block (i <= nr); the offsets of rows past nr count as off(nr).
template <int W, int R, typename Off> __host__ __device__ __forceinline__ bool split_is_row_aligned(Off&& off, int nr, int per)
{
    if constexpr (R == 1) {
        return false;  // one row per workgroup: the even split is the aligned one
    } else {
        const int cap = per + (per >> 2);
        int worst = 0;
        if constexpr (R % W == 0) {
            constexpr int k = R / W;
            for (int x = 0; x < W; ++x) {
                const int lo = x * k < nr ? x * k : nr, hi = (x + 1) * k < nr ? (x + 1) * k : nr;
                const int load = off(hi) - off(lo);
                worst = load > worst ? load : worst;
            }
        } else {
            static_assert(W % R == 0, "rows per workgroup and waves per workgroup divide one another");
            constexpr int m = W / R;
            for (int r = 0; r < nr; ++r) {
                const int load = (off(r + 1) - off(r) + m - 1) / m;
                worst = load > worst ? load : worst;
            }
        }
        return worst <= cap;
    }
}
// nonzero range [a, b) of wave w (absolute positions), for either split
template <int W, int R, typename Off>
__host__ __device__ __forceinline__ void wave_range(bool aligned, Off&& off, int nr, int w, int T0, int T, int per, int& a,
                                                    int& b)
{
    if (!aligned) {
        a = T0 + (T < w * per ? T : w * per);
        b = T0 + (T < (w + 1) * per ? T : (w + 1) * per);
    } else if constexpr (R % W == 0) {
        constexpr int k = R / W;
        a = off(w * k < nr ? w * k : nr);
        b = off((w + 1) * k < nr ? (w + 1) * k : nr);
    } else {
        constexpr int m = W / R;
        const int r = w / m, j = w % m;
        if (r >= nr) {
            a = b = T0 + T;
        } else {
            const int rs = off(r), len = off(r + 1) - rs;
            const int part = (len + m - 1) / m;
            a = rs + (len < j * part ? len : j * part);
            b = rs + (len < (j + 1) * part ? len : (j + 1) * part);
        }
    }
}

// ---- the rows of one workgroup (row-block kernels of all three ops) -------------------------------------------
// A workgroup of W waves owns R consecutive rows ("row block" rb). RowBlock reads their offsets, splits their nonzeros
// over the waves and walks wave w's share segment by segment (a segment = the part of one row inside the share).
//   SLICED = false: row i owns the nonzeros [row_offsets[i], row_offsets[i + 1]).
//   SLICED = true:  row i owns [row_offsets[i], row_ends[i]), a part of the CSR row (its columns inside one range of
//                   columns), so the rows of a block are not contiguous in memory: the split then works on the running
//                   sum of their lengths ("virtual" offsets, 0 at the block's first row) and every segment is shifted
//                   back to where it lies in memory.
//   PLANNED (with SLICED and R == 1): workgroup i works on row row_ids[i], whose nonzeros are
//                   [row_offsets[i], row_ends[i]): a row plan hands the rows out in an order of its own.
//                   kPlanPieces: the entry may be a PIECE of a row (a row longer than one compute unit's share of the
//                   nonzeros is cut into several entries): row_slots[i] is -1 for a whole row, s >= 0 for a piece whose
//                   partial row goes to slot s of a buffer of partial rows (a second kernel adds the pieces of a row
//                   in order), and below -1 for an entry that holds nothing (the plan has room for the most pieces
//                   any matrix of its height can need).
// The R + 1 offsets are read without LDS or a barrier: with R == 1 they are the same two words for every lane (scalar
// loads); otherwise lane i of every wave holds offset i and v_readlane picks one.
constexpr int kPlanNone = 0, kPlanRows = 1, kPlanPieces = 2;
// What a cut plan says of an entry that is a piece of a row, in one word: the slot of its partial row | which piece of the
// row it is << 15 | log2 of the number of pieces << 23. A row is cut into 2, 4, ... 256 equal pieces, and the entry
// holds the range of the WHOLE row: piece k of c takes the nonzeros piece_range() says, or 1/c of the columns.
constexpr int kPieceSlotMask = 0x7FFF, kPieceNumberShift = 15, kPieceNumberMask = 0xFF, kPieceCountShift = 23, kPieceCountMask = 0xF;
constexpr int kMaxPiecesOfARow = 256;
// piece k of 1 << lg of a row of len nonzeros: [*first, *first + *count) of the row
__device__ __forceinline__ void piece_range(int len, int word, int* first, int* count)
{
    const int k = (word >> kPieceNumberShift) & kPieceNumberMask, lg = (word >> kPieceCountShift) & kPieceCountMask;
    const int piece = (len + (1 << lg) - 1) >> lg;
    *first = min(len, k * piece);
    *count = min(piece, len - *first);
}
template <int W, int R, bool SLICED, int PLANNED>
struct RowBlock {
    static_assert(!PLANNED || (SLICED && R == 1), "a row plan names one row per workgroup");
    int lane, w;
    int piece = -1;  // kPlanPieces: the entry's slot among the partial rows, -1 a whole row, below -1 nothing
    int rows_total;  // rows of the matrix
    int stream_rule;  // results with the non-temporal hint: 0 by the size rule, 1 never, 2 always (launch flags, bits 1-2)
    int nr;    // rows in this block (fewer than R at the end of the matrix)
    int row0;  // row of the dense operands and of the output that belongs to the block's first row
    int off_lo, off_hi, off_win, start_lo, start_win;
    int T0, T, per, a, b;  // first offset, nonzeros of the block, even share of a wave, this wave's range [a, b)
    bool aligned;          // the row-aligned split is in use (the same for every wave of the workgroup)

    // `prefetch()` is called right after the offsets were requested: what it asks for arrives in the same round trip
    // `flags`: the launch flags (launch.hpp). Bit 0, XCD-contiguous (plain row blocks in one column tile only): workgroup
    // 8 i + x runs on XCD x, as the hardware deals them; it then takes row block i of XCD x's own contiguous run of row
    // blocks instead of row block 8 i + x.
    template <typename Prefetch>
    __device__ __forceinline__ void load(int rb, int M, int nnz, const int* __restrict__ row_offsets,
                                         const int* __restrict__ row_ends, const int* __restrict__ row_ids,
                                         Prefetch&& prefetch, int flags = 0, const int* __restrict__ row_slots = nullptr,
                                         int slots = 0)
    {
        lane = threadIdx.x & 63;
        w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
        rows_total = M;
        stream_rule = (flags >> 1) & 3;
        if constexpr (!SLICED && !PLANNED) {
            if (flags & 1) {
                const int nb = (M - 1) / R + 1, x = rb & 7, each = nb >> 3, extra = nb & 7;
                rb = x * each + min(x, extra) + (rb >> 3);  // XCD x owns each + (x < extra) row blocks
            }
        }
        const int r0 = rb * R;
        nr = PLANNED ? 1 : min(R, M - r0);
        row0 = r0;
        off_lo = off_hi = off_win = start_lo = start_win = 0;
        if constexpr (!SLICED) {
            if constexpr (R == 1) {
                off_lo = row_offsets[r0];
                off_hi = row_offsets[r0 + 1];
            } else {
                static_assert(R + 1 <= kWave, "one offset per lane");
                off_win = row_offsets[r0 + min(lane, nr)];
            }
        } else {
            if constexpr (R == 1) {
                start_lo = row_offsets[r0];
                off_hi = row_ends[r0] - start_lo;
                if constexpr (PLANNED) {
                    // a plan that was built for another matrix must not take the kernel outside the arrays
                    row0 = min(max(row_ids[r0], 0), M - 1);
                    start_lo = min(max(start_lo, 0), nnz);
                    off_hi = min(max(off_hi, 0), nnz - start_lo);
                    if constexpr (PLANNED == kPlanPieces) {
                        const int word = row_slots[r0];  // -1 a whole row, -2 nothing, else a piece of the row entered here
                        piece = word < 0 ? word : min(word & kPieceSlotMask, slots - 1);
                        if (word >= 0) {
                            int first, count;
                            piece_range(off_hi, word, &first, &count);
                            start_lo += first;
                            off_hi = count;
                        }
                    }
                }
            } else {
                static_assert(R + 1 <= 32, "the running sum covers 32 lanes");
                const int i = r0 + min(lane, nr - 1);
                start_win = row_offsets[i];
                off_win = lanes_exclusive_sum32(lane < nr ? row_ends[i] - start_win : 0, lane);
            }
        }
        prefetch();
        split(flags);
    }
    // the work split of the block over its waves, from the offsets that load() left
    __device__ __forceinline__ void split(int flags)
    {
        T0 = off(0);
        T = off(nr) - T0;
        per = split_per_wave(T, W);
        auto o = [&](int i) { return off(i); };
        aligned = (flags & 8) == 0 && split_is_row_aligned<W, R>(o, nr, per);  // (bit 3: the rule is switched off for a measurement)
        int a_, b_;
        wave_range<W, R>(aligned, o, nr, w, T0, T, per, a_, b_);
        a = __builtin_amdgcn_readfirstlane(a_);
        b = __builtin_amdgcn_readfirstlane(b_);
    }
    // offset i of the block in the split (i <= nr)
    __device__ __forceinline__ int off(int i) const
    {
        if constexpr (R == 1) return i == 0 ? off_lo : off_hi;
        else return __builtin_amdgcn_readlane(off_win, __builtin_amdgcn_readfirstlane(i));
    }
    // where row i's first nonzero lies in memory, minus its offset in the split
    __device__ __forceinline__ int shift(int i) const
    {
        if constexpr (!SLICED) return 0;
        else if constexpr (R == 1) return start_lo;
        else return __builtin_amdgcn_readlane(start_win, __builtin_amdgcn_readfirstlane(i)) - off(i);
    }
    // f(r, p, q, rs, re) for every segment [p, q) of this wave's range, in order: r = row of the block, [rs, re) that
    // row's whole range (all in split positions; add shift(r) for memory positions); rows without nonzeros are skipped
    template <typename F> __device__ __forceinline__ void for_each_segment(F&& f) const
    {
        if (a >= b) return;
        int r = 0;
        while (off(r + 1) <= a) ++r;  // first row owning nonzero `a`; exists because a < off(nr)
        int pos = a;
        while (pos < b) {
            const int rs = off(r);
            const int re = off(r + 1);
            const int q = __builtin_amdgcn_readfirstlane(min(re, b));
            const int p = __builtin_amdgcn_readfirstlane(pos);
            f(r, p, q, rs, re);
            pos = q;
            ++r;
            while (r < nr && off(r + 1) <= pos) ++r;
        }
    }
};

// A row block whose result is one dense row per CSR row (SpMM, the fused op): the lanes' columns, the segments of this
// wave, and the rows' sums. `segment(acc, r, p, q, colv)` leaves in acc[v] the sum over the nonzeros [p, q) (memory
// positions) of block row r for this lane's columns colv[v] .. colv[v] + VEC of column tile ct. Rows finished inside one
// wave are stored straight to `out` (row blk.row0 + r, `width` floats per row); rows shared by several waves leave
// per-wave partial sums in LDS which are added in wave order after one barrier, so the result does not depend on
// timing (no atomics, no pre-zeroed output); rows without nonzeros are written as zeros.
// kPlanPieces: an entry that is a piece of a row stores its sum to `pieces` (slot blk.piece) instead, with ordinary stores
// (it is read again), and an entry that holds nothing leaves at once (the whole workgroup, before any barrier).
// The window form works on the columns [col0, col_end) of rows of `width` floats, col_end - col0 <= G * VEC * V and >= VEC;
// the tile form on column tile ct of the whole width.
template <int VEC, int G, int V, int W, int R, bool SLICED, int PLANNED, typename Segment>
__device__ __forceinline__ void dense_rows_window(const RowBlock<W, R, SLICED, PLANNED>& blk, int col0, int col_end, int width,
                                                  float* __restrict__ out, Segment&& segment,
                                                  float* __restrict__ pieces = nullptr);
template <int VEC, int G, int V, int W, int R, bool SLICED, int PLANNED, typename Segment>
__device__ __forceinline__ void dense_rows_block(const RowBlock<W, R, SLICED, PLANNED>& blk, int ct, int width,
                                                 float* __restrict__ out, Segment&& segment,
                                                 float* __restrict__ pieces = nullptr)
{
    dense_rows_window<VEC, G, V>(blk, ct * (G * VEC * V), width, width, out, static_cast<Segment&&>(segment), pieces);
}
template <int VEC, int G, int V, int W, int R, bool SLICED, int PLANNED, typename Segment>
__device__ __forceinline__ void dense_rows_window(const RowBlock<W, R, SLICED, PLANNED>& blk, int col0, int col_end, int width,
                                                  float* __restrict__ out, Segment&& segment, float* __restrict__ pieces)
{
    if constexpr (PLANNED == kPlanPieces) {
        if (blk.piece < -1) return;
    }
    constexpr int TW = G * VEC * V;  // columns covered by one wave
    constexpr int NP = R == 1 ? 1 : 2;  // with one row per workgroup a wave never ends a second segment
    using VecT = Vec<VEC>;
    __shared__ __attribute__((aligned(16))) float s_part[W][NP][TW];

    const int lane = blk.lane, w = blk.w, nr = blk.nr;
    const int g = lane % G;
    const int slot = lane / G;
    int colv[V];  // first of this lane's VEC columns for access v; clamped to a valid column when outside
    bool act[V];
#pragma unroll
    for (int v = 0; v < V; ++v) {
        const int col = col0 + (v * G + g) * VEC;
        act[v] = col < col_end;
        // a lane whose VEC columns would run past the end moves back to end there: it then repeats columns of its
        // left neighbour, with the same operations, and stores the same values there (col_end - col0 >= VEC)
        colv[v] = act[v] ? min(col, col_end - VEC) : 0;
    }
    auto s_off = [&](int i) { return blk.off(i); };
    const int T0 = blk.T0, T = blk.T, per = blk.per, a = blk.a;
    // Results of kStreamedOutputFloats (4 MiB, one L2's worth) and more are stored with the non-temporal hint: they are
    // written once, and ordinary stores are held in the L2 as dirty lines to be written back later, where hinted ones
    // drain as they are issued (hits, misses and fetched bytes of the L2 stay the same; the time does not). Measured with
    // both kinds of store in one process (SpMM): 4-8 MiB -0.5 ... -1.3 %; 8192 x 1024 at 5 %, N = 1024 (32 MiB)
    // 58.3 -> 56.9 us; 65536 x 1024 at 2 %, N = 256 (64 MiB) 52.3 -> 49.2 us; 131072 x 512, N = 128 41.2 -> 38.8 us;
    // fused 65536 x 2048, D = 64 (16 MiB) 42.3 -> 40.8 us. Below 4 MiB there is nothing to gain (+-0.8 %). Not for the
    // partial rows of the column-sliced schedule, which are read again.
    constexpr long long kStreamedOutputFloats = 1024 * 1024;
    const long long out_floats = (long long)blk.rows_total * width;
    // (dlspm_tuning.stream_results switches the rule off or on for sweeps and tests: blk.stream_rule)
    const bool streaming = (!SLICED || PLANNED) && blk.stream_rule != 1 && (PLANNED != kPlanPieces || blk.piece < 0) &&
                           (blk.stream_rule == 2 || out_floats >= kStreamedOutputFloats);
    // where row r of the block is stored
    auto out_row = [&](int r) -> float* {
        if constexpr (PLANNED == kPlanPieces) {
            if (blk.piece >= 0) return pieces + (size_t)blk.piece * width;
        }
        return out + (size_t)(blk.row0 + r) * width;
    };

    blk.for_each_segment([&](int r, int p, int q, int rs, int re) {
        VecT acc[V];
        const int shift = blk.shift(r);
        segment(acc, r, p + shift, q + shift, colv);
        const bool whole_row = (p == rs) && (q == re);
        if (slot == 0) {
            if (whole_row) {
                float* orow = out_row(r);
#pragma unroll
                for (int v = 0; v < V; ++v)
                    if (act[v]) acc[v].gstore(orow + colv[v], streaming);
            } else {
                float* part = s_part[w][(NP == 1 || p == a) ? 0 : 1];
#pragma unroll
                for (int v = 0; v < V; ++v) acc[v].store(part + (v * G + g) * VEC);
            }
        }
    });
    if (blk.aligned) {  // R > 1 only, and the same for every wave of the workgroup
        if constexpr (R % W == 0) {
            // every wave stored its rows whole: nothing to combine, no barrier; rows without nonzeros are left
            if (slot == 0) {
                for (int r = w; r < nr; r += W) {
                    if (s_off(r) != s_off(r + 1)) continue;
                    float* orow = out + (size_t)(blk.row0 + r) * width;
#pragma unroll
                    for (int v = 0; v < V; ++v)
                        if (act[v]) VecT::zero().gstore(orow + colv[v], streaming);
                }
            }
        } else {
            // the m = W/R waves of a row hold its parts in order, each in its first partial slot
            constexpr int m = W / R;
            __syncthreads();
            if (slot == 0) {
                for (int r = w; r < nr; r += W) {
                    const int len = s_off(r + 1) - s_off(r);
                    const int part = (len + m - 1) / m;
                    float* orow = out + (size_t)(blk.row0 + r) * width;
                    if (len > 0 && len <= part) continue;  // one wave held the whole row and stored it
#pragma unroll
                    for (int v = 0; v < V; ++v) {
                        VecT sum = VecT::zero();
#pragma unroll
                        for (int j = 0; j < m; ++j)
                            if (j * part < len) sum.add(VecT::load(&s_part[r * m + j][0][(v * G + g) * VEC]));
                        if (act[v]) sum.gstore(orow + colv[v], streaming);
                    }
                }
            }
        }
        return;
    }
    __syncthreads();

    if constexpr (R == 1) {
        // one row per workgroup: wave x had nonzeros iff x * per < T, and wave 0 adds them up (no division, the
        // partial sums of all waves are requested from LDS together)
        if (w == 0 && slot == 0) {
            float* orow = out_row(0);
            if (T == 0) {
#pragma unroll
                for (int v = 0; v < V; ++v)
                    if (act[v]) VecT::zero().gstore(orow + colv[v], streaming);
            } else if (T > per) {  // T <= per: wave 0 held the whole row and has stored it
#pragma unroll
                for (int v = 0; v < V; ++v) {
                    VecT sum = VecT::zero();
#pragma unroll
                    for (int x = 0; x < W; ++x)
                        if (x * per < T) sum.add(VecT::load(&s_part[x][0][(v * G + g) * VEC]));
                    if (act[v]) sum.gstore(orow + colv[v], streaming);
                }
            }
        }
        return;
    }
    // rows shared by several waves: add the partial sums in wave order; empty rows: write zeros
    if (slot == 0) {
        for (int r = w; r < nr; r += W) {
            const int rs = s_off(r);
            const int re = s_off(r + 1);
            float* orow = out + (size_t)(blk.row0 + r) * width;
            if (rs == re) {
#pragma unroll
                for (int v = 0; v < V; ++v)
                    if (act[v]) VecT::zero().gstore(orow + colv[v], streaming);
                continue;
            }
            const int wl = (rs - T0) / per;
            const int wh = (re - 1 - T0) / per;
            if (wl == wh) continue;  // finished inside one wave, already stored
#pragma unroll
            for (int v = 0; v < V; ++v) {
                VecT sum = VecT::zero();
                for (int x = wl; x <= wh; ++x) {
                    const int k = (NP == 2 && x == wl && T0 + x * per != rs) ? 1 : 0;
                    sum.add(VecT::load(&s_part[x][k][(v * G + g) * VEC]));
                }
                if (act[v]) sum.gstore(orow + colv[v], streaming);
            }
        }
    }
}

// ---- flat schedule: every wave owns `chunk` consecutive nonzeros of the whole matrix ------------------------
// Largest row r with row_offsets[r] <= pos, for 0 <= pos < row_offsets[M] (so the row is not empty and holds
// nonzero `pos`). A 64-ary search by the whole wave: each round reads 64 evenly spaced offsets with one load and
// narrows the interval to one of 65 parts; ceil(log64(M)) dependent loads. Everything is wave-uniform.
__device__ __forceinline__ int find_row(const int* __restrict__ row_offsets, int M, int pos, int lane)
{
    int lo = 0, hi = M;  // row_offsets[lo] <= pos < row_offsets[hi]
    while (hi - lo > 1) {
        const long long span = hi - lo;
        const int idx = lo + (int)((span * (lane + 1)) >> 6);  // non-decreasing in lane, lane 63 reads `hi`
        const unsigned long long le = __ballot(row_offsets[idx] <= pos);  // a prefix of the lanes
        const int n = min(__popcll(le), 63);  // < 64 because row_offsets[hi] > pos (clamped: offsets that are not
                                              // sorted must not take the search outside [0, M])
        const int new_lo = lo + (int)((span * n) >> 6);        // n == 0: lo itself
        const int new_hi = lo + (int)((span * (n + 1)) >> 6);  // first sample above pos
        lo = __builtin_amdgcn_readfirstlane(new_lo);
        hi = __builtin_amdgcn_readfirstlane(new_hi);
    }
    return lo;
}

// 64 consecutive row offsets in the lanes of one register (offsets past M repeat row_offsets[M]); entry j is read
// with v_readlane. Rows rbase .. rbase+62 have both their ends inside the window.
constexpr int kWinRows = 63;
__device__ __forceinline__ int window_load(const int* __restrict__ row_offsets, int M, int rbase, int lane)
{
    return row_offsets[min(rbase + lane, M)];
}
__device__ __forceinline__ int window_get(int win, int j)
{
    return __builtin_amdgcn_readlane(win, __builtin_amdgcn_readfirstlane(j));
}
// First row after the one that ended at `pos` that holds nonzero `pos` (rows without nonzeros are skipped), for
// pos < row_offsets[M]. Reloads the window (by search) when that row is not inside it.
__device__ __forceinline__ int window_next_row(const int* __restrict__ row_offsets, int M, int pos, int lane, int& win,
                                               int& rbase)
{
    const unsigned long long gt = __ballot(win > pos);  // a suffix of the lanes: entries are non-decreasing
    if (gt != 0) {
        const int t = __builtin_ctzll(gt);  // smallest entry above pos: the row ends there, so it is row t - 1
        return min(rbase + max(t, 1) - 1, M - 1);  // t >= 1 (entry 0 starts a row at or before pos) and the row is
                                                   // below M for sorted offsets; clamped for unsorted ones
    }
    const int r = find_row(row_offsets, M, pos, lane);
    rbase = r;
    win = window_load(row_offsets, M, rbase, lane);
    return r;
}

// ---- dense-row accumulation (SpMM kernel and stage 2 of the fused kernel) -----------------------------
// A dense operand of fewer than 4 GiB as a raw buffer (stride 0, no swizzle, 32-bit data format): the descriptor that
// buffer loads take. Their address is base + lane offset + wave-uniform offset, so a row of B needs one scalar multiply
// (column x row pitch) where a global load needs a 64-bit multiply, shift and add on the scalar unit plus a 64-bit add
// per access on the vector unit.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t dense_buffer(const float* p)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p), 0, -1, 0x00020000);
}

// The wave holds `cnt` <= 64 nonzeros of one row segment, one per lane: column index `c` and value `av`
// (lanes >= cnt hold c = 0, av = 0). Adds sum_j av_j * dense[c_j, colv[v] .. colv[v]+VEC) into acc[v].
// G lanes cover one dense row; the S = 64/G lane groups ("slots") take different nonzeros j = t*S + slot.
// Loads are issued U dense rows at a time before the first FMA so that U*V requests per lane are in
// flight. `colv` must be a valid column for every lane (lanes outside the matrix pass a safe column and
// simply never store their accumulator), so the loop body has no predicates.
// BUF (dense operand below 4 GiB, fewer than 2^24 rows of fewer than 2^24 bytes): the rows are read with buffer loads
// (dense_buffer above); with G < 64 every lane group has its own row, whose offset is then one 24-bit multiply-add per
// access on the vector unit instead of a 64-bit multiply, shift and add.
template <int VEC, int G, int V, bool BUF = false>
__device__ __forceinline__ void dense_rows_fma(Vec<VEC>* acc, int c, float av, int cnt, const float* __restrict__ dense,
                                               int ld, const int* colv, int lane)
{
    using VecT = Vec<VEC>;
    constexpr int S = kWave / G;
    constexpr int U = V >= 4 ? 2 : 8 / V;
    const int slot = lane / G;
    const int full = cnt / S;  // steps in which every slot has a nonzero
    unsigned offv[V];  // BUF: the lane's columns as byte offsets into a dense row
#pragma unroll
    for (int v = 0; v < V; ++v) offv[v] = (unsigned)colv[v] * (unsigned)sizeof(float);
    const unsigned pitch = (unsigned)ld * (unsigned)sizeof(float);
    const __amdgpu_buffer_rsrc_t rsrc = dense_buffer(dense);
    // dense row cj, access v of this lane
    auto row_load = [&](int cj, int v) -> VecT {
        if constexpr (BUF && S == 1) return VecT::bload(rsrc, offv[v], (unsigned)cj * pitch);
        else if constexpr (BUF) return VecT::bload(rsrc, __umul24((unsigned)cj, pitch) + offv[v], 0u);
        else return VecT::gload(dense + (size_t)cj * ld + colv[v]);
    };
    int t = 0;
    for (; t + U <= full; t += U) {
        VecT bv[U][V];
        float aj[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            int cj;
            if constexpr (S == 1) {
                cj = lane_bcast(c, t + u);
                aj[u] = lane_bcast(av, t + u);
            } else {
                cj = lane_get(c, (t + u) * S + slot);
                aj[u] = lane_get(av, (t + u) * S + slot);
            }
#pragma unroll
            for (int v = 0; v < V; ++v) bv[u][v] = row_load(cj, v);
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int v = 0; v < V; ++v) acc[v].fma(aj[u], bv[u][v]);
    }
    if (t < full) {  // fewer than U steps left: same batching, each step guarded by a wave-uniform test
        const int rem = full - t;
        VecT bv[U - 1][V];
        float aj[U - 1];
#pragma unroll
        for (int u = 0; u < U - 1; ++u) {
            if (u < rem) {
                int cj;
                if constexpr (S == 1) {
                    cj = lane_bcast(c, t + u);
                    aj[u] = lane_bcast(av, t + u);
                } else {
                    cj = lane_get(c, (t + u) * S + slot);
                    aj[u] = lane_get(av, (t + u) * S + slot);
                }
#pragma unroll
                for (int v = 0; v < V; ++v) bv[u][v] = row_load(cj, v);
            }
        }
#pragma unroll
        for (int u = 0; u < U - 1; ++u) {
            if (u < rem) {
#pragma unroll
                for (int v = 0; v < V; ++v) acc[v].fma(aj[u], bv[u][v]);
            }
        }
    }
    if constexpr (S > 1) {
        if (full * S < cnt) {  // last step: only the first cnt - full*S slots have a nonzero
            const int jj = full * S + slot;
            const int cj = lane_get(c, jj & 63);  // lanes >= cnt hold column 0: a valid row, result unused
            const float aj = lane_get(av, jj & 63);
            VecT bv[V];
#pragma unroll
            for (int v = 0; v < V; ++v) bv[v] = row_load(cj, v);
            if (jj < cnt) {
#pragma unroll
                for (int v = 0; v < V; ++v) acc[v].fma(aj, bv[v]);
            }
        }
    }
}

// Adds the slots' partial sums so that every lane (in particular slot 0) ends with the total. G >= 8.
template <int VEC, int G, int V> __device__ __forceinline__ void slots_sum(Vec<VEC>* acc, int lane)
{
    (void)lane;
#pragma unroll
    for (int v = 0; v < V; ++v) {
        if constexpr (VEC == 4) {
            if constexpr (G <= 8) { acc[v].v.x = add_xor8(acc[v].v.x); acc[v].v.y = add_xor8(acc[v].v.y); acc[v].v.z = add_xor8(acc[v].v.z); acc[v].v.w = add_xor8(acc[v].v.w); }
            if constexpr (G <= 16) { acc[v].v.x = add_xor16(acc[v].v.x); acc[v].v.y = add_xor16(acc[v].v.y); acc[v].v.z = add_xor16(acc[v].v.z); acc[v].v.w = add_xor16(acc[v].v.w); }
            if constexpr (G <= 32) { acc[v].v.x = add_xor32(acc[v].v.x); acc[v].v.y = add_xor32(acc[v].v.y); acc[v].v.z = add_xor32(acc[v].v.z); acc[v].v.w = add_xor32(acc[v].v.w); }
        } else {
            if constexpr (G <= 8) acc[v].v = add_xor8(acc[v].v);
            if constexpr (G <= 16) acc[v].v = add_xor16(acc[v].v);
            if constexpr (G <= 32) acc[v].v = add_xor32(acc[v].v);
        }
    }
}

// ---- sampled dot products (SDDMM kernel and stage 1 of the fused kernel) -------------------------------
// One round: the lane group handling nonzero `n` of the chunk (column index fetched from lane n) reads
// that rhs row against the lhs row and returns the group's dot product in all of its lanes.
// MASKED: D is not G1*VEC*DS; lanes past D read a safe in-row address and contribute 0, the lane that straddles D
// reads the row's last VEC floats with the overlap zeroed. All DS loads are issued first and the zeroing follows as
// selects (where and how many elements: the same in every round, so the compiler keeps it outside the loop): zeroing
// under a condition right behind each load made every load wait for the one before (D = 192 took 1.7 times the time
// of D = 256). An access that lies past D for the whole wave is issued all the same (it reads the row's first floats
// again): leaving it out under a branch cost 5-45 % at D = 132 ... 320, the wait for all loads then comes before the
// first product.
// MASKED == kMaskedByRange (D a multiple of four, rhs of at most 1 GiB and fewer than 2^24 rows: the host checks): rhs is
// read as a raw buffer of 1 GiB, and a lane whose floats lie past D adds 3 GiB to its offset -- out of the buffer's
// range, for which the load returns zeros without touching memory. No select, no second address, and 0 * 0 where the
// other kind must keep 0 * (whatever it re-read) out of the sum.
constexpr int kExactWidth = 0, kMaskedBySelect = 1, kMaskedByRange = 2;
constexpr unsigned kRangeWindowBytes = 1u << 30, kRangeOutside = 3u << 30;
template <int VEC, int G1, int DS, int MASKED>
__device__ __forceinline__ void sddmm_rounds_load(int D, int g, const float* __restrict__ rhs, int cn, Vec<VEC>* x)
{
    const float* rrow = rhs + (size_t)cn * D;
    if constexpr (MASKED == kMaskedByRange) {
        const __amdgpu_buffer_rsrc_t window = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(rhs), 0, (int)kRangeWindowBytes, 0x00020000);
        const unsigned row = __umul24((unsigned)cn, (unsigned)D * (unsigned)sizeof(float));
#pragma unroll
        for (int s = 0; s < DS; ++s) {
            const int d = (s * G1 + g) * VEC;
            x[s] = Vec<VEC>::bload(window, row + (d < D ? (unsigned)d * (unsigned)sizeof(float) : kRangeOutside), 0u);
        }
    } else if constexpr (MASKED) {
        int gone[DS];  // leading elements of the access that are not the lane's to add
#pragma unroll
        for (int s = 0; s < DS; ++s) {
            const int d = (s * G1 + g) * VEC;
            const int from = d < D ? min(d, D - VEC) : 0;
            gone[s] = d < D ? d - from : VEC;  // (not 0 * whatever sits at column 0: that could be 0 * inf)
            x[s] = Vec<VEC>::gload(rrow + from);
        }
#pragma unroll
        for (int s = 0; s < DS; ++s) x[s].zero_first(gone[s]);
    } else {
#pragma unroll
        for (int s = 0; s < DS; ++s) x[s] = Vec<VEC>::gload(rrow + (s * G1 + g) * VEC);
    }
}

// One chunk of `cnt` <= 64 nonzeros of one row: returns in lane l the dot product of the chunk's nonzero l
// (lanes past the chunk return an unspecified value that the caller must not store). `c` is the lane's
// column index (0 past the chunk). `lq` holds the lhs row as laid out by the caller:
// lq[s] = lhs_row[(s*G1 + g)*VEC ..] (Vec::gload_clip), zero past D. With DS = 0 the row is re-read from lhs_row.
template <int VEC, int G1, int DS, int MASKED>
__device__ __forceinline__ float sddmm_chunk(int D, int lane, int cnt, int c, const float* __restrict__ lhs_row,
                                             const Vec<VEC>* lq, const float* __restrict__ rhs)
{
    using VecT = Vec<VEC>;
    constexpr int P = kWave / G1;  // nonzeros in flight per access
    const int g = lane % G1;
    const int grp = lane / G1;
    const int rounds = (cnt + P - 1) / P;  // <= G1
    float res = 0.f;
    if constexpr (DS > 0) {
        constexpr int U = DS >= 8 ? 1 : 8 / DS;  // rounds whose loads are issued together
        int t = 0;
        for (; t + U <= rounds; t += U) {
            VecT x[U][DS];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int cn = lane_get(c, ((t + u) * P + grp) & 63);
                sddmm_rounds_load<VEC, G1, DS, MASKED>(D, g, rhs, cn, x[u]);
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                float dot = 0.f;
#pragma unroll
                for (int s = 0; s < DS; ++s) dot = lq[s].dot(x[u][s], dot);
                dot = group_sum<G1>(dot);
                if (g == t + u) res = dot;  // lane grp*G1 + t keeps the result of nonzero t*P + grp
            }
        }
        if constexpr (U > 1) {
            if (t < rounds) {  // fewer than U rounds left: same batching under wave-uniform guards
                const int rem = rounds - t;
                VecT x[U - 1][DS];
#pragma unroll
                for (int u = 0; u < U - 1; ++u) {
                    if (u < rem) {
                        const int cn = lane_get(c, ((t + u) * P + grp) & 63);
                        sddmm_rounds_load<VEC, G1, DS, MASKED>(D, g, rhs, cn, x[u]);
                    }
                }
#pragma unroll
                for (int u = 0; u < U - 1; ++u) {
                    if (u < rem) {
                        float dot = 0.f;
#pragma unroll
                        for (int s = 0; s < DS; ++s) dot = lq[s].dot(x[u][s], dot);
                        dot = group_sum<G1>(dot);
                        if (g == t + u) res = dot;
                    }
                }
            }
        }
    } else {
        for (int t = 0; t < rounds; ++t) {
            const int cn = lane_get(c, (t * P + grp) & 63);
            const float* rrow = rhs + (size_t)cn * D;
            float dot = 0.f;
            for (int d = g * VEC; d < D; d += G1 * VEC)
                dot = VecT::gload_clip(lhs_row, d, D).dot(VecT::gload_clip(rrow, d, D), dot);
            dot = group_sum<G1>(dot);
            if (g == t) res = dot;
        }
    }
    // transpose: lane l wants nonzero l, which sits in lane (l % P) * G1 + l / P
    return lane_get(res, (lane % P) * G1 + lane / P);
}

}  // namespace dlspm
