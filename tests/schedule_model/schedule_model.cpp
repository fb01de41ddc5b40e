// Host model of the GPU schedule: the same work split (workgroups of W waves owning R rows, nonzeros divided
// evenly over the waves, lane groups taking every S-th nonzero, partial sums added in wave order) and the same
// fp32 operation sequence per output element as the HIP kernels in dlspm-esimd_amd/csrc, in scalar C++.
// TEST INFRASTRUCTURE: it lets the work decomposition be checked without a GPU (every output written exactly
// once, nothing read out of range) and lets the GPU results be compared BIT FOR BIT instead of within a
// tolerance. It plays the role the reference's SpmmEsimdCPU / FusedEsimdCPU (SPMM/spmm-esimd-v1.cpp:83-169,
// FUSED/fused.cpp:93-216) play for its kernels. The library never uses it.
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <vector>

namespace {

int split_per_wave(int T, int W)
{
    int per = (T + W - 1) / W;
    return per < 1 ? 1 : per;
}

// the row-aligned split of the kernels (common.hpp: split_is_row_aligned, wave_range), with W and R at run time
bool split_is_row_aligned(const int* off, int nr, int per, int W, int R)
{
    if (R == 1) return false;
    const int cap = per + (per >> 2);
    int worst = 0;
    if (R % W == 0) {
        const int k = R / W;
        for (int x = 0; x < W; ++x) worst = std::max(worst, off[std::min((x + 1) * k, nr)] - off[std::min(x * k, nr)]);
    } else {
        const int m = W / R;
        for (int r = 0; r < nr; ++r) worst = std::max(worst, (off[r + 1] - off[r] + m - 1) / m);
    }
    return worst <= cap;
}

void wave_range(bool aligned, const int* off, int nr, int w, int T0, int T, int per, int W, int R, int& a, int& b)
{
    if (!aligned) {
        a = T0 + std::min(T, w * per);
        b = T0 + std::min(T, (w + 1) * per);
    } else if (R % W == 0) {
        const int k = R / W;
        a = off[std::min(w * k, nr)];
        b = off[std::min((w + 1) * k, nr)];
    } else {
        const int m = W / R, r = w / m, j = w % m;
        if (r >= nr) { a = b = T0 + T; return; }
        const int rs = off[r], len = off[r + 1] - rs, piece = (len + m - 1) / m;
        a = rs + std::min(len, j * piece);
        b = rs + std::min(len, (j + 1) * piece);
    }
}

// sum of the S lane groups' accumulators in the order the kernel's cross-lane steps add them:
// neighbours first (xor G), then pairs of pairs (xor 2G), ... : a balanced tree over the slots
float slots_tree(const float* s, int S)
{
    if (S == 1) return s[0];
    std::vector<float> v(s, s + S);
    for (int step = 1; step < S; step <<= 1)
        for (int i = 0; i + step < S; i += 2 * step) v[i] = v[i] + v[i + step];
    return v[0];
}

// C[M x N] (+= semantics: every element written exactly once; `writes` counts them) for "values" per nonzero.
// Mirrors spmm_kernel / stage 2 of fused_kernel: shape = lanes G per dense row (S = 64/G slots), W waves, R rows.
int model_rows(int M, int N, const int* ro, const int* ci, const float* va, const float* B, int G, int W, int R,
               float* C, int* writes)
{
    const int S = 64 / G;
    std::vector<float> acc((size_t)S * N), part;
    for (int r0 = 0; r0 < M; r0 += R) {
        const int nr = std::min(R, M - r0);
        const int* off = ro + r0;
        const int T0 = off[0], T = off[nr] - T0;
        const int per = split_per_wave(T, W);
        const bool aligned = split_is_row_aligned(off, nr, per, W, R);
        part.assign((size_t)W * 2 * N, NAN);
        for (int w = 0; w < W; ++w) {
            int a, b;
            wave_range(aligned, off, nr, w, T0, T, per, W, R, a, b);
            if (a >= b) continue;
            int r = 0;
            while (off[r + 1] <= a) ++r;
            int pos = a;
            while (pos < b) {
                const int rs = off[r], re = off[r + 1];
                const int p = pos, q = std::min(re, b);
                std::fill(acc.begin(), acc.end(), 0.0f);
                for (int idx = p; idx < q; ++idx) {
                    const int slot = (idx - p) % S;  // 64 % S == 0, so the chunking does not change the slot
                    const float* brow = B + (size_t)ci[idx] * N;
                    float* as = acc.data() + (size_t)slot * N;
                    for (int j = 0; j < N; ++j) as[j] = std::fmaf(va[idx], brow[j], as[j]);
                }
                std::vector<float> sl(S);
                const bool whole = (p == rs) && (q == re);
                for (int j = 0; j < N; ++j) {
                    for (int s = 0; s < S; ++s) sl[s] = acc[(size_t)s * N + j];
                    const float tot = slots_tree(sl.data(), S);
                    if (whole) {
                        C[(size_t)(r0 + r) * N + j] = tot;
                        writes[(size_t)(r0 + r) * N + j]++;
                    } else {
                        part[((size_t)w * 2 + (p == a || R == 1 ? 0 : 1)) * N + j] = tot;
                    }
                }
                pos = q;
                ++r;
                while (r < nr && off[r + 1] <= pos) ++r;
            }
        }
        for (int r = 0; r < nr; ++r) {
            const int rs = off[r], re = off[r + 1];
            float* crow = C + (size_t)(r0 + r) * N;
            int* wrow = writes + (size_t)(r0 + r) * N;
            if (rs == re) {
                for (int j = 0; j < N; ++j) { crow[j] = 0.0f; wrow[j]++; }
                continue;
            }
            if (aligned && R % W == 0) continue;  // every wave stored its rows whole
            if (aligned) {                        // the m = W/R waves of the row hold its parts in order
                const int m = W / R, len = re - rs, piece = (len + m - 1) / m;
                if (len <= piece) continue;
                for (int j = 0; j < N; ++j) {
                    float sum = 0.0f;
                    for (int x = 0; x < m; ++x) {
                        if (x * piece >= len) continue;
                        const float pv = part[((size_t)(r * m + x) * 2) * N + j];
                        if (std::isnan(pv) && !std::isnan(B[0])) return 1;
                        sum = sum + pv;
                    }
                    crow[j] = sum;
                    wrow[j]++;
                }
                continue;
            }
            const int wl = (rs - T0) / per, wh = (re - 1 - T0) / per;
            if (wl == wh) continue;
            for (int j = 0; j < N; ++j) {
                float sum = 0.0f;
                for (int x = wl; x <= wh; ++x) {
                    const int k = (R != 1 && x == wl && T0 + x * per != rs) ? 1 : 0;
                    const float pv = part[((size_t)x * 2 + k) * N + j];
                    if (std::isnan(pv) && !std::isnan(B[0])) return 1;  // a partial sum the schedule never produced
                    sum = sum + pv;
                }
                crow[j] = sum;
                wrow[j]++;
            }
        }
    }
    return 0;
}

// dot product of one nonzero as the SDDMM lane group computes it: lane g accumulates its elements in order with
// fused multiply-adds, then the G1 lanes are added pairwise (lane^1, lane^2, then the mirrored halves). Positions
// past D contribute fma(0, 0, acc) = acc, wherever the kernel places them in a lane's sequence.
float model_dot(const float* l, const float* r, int D, int vec, int G1, int DS)
{
    std::vector<float> lane(G1, 0.0f);
    for (int g = 0; g < G1; ++g) {
        float acc = 0.0f;
        if (DS > 0) {
            for (int s = 0; s < DS; ++s) {
                const int d = (s * G1 + g) * vec;
                for (int e = 0; e < vec; ++e)
                    if (d + e < D) acc = std::fmaf(l[d + e], r[d + e], acc);
                    else acc = std::fmaf(0.0f, 0.0f, acc);
            }
        } else {
            for (int d = g * vec; d < D; d += G1 * vec)
                for (int e = 0; e < vec; ++e)
                    if (d + e < D) acc = std::fmaf(l[d + e], r[d + e], acc);
        }
        lane[g] = acc;
    }
    for (int step = 1; step < G1; step <<= 1)
        for (int i = 0; i + step < G1; i += 2 * step) lane[i] = lane[i] + lane[i + step];
    return lane[0];
}


// ---- flat schedule (spmm_flat_kernel / fused_flat_kernel + row_fixup_kernel) ------------------------------------
// The row search and the 64-entry offset window are modelled lane by lane, with every index checked, so that an
// indexing mistake in them shows on the CPU: any out-of-range access makes the model return 2.
struct Checked {
    const int* ro;
    int M;
    bool bad = false;
    int at(long long i)
    {
        if (i < 0 || i > M) { bad = true; return 0; }
        return ro[i];
    }
};

int model_find_row(Checked& c, int pos)
{
    int lo = 0, hi = c.M;
    while (hi - lo > 1) {
        const long long span = hi - lo;
        int n = 0;
        bool prefix = true;
        for (int lane = 0; lane < 64; ++lane) {
            const int idx = lo + (int)((span * (lane + 1)) >> 6);
            const bool le = c.at(idx) <= pos;
            if (le && !prefix) c.bad = true;  // the kernel counts on a prefix of lanes
            if (le) ++n; else prefix = false;
        }
        if (n >= 64) { c.bad = true; return lo; }
        const int new_lo = lo + (int)((span * n) >> 6);
        const int new_hi = lo + (int)((span * (n + 1)) >> 6);
        if (new_hi - new_lo >= hi - lo) { c.bad = true; return lo; }  // no progress
        lo = new_lo;
        hi = new_hi;
    }
    return lo;
}

void model_window_load(Checked& c, int rbase, int* win)
{
    for (int lane = 0; lane < 64; ++lane) win[lane] = c.at(std::min(rbase + lane, c.M));
}

int model_rows_flat(int M, int N, int nnz, const int* ro, const int* ci, const float* va, const float* B, int G, int chunk,
                    float* C, int* writes)
{
    const int S = 64 / G;
    const int units = (int)(((long long)nnz + chunk - 1) / chunk);
    std::vector<float> part((size_t)units * 2 * N, NAN), acc((size_t)S * N), sl(S);
    Checked c{ro, M};
    for (int unit = 0; unit < units; ++unit) {
        const int a = unit * chunk, b = std::min(nnz, a + chunk);
        int r = model_find_row(c, a);
        int rbase = r, win[64];
        model_window_load(c, rbase, win);
        int pos = a;
        while (true) {
            if (r - rbase >= 63) { rbase = r; model_window_load(c, rbase, win); }
            if (r - rbase < 0 || r - rbase + 1 > 63) return 2;
            const int rs = win[r - rbase], re = win[r - rbase + 1];
            if (r < 0 || r >= M || rs != ro[r] || re != ro[r + 1] || !(rs <= pos && pos < re)) return 2;
            const int p = pos, q = std::min(re, b);
            std::fill(acc.begin(), acc.end(), 0.0f);
            for (int idx = p; idx < q; ++idx) {
                const float* brow = B + (size_t)ci[idx] * N;
                float* as = acc.data() + (size_t)((idx - p) % S) * N;
                for (int j = 0; j < N; ++j) as[j] = std::fmaf(va[idx], brow[j], as[j]);
            }
            const bool whole = p == rs && q == re;
            for (int j = 0; j < N; ++j) {
                for (int s = 0; s < S; ++s) sl[s] = acc[(size_t)s * N + j];
                const float tot = slots_tree(sl.data(), S);
                if (whole) { C[(size_t)r * N + j] = tot; writes[(size_t)r * N + j]++; }
                else part[((size_t)unit * 2 + (p == a ? 0 : 1)) * N + j] = tot;
            }
            pos = q;
            if (pos >= b) break;
            int t = -1;
            for (int lane = 0; lane < 64; ++lane)
                if (win[lane] > pos) { t = lane; break; }
            if (t >= 0) {
                if (t < 1) return 2;
                r = rbase + t - 1;
            } else {
                r = model_find_row(c, pos);
                rbase = r;
                model_window_load(c, rbase, win);
            }
        }
    }
    if (c.bad) return 2;
    for (int r = 0; r < M; ++r) {
        const int rs = ro[r], re = ro[r + 1];
        float* crow = C + (size_t)r * N;
        int* wrow = writes + (size_t)r * N;
        if (rs == re) {
            for (int j = 0; j < N; ++j) { crow[j] = 0.0f; wrow[j]++; }
            continue;
        }
        const int ul = rs / chunk, uh = (re - 1) / chunk;
        if (ul == uh) continue;
        for (int j = 0; j < N; ++j) {
            float sum = 0.0f;
            for (int u = ul; u <= uh; ++u) {
                const int k = (u == ul && (long long)u * chunk != rs) ? 1 : 0;
                const float pv = part[((size_t)u * 2 + k) * N + j];
                if (std::isnan(pv) && !std::isnan(B[0])) return 1;
                sum = sum + pv;
            }
            crow[j] = sum;
            wrow[j]++;
        }
    }
    return 0;
}

}  // namespace

extern "C" {

// returns 0, or 1 if the schedule is inconsistent (a partial sum consumed that no wave produced)
int model_spmm(int M, int N, const int* ro, const int* ci, const float* va, const float* B, int G, int W, int R, float* C,
               int* writes)
{
    std::memset(writes, 0, (size_t)M * N * sizeof(int));
    return model_rows(M, N, ro, ci, va, B, G, W, R, C, writes);
}

// flat schedule: 0 ok, 1 a partial row consumed that no wave produced, 2 an index out of range in the row search or
// the offset window
int model_spmm_flat(int M, int N, const int* ro, const int* ci, const float* va, const float* B, int G, int chunk,
                    float* C, int* writes)
{
    std::memset(writes, 0, (size_t)M * N * sizeof(int));
    return model_rows_flat(M, N, ro[M], ro, ci, va, B, G, chunk, C, writes);
}

int model_fused_flat(int M, int D, const int* ro, const int* ci, const float* Q, const float* Km, const float* V,
                     float scale, int vec, int G1, int DS, int G, int chunk, float* scores, float* O, int* writes);

void model_sddmm(int M, int D, const int* ro, const int* ci, const float* lhs, const float* rhs, int vec, int G1, int DS,
                 float* out)
{
    for (int i = 0; i < M; ++i)
        for (int j = ro[i]; j < ro[i + 1]; ++j)
            out[j] = model_dot(lhs + (size_t)i * D, rhs + (size_t)ci[j] * D, D, vec, G1, DS);
}

int model_fused(int M, int D, const int* ro, const int* ci, const float* Q, const float* Km, const float* V, float scale,
                int vec, int G1, int DS, int G, int W, int R, float* scores, float* O, int* writes)
{
    model_sddmm(M, D, ro, ci, Q, Km, vec, G1, DS, scores);
    const int nnz = ro[M];
    for (int j = 0; j < nnz; ++j) scores[j] = scores[j] * scale;
    std::memset(writes, 0, (size_t)M * D * sizeof(int));
    return model_rows(M, D, ro, ci, scores, V, G, W, R, O, writes);
}

int model_fused_flat(int M, int D, const int* ro, const int* ci, const float* Q, const float* Km, const float* V,
                     float scale, int vec, int G1, int DS, int G, int chunk, float* scores, float* O, int* writes)
{
    model_sddmm(M, D, ro, ci, Q, Km, vec, G1, DS, scores);
    const int nnz = ro[M];
    for (int j = 0; j < nnz; ++j) scores[j] = scores[j] * scale;
    std::memset(writes, 0, (size_t)M * D * sizeof(int));
    return model_rows_flat(M, D, nnz, ro, ci, scores, V, G, chunk, O, writes);
}

// Host model of the row plan that dlspm_row_plan_build builds on the device: rows sorted longest first (by row number
// among equals); the first min(M, 8 x bins) of them packed into `bins` bins of equal size, longest row first into the
// least loaded bin OF ITS GROUP that still has room (ties: the lower bin), bin b becoming the positions b, b + bins,
// b + 2 bins, ...; the groups -- at most 64 bins each, sorted row t and bin b in group t % groups and b % groups --
// are packed independently of each other (one wave each on the device);
// rows without nonzeros fill the positions still free, in ascending order; the rest follow in sorted order.
// order 1: groups of `bins` alternate between descending and ascending length instead; order 2: plainly descending.
// plan[0 .. M) first nonzero, plan[M .. 2M) end, plan[2M .. 3M) row. This sequential statement is the definition; the
// device finds the same packing in parallel batches.
void model_row_plan(int M, const int* ro, int bins, int order, int* plan)
{
    std::vector<int> sorted((size_t)M);
    for (int i = 0; i < M; ++i) sorted[i] = i;
    auto len = [&](int i) { return ro[i + 1] - ro[i] > 0 ? ro[i + 1] - ro[i] : 0; };
    std::stable_sort(sorted.begin(), sorted.end(), [&](int a, int b) { return len(a) > len(b); });
    const int head = M < 8 * bins ? M : 8 * bins;
    std::vector<int> at((size_t)M);
    for (int i = 0; i < M; ++i) at[i] = sorted[i];
    if (order == 1) {
        for (int g = bins; g < head; g += 2 * bins) std::reverse(at.begin() + g, at.begin() + (g + bins < head ? g + bins : head));
    } else if (order == 0) {
        // groups: the smallest number g >= bins / 64 that divides bins; sorted row t and bin b belong to group t % g, b % g
        int groups = (bins + 63) / 64;
        while (bins % groups != 0) ++groups;
        std::vector<long long> load((size_t)bins, 0);
        std::vector<int> cnt((size_t)bins, 0), placed((size_t)head, -1);
        int t = 0;
        for (; t < head && len(sorted[t]) > 0; ++t) {
            int best = -1;
            for (int b = t % groups; b < bins; b += groups)
                if ((long long)cnt[b] * bins + b < head && (best < 0 || load[b] < load[best])) best = b;
            placed[(size_t)cnt[best] * bins + best] = sorted[t];
            load[best] += len(sorted[t]);
            ++cnt[best];
        }
        for (int p = 0; p < head; ++p)
            if (placed[p] < 0) placed[p] = sorted[t++];
        for (int p = 0; p < head; ++p) at[p] = placed[p];
    }
    for (int i = 0; i < M; ++i) {
        plan[i] = ro[at[i]];
        plan[(size_t)M + i] = ro[at[i] + 1];
        plan[2 * (size_t)M + i] = at[i];
    }
}

// Host model of the cut rule of a cut plan (plan_cut_kernel): with share = max(1, ceil(nnz / bins)), piece_max =
// ceil(share x piece_pct / 100) and longest = max(piece_max, ceil(share x longest_pct / 100)), a row of more than
// `longest` nonzeros becomes c pieces of ceil(length / c) nonzeros each (the last ones what is left, possibly nothing),
// c the smallest power of two >= ceil(length / piece_max), 256 at most; the rows and pieces in matrix order are the
// "virtual rows" 0 .. used-1 of `entries` = M + 2 x extra, extra = ceil(bins x 100 / piece_pct); the others hold nothing.
// v_off[entries + 1], v_row[entries] (-1: nothing), v_slot[entries] (-1 a whole row, s >= 0 piece number s among all
// pieces in matrix order, -2 nothing); cut[0] = cut rows, cut[1] = share, cut[2] = used, cut[3] = 0, then max_cut =
// ceil(bins x 100 / longest_pct) records of four ints (row, first slot, pieces, 1; records beyond cut[0] are zeros).
// Returns 0, or 1 if a bound that the plan's size relies on does not hold (more than entries virtual rows, 2 x extra +
// max_cut pieces or max_cut cut rows).
int model_cut_rows(int M, const int* ro, int bins, int piece_pct, int longest_pct, int* v_off, int* v_row, int* v_slot, int* cut)
{
    const int extra = (bins * 100 + piece_pct - 1) / piece_pct, max_cut = (bins * 100 + longest_pct - 1) / longest_pct;
    const int entries = M + 2 * extra, slots = 2 * extra + max_cut;
    long long nnz = 0;
    for (int i = 0; i < M; ++i) nnz += std::max(ro[i + 1] - ro[i], 0);
    const long long share = std::max((nnz + bins - 1) / bins, 1ll);
    const long long piece_max = std::max((share * piece_pct + 99) / 100, 1ll);
    const long long longest_whole = std::max((share * longest_pct + 99) / 100, piece_max);
    int e = 0, s = 0, j = 0;
    for (int i = 0; i < M; ++i) {
        const int len = std::max(ro[i + 1] - ro[i], 0);
        if (len <= longest_whole) {
            if (e >= entries) return 1;
            v_off[e] = ro[i]; v_row[e] = i; v_slot[e] = -1;
            ++e;
            continue;
        }
        const long long need = (len + piece_max - 1) / piece_max;
        int c = 2;
        while (c < need && c < 256) c *= 2;
        const int piece = (len + c - 1) / c;
        if (e + c > entries || s + c > slots || j >= max_cut) return 1;
        cut[4 + 4 * j] = i; cut[4 + 4 * j + 1] = s; cut[4 + 4 * j + 2] = c; cut[4 + 4 * j + 3] = 1;
        for (int k = 0; k < c; ++k) {
            v_off[e] = ro[i] + std::min(len, k * piece); v_row[e] = i; v_slot[e] = s;
            ++e; ++s;
        }
        ++j;
    }
    cut[0] = j; cut[1] = (int)share; cut[2] = e; cut[3] = 0;
    for (; j < max_cut; ++j) cut[4 + 4 * j] = cut[4 + 4 * j + 1] = cut[4 + 4 * j + 2] = cut[4 + 4 * j + 3] = 0;
    for (; e <= entries; ++e) {
        v_off[e] = ro[M];
        if (e < entries) { v_row[e] = -1; v_slot[e] = -2; }
    }
    return 0;
}

// The cut plan that dlspm_row_plan_build_cut builds: the row plan (model_row_plan) of the virtual rows, each entry then
// naming its matrix row and its slot. plan[4 x entries]: first nonzero, end, row, slot word. The slot word of piece k of
// a row cut into c = 1 << lg is slot | k << 15 | lg << 23, and such an entry holds the range of its WHOLE row (a launch
// takes the piece's share of the nonzeros, or of the columns, from the word); -1 for a whole row, -2 for an entry that
// holds nothing.
int model_row_plan_cut(int M, const int* ro, int bins, int piece_pct, int longest_pct, int order, int* plan, int* cut)
{
    const int entries = M + 2 * ((bins * 100 + piece_pct - 1) / piece_pct);
    std::vector<int> v_off((size_t)entries + 1), v_row((size_t)entries), v_slot((size_t)entries), vp((size_t)3 * entries);
    if (model_cut_rows(M, ro, bins, piece_pct, longest_pct, v_off.data(), v_row.data(), v_slot.data(), cut)) return 1;
    model_row_plan(entries, v_off.data(), bins, order, vp.data());
    for (int p = 0; p < entries; ++p) {
        const int v = vp[2 * (size_t)entries + p];
        plan[p] = vp[p];
        plan[(size_t)entries + p] = vp[(size_t)entries + p];
        plan[2 * (size_t)entries + p] = v_row[v];
        int word = v_slot[v];
        if (word >= 0) {
            int first = v, last = v;  // the virtual rows of one matrix row are neighbours
            while (first > 0 && v_row[first - 1] == v_row[v]) --first;
            while (last + 1 < entries && v_row[last + 1] == v_row[v]) ++last;
            int lg = 0;
            while ((1 << lg) < last - first + 1) ++lg;
            word = (word & 0x7fff) | (v - first) << 15 | lg << 23;
            plan[p] = v_off[first];
            plan[(size_t)entries + p] = v_off[last + 1];
        }
        plan[3 * (size_t)entries + p] = word;
    }
    return 0;
}

}  // extern "C"
