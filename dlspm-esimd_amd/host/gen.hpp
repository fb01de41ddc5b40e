// Seeded synthetic inputs for the sparse-kernel drivers, tests and benchmark.
//
// The reference fills its inputs with the C library's rand() left at its default seed
// (Bernoulli pattern: SPMM/spmm-esimd-allbenchs2.cpp:64-78; dense operands: :88-91), which is
// reproducible only against one libc. Here every stream comes from one explicit 64-bit seed through
// xoshiro256** (seeded by splitmix64), so the host drivers and the Python tests build bit-identical
// inputs everywhere. Column indices inside a row are unique and ascending, as in the DLMC files.
#pragma once

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <numeric>
#include <vector>

namespace dlspm {

class Rng {
public:
    explicit Rng(uint64_t seed)
    {
        for (auto& w : s_) {  // splitmix64 expansion of the seed
            seed += 0x9E3779B97F4A7C15ull;
            uint64_t z = seed;
            z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
            z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
            w = z ^ (z >> 31);
        }
    }
    uint64_t next()
    {
        const uint64_t r = rotl(s_[1] * 5, 7) * 9;
        const uint64_t t = s_[1] << 17;
        s_[2] ^= s_[0];
        s_[3] ^= s_[1];
        s_[1] ^= s_[2];
        s_[0] ^= s_[3];
        s_[2] ^= t;
        s_[3] = rotl(s_[3], 45);
        return r;
    }
    // uniform in [0, 1) with 53 random bits
    double uniform() { return static_cast<double>(next() >> 11) * (1.0 / 9007199254740992.0); }
    // uniform integer in [0, n)
    uint32_t below(uint32_t n) { return static_cast<uint32_t>((static_cast<unsigned __int128>(next()) * n) >> 64); }
    // standard normal (Box-Muller, one value per call)
    double normal()
    {
        if (have_spare_) {
            have_spare_ = false;
            return spare_;
        }
        double u1;
        do {
            u1 = uniform();
        } while (u1 <= 0.0);
        const double u2 = uniform();
        const double r = std::sqrt(-2.0 * std::log(u1));
        const double a = 6.283185307179586476925286766559 * u2;
        spare_ = r * std::sin(a);
        have_spare_ = true;
        return r * std::cos(a);
    }

private:
    static uint64_t rotl(uint64_t x, int k) { return (x << k) | (x >> (64 - k)); }
    uint64_t s_[4];
    bool have_spare_ = false;
    double spare_ = 0.0;
};

struct Csr {
    int M = 0, K = 0;
    std::vector<int> row_offsets;  // M + 1
    std::vector<int> col_indices;  // nnz, ascending and unique inside each row
    int nnz() const { return row_offsets.empty() ? 0 : row_offsets.back(); }
};

// k distinct columns out of [0, K), ascending, appended to `out`. `scratch` must hold 0..K-1 in any order.
inline void sample_row(Rng& rng, int K, int k, std::vector<int>& scratch, std::vector<int>& out)
{
    k = std::max(0, std::min(k, K));
    for (int t = 0; t < k; ++t) {  // partial Fisher-Yates
        const int j = t + static_cast<int>(rng.below(static_cast<uint32_t>(K - t)));
        std::swap(scratch[t], scratch[j]);
    }
    const size_t at = out.size();
    out.insert(out.end(), scratch.begin(), scratch.begin() + k);
    std::sort(out.begin() + at, out.end());
}

// Row i holds floor((i+1)*density*K) - floor(i*density*K) entries (so the total is floor(M*density*K)),
// at uniform-random distinct columns.
inline Csr pattern_uniform_rows(uint64_t seed, int M, int K, double density)
{
    Rng rng(seed);
    Csr a;
    a.M = M;
    a.K = K;
    a.row_offsets.assign(M + 1, 0);
    std::vector<int> scratch(K);
    std::iota(scratch.begin(), scratch.end(), 0);
    const double per_row = density * K;
    for (int i = 0; i < M; ++i) {
        const int k = static_cast<int>(std::floor((i + 1) * per_row)) - static_cast<int>(std::floor(i * per_row));
        sample_row(rng, K, k, scratch, a.col_indices);
        a.row_offsets[i + 1] = static_cast<int>(a.col_indices.size());
    }
    return a;
}

// Row lengths clamp(round(LogNormal(ln(mean) - sigma^2/2, sigma)), 0, K): mean `mean`, skewed.
inline Csr pattern_lognormal_rows(uint64_t seed, int M, int K, double mean, double sigma)
{
    Rng rng(seed);
    Csr a;
    a.M = M;
    a.K = K;
    a.row_offsets.assign(M + 1, 0);
    std::vector<int> scratch(K);
    std::iota(scratch.begin(), scratch.end(), 0);
    const double mu = std::log(mean) - 0.5 * sigma * sigma;
    for (int i = 0; i < M; ++i) {
        const double len = std::exp(mu + sigma * rng.normal());
        const int k = static_cast<int>(std::min<double>(K, std::max(0.0, std::floor(len + 0.5))));
        sample_row(rng, K, k, scratch, a.col_indices);
        a.row_offsets[i + 1] = static_cast<int>(a.col_indices.size());
    }
    return a;
}

// Every (i, j) kept independently with probability `density` -- the reference's own pattern
// (SPMM/spmm-esimd-allbenchs2.cpp:64-78), with this file's generator in place of rand().
inline Csr pattern_bernoulli(uint64_t seed, int M, int K, double density)
{
    Rng rng(seed);
    Csr a;
    a.M = M;
    a.K = K;
    a.row_offsets.assign(M + 1, 0);
    a.col_indices.reserve(static_cast<size_t>(1.01 * M * K * density) + 100);
    for (int i = 0; i < M; ++i) {
        for (int j = 0; j < K; ++j)
            if (rng.uniform() < density) a.col_indices.push_back(j);
        a.row_offsets[i + 1] = static_cast<int>(a.col_indices.size());
    }
    return a;
}

// Sparse-attention mask: row i keeps the band [i - band/2, i + band/2) clipped to [0, K) plus
// `n_random` uniform-random columns; duplicates collapse, so a row has at most band + n_random entries.
inline Csr pattern_band_plus_random(uint64_t seed, int M, int K, int band, int n_random)
{
    Rng rng(seed);
    Csr a;
    a.M = M;
    a.K = K;
    a.row_offsets.assign(M + 1, 0);
    std::vector<int> row;
    for (int i = 0; i < M; ++i) {
        row.clear();
        for (int j = std::max(0, i - band / 2); j < std::min(K, i + band / 2); ++j) row.push_back(j);
        for (int t = 0; t < n_random; ++t) row.push_back(static_cast<int>(rng.below(static_cast<uint32_t>(K))));
        std::sort(row.begin(), row.end());
        row.erase(std::unique(row.begin(), row.end()), row.end());
        a.col_indices.insert(a.col_indices.end(), row.begin(), row.end());
        a.row_offsets[i + 1] = static_cast<int>(a.col_indices.size());
    }
    return a;
}

// Magnitude pruning per row: draw a dense M x K matrix N(0, stddev), keep each row's `keep` largest
// |w| (ties broken by lower column). Returns the pattern and writes the kept weights to `values`.
inline Csr pattern_topk_rows(uint64_t seed, int M, int K, int keep, double stddev, std::vector<float>& values)
{
    Rng rng(seed);
    Csr a;
    a.M = M;
    a.K = K;
    a.row_offsets.assign(M + 1, 0);
    keep = std::max(0, std::min(keep, K));
    std::vector<float> w(K);
    std::vector<int> order(K);
    values.clear();
    for (int i = 0; i < M; ++i) {
        for (int j = 0; j < K; ++j) w[j] = static_cast<float>(stddev * rng.normal());
        std::iota(order.begin(), order.end(), 0);
        std::partial_sort(order.begin(), order.begin() + keep, order.end(), [&](int x, int y) {
            const float ax = std::fabs(w[x]), ay = std::fabs(w[y]);
            return ax > ay || (ax == ay && x < y);
        });
        std::sort(order.begin(), order.begin() + keep);
        for (int t = 0; t < keep; ++t) {
            a.col_indices.push_back(order[t]);
            values.push_back(w[order[t]]);
        }
        a.row_offsets[i + 1] = static_cast<int>(a.col_indices.size());
    }
    return a;
}

inline void fill_uniform(uint64_t seed, size_t n, float lo, float hi, float* out)
{
    Rng rng(seed);
    for (size_t i = 0; i < n; ++i) out[i] = static_cast<float>(lo + (hi - lo) * rng.uniform());
}

inline void fill_normal(uint64_t seed, size_t n, float mean, float stddev, float* out)
{
    Rng rng(seed);
    for (size_t i = 0; i < n; ++i) out[i] = static_cast<float>(mean + stddev * rng.normal());
}

// Post-ReLU-like activations: zero with probability p_zero, otherwise U[0, 1).
inline void fill_relu_like(uint64_t seed, size_t n, double p_zero, float* out)
{
    Rng rng(seed);
    for (size_t i = 0; i < n; ++i) {
        const double keep = rng.uniform();
        const double v = rng.uniform();
        out[i] = keep < p_zero ? 0.0f : static_cast<float>(v);
    }
}

// ---------------------------------------------------------------------------------------------
// The five benchmark configurations (one problem = CSR structure + values + up to three dense operands)
// ---------------------------------------------------------------------------------------------

enum Op { kSpmm = 0, kSddmm = 1, kFused = 2 };

struct Problem {
    int cfg = 0;
    Op op = kSpmm;
    const char* name = "";
    int M = 0, K = 0, N = 0;  // N = dense width (SpMM) or inner dimension D (SDDMM / fused)
    float scale = 1.0f;       // fused only
    Csr a;
    std::vector<float> values;  // SpMM: nnz values of A
    std::vector<float> d0;      // SpMM: B (K x N) | SDDMM: lhs (M x D) | fused: Q (M x D)
    std::vector<float> d1;      // SDDMM: rhs (K x D) | fused: Kmat (K x D)
    std::vector<float> d2;      // fused: V (K x D)
};

inline const char* config_name(int cfg)
{
    switch (cfg) {
        case 1: return "cfg1_spmm_512x512x128_s70_uniform";
        case 2: return "cfg2_spmm_2048x512x256_s90_lognormal";
        case 3: return "cfg3_sddmm_2048x2048_d128_s95";
        case 4: return "cfg4_spmm_2048x512x392_s80_topk_relu";
        case 5: return "cfg5_fused_4096x4096_d64_band32_rand48";
        default: return "unknown";
    }
}

// Builds configuration `cfg` (1..5) from its fixed seed 1000 + cfg. Returns false for an unknown id.
inline bool make_config(int cfg, Problem& p)
{
    const uint64_t seed = 1000 + static_cast<uint64_t>(cfg);
    p = Problem();
    p.cfg = cfg;
    p.name = config_name(cfg);
    switch (cfg) {
        case 1: {  // A 512x512, 70 % sparse, uniform positions, U[-1,1]; B 512x128 U[-1,1]
            p.op = kSpmm; p.M = 512; p.K = 512; p.N = 128;
            p.a = pattern_uniform_rows(seed, p.M, p.K, 0.30);
            p.values.resize(p.a.nnz());
            fill_uniform(seed ^ 0xA1, p.values.size(), -1.f, 1.f, p.values.data());
            p.d0.resize(static_cast<size_t>(p.K) * p.N);
            fill_uniform(seed ^ 0xB2, p.d0.size(), -1.f, 1.f, p.d0.data());
            return true;
        }
        case 2: {  // A 2048x512, 90 % sparse, lognormal(sigma 0.6) row lengths, N(0, 0.02); B 512x256 U[-1,1]
            p.op = kSpmm; p.M = 2048; p.K = 512; p.N = 256;
            p.a = pattern_lognormal_rows(seed, p.M, p.K, 0.10 * p.K, 0.6);
            p.values.resize(p.a.nnz());
            fill_normal(seed ^ 0xA1, p.values.size(), 0.f, 0.02f, p.values.data());
            p.d0.resize(static_cast<size_t>(p.K) * p.N);
            fill_uniform(seed ^ 0xB2, p.d0.size(), -1.f, 1.f, p.d0.data());
            return true;
        }
        case 3: {  // mask 2048x2048, 95 % sparse, uniform positions; lhs, rhs 2048x128 N(0,1)
            p.op = kSddmm; p.M = 2048; p.K = 2048; p.N = 128;
            p.a = pattern_uniform_rows(seed, p.M, p.K, 0.05);
            p.d0.resize(static_cast<size_t>(p.M) * p.N);
            fill_normal(seed ^ 0xB2, p.d0.size(), 0.f, 1.f, p.d0.data());
            p.d1.resize(static_cast<size_t>(p.K) * p.N);
            fill_normal(seed ^ 0xC3, p.d1.size(), 0.f, 1.f, p.d1.data());
            return true;
        }
        case 4: {  // W 2048x512 N(0, 0.05) keeping each row's top-102 |w|; X 512x392 half zero, half U[0,1)
            p.op = kSpmm; p.M = 2048; p.K = 512; p.N = 392;
            p.a = pattern_topk_rows(seed, p.M, p.K, static_cast<int>(0.20 * p.K), 0.05, p.values);
            p.d0.resize(static_cast<size_t>(p.K) * p.N);
            fill_relu_like(seed ^ 0xB2, p.d0.size(), 0.5, p.d0.data());
            return true;
        }
        case 5: {  // mask 4096x4096: band 32 + 48 random columns; Q, K, V 4096x64 N(0,1); scale 1/8
            p.op = kFused; p.M = 4096; p.K = 4096; p.N = 64; p.scale = 0.125f;
            p.a = pattern_band_plus_random(seed, p.M, p.K, 32, 48);
            p.d0.resize(static_cast<size_t>(p.M) * p.N);
            fill_normal(seed ^ 0xB2, p.d0.size(), 0.f, 1.f, p.d0.data());
            p.d1.resize(static_cast<size_t>(p.K) * p.N);
            fill_normal(seed ^ 0xC3, p.d1.size(), 0.f, 1.f, p.d1.data());
            p.d2.resize(static_cast<size_t>(p.K) * p.N);
            fill_normal(seed ^ 0xD4, p.d2.size(), 0.f, 1.f, p.d2.data());
            return true;
        }
        default: return false;
    }
}

// ---------------------------------------------------------------------------------------------
// Byte / flop accounting used in every report
// ---------------------------------------------------------------------------------------------

struct Accounting {
    double flops;            // the reference's flop formula
    double algorithmic_B;    // every input read once + every output written once
    double effective_B;      // the reference's "application bandwidth": every gathered dense row counted
};

inline Accounting account(Op op, double M, double K, double N, double nnz)
{
    Accounting a{};
    switch (op) {
        case kSpmm:  // flops: SPMM/spmm-esimd-fromfile2.cpp:253
            a.flops = (2.0 * nnz - M) * N;
            a.algorithmic_B = 4.0 * (M + 1) + 8.0 * nnz + 4.0 * K * N + 4.0 * M * N;
            a.effective_B = 4.0 * (M + 1) + 8.0 * nnz + 4.0 * nnz * N + 4.0 * M * N;
            break;
        case kSddmm:  // flops: SDDMM/sddmm-esimd-fromfile.cpp:160; bytes convention: SDDMM/sddmm-esimd-v1.cpp:190
            a.flops = nnz * (2.0 * N - 1.0);
            a.algorithmic_B = 4.0 * (M + 1) + 4.0 * nnz + 4.0 * M * N + 4.0 * K * N + 4.0 * nnz;
            a.effective_B = 4.0 * (M + 1) + 4.0 * nnz + 4.0 * M * N + 4.0 * nnz * N + 4.0 * nnz;
            break;
        case kFused:  // flops: FUSED/fused-esimd_cb.cpp:346-348, plus one multiply per score for the scale
            a.flops = (2.0 * nnz - M) * N + nnz * (2.0 * N - 1.0) + nnz;
            a.algorithmic_B = 4.0 * (M + 1) + 4.0 * nnz + 4.0 * M * N + 8.0 * K * N + 4.0 * M * N;
            a.effective_B = 4.0 * (M + 1) + 4.0 * nnz + 4.0 * M * N + 8.0 * nnz * N + 4.0 * M * N;
            break;
    }
    return a;
}

}  // namespace dlspm
