// C ABI over gen.hpp (libdlspm_gen.so) so that the Python tests and the benchmark build exactly the
// inputs the C++ drivers build. Host code only; nothing here touches the GPU.
#include "gen.hpp"

#include <cstring>

using namespace dlspm;

extern "C" {

// ---- whole benchmark configurations -----------------------------------------------------------
void* dlspm_gen_config_create(int cfg)
{
    auto* p = new Problem();
    if (!make_config(cfg, *p)) {
        delete p;
        return nullptr;
    }
    return p;
}
void dlspm_gen_config_destroy(void* h) { delete static_cast<Problem*>(h); }

// op, M, K, N, nnz into dims[5]; scale separately
void dlspm_gen_config_dims(const void* h, int* dims, float* scale)
{
    const auto* p = static_cast<const Problem*>(h);
    dims[0] = p->op; dims[1] = p->M; dims[2] = p->K; dims[3] = p->N; dims[4] = p->a.nnz();
    *scale = p->scale;
}
const char* dlspm_gen_config_name(int cfg) { return config_name(cfg); }
const int* dlspm_gen_config_row_offsets(const void* h) { return static_cast<const Problem*>(h)->a.row_offsets.data(); }
const int* dlspm_gen_config_col_indices(const void* h) { return static_cast<const Problem*>(h)->a.col_indices.data(); }
const float* dlspm_gen_config_values(const void* h) { return static_cast<const Problem*>(h)->values.data(); }
// which = 0, 1, 2 -> d0, d1, d2; *count receives the element count
const float* dlspm_gen_config_dense(const void* h, int which, size_t* count)
{
    const auto* p = static_cast<const Problem*>(h);
    const std::vector<float>& v = which == 0 ? p->d0 : which == 1 ? p->d1 : p->d2;
    *count = v.size();
    return v.data();
}

// ---- single patterns ---------------------------------------------------------------------------
// kind: 0 uniform rows (p0 = density) | 1 lognormal rows (p0 = mean, p1 = sigma) | 2 Bernoulli (p0 = density)
//       3 band + random (p0 = band, p1 = n_random)
void* dlspm_gen_pattern_create(int kind, uint64_t seed, int M, int K, double p0, double p1)
{
    auto* a = new Csr();
    switch (kind) {
        case 0: *a = pattern_uniform_rows(seed, M, K, p0); break;
        case 1: *a = pattern_lognormal_rows(seed, M, K, p0, p1); break;
        case 2: *a = pattern_bernoulli(seed, M, K, p0); break;
        case 3: *a = pattern_band_plus_random(seed, M, K, static_cast<int>(p0), static_cast<int>(p1)); break;
        default: delete a; return nullptr;
    }
    return a;
}
void dlspm_gen_pattern_destroy(void* h) { delete static_cast<Csr*>(h); }
int dlspm_gen_pattern_nnz(const void* h) { return static_cast<const Csr*>(h)->nnz(); }
void dlspm_gen_pattern_copy(const void* h, int* row_offsets, int* col_indices)
{
    const auto* a = static_cast<const Csr*>(h);
    std::memcpy(row_offsets, a->row_offsets.data(), a->row_offsets.size() * sizeof(int));
    if (!a->col_indices.empty()) std::memcpy(col_indices, a->col_indices.data(), a->col_indices.size() * sizeof(int));
}

// ---- dense fills ---------------------------------------------------------------------------------
void dlspm_gen_fill_uniform(uint64_t seed, size_t n, float lo, float hi, float* out) { fill_uniform(seed, n, lo, hi, out); }
void dlspm_gen_fill_normal(uint64_t seed, size_t n, float mean, float stddev, float* out) { fill_normal(seed, n, mean, stddev, out); }
void dlspm_gen_fill_relu_like(uint64_t seed, size_t n, double p_zero, float* out) { fill_relu_like(seed, n, p_zero, out); }

// ---- accounting ----------------------------------------------------------------------------------
// out[0] = flops, out[1] = algorithmic bytes, out[2] = effective ("application") bytes
void dlspm_account(int op, double M, double K, double N, double nnz, double* out)
{
    const Accounting a = account(static_cast<Op>(op), M, K, N, nnz);
    out[0] = a.flops; out[1] = a.algorithmic_B; out[2] = a.effective_B;
}

}  // extern "C"
