/*
 * CPU oracle for the SpMM / SDDMM / fused SDDMM->SpMM path.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE. It restates, in plain C, the scalar single-thread
 * loops the reference uses as its own gold, with the same loop order and the same accumulator
 * types, so that the HIP kernels can be checked against it. Only the tests, the smoke check and the
 * CPU-baseline leg of the benchmark may load it; the library never does.
 *
 * Reference loops followed (paths relative to the reference tree):
 *   oracle_spmm_f32      SPMM/spmm-esimd-fromfile.cpp:63-83   (float accumulator, order i -> j -> l)
 *   oracle_spmm_f64acc   FUSED/fused.cpp:67-89                (double accumulator, cast at the end)
 *   oracle_sddmm_f32     SDDMM/sddmm-esimd-fromfile.cpp:18-36 (double accumulator, cast at the end;
 *                        identical text at FUSED/fused.cpp:47-65)
 *   oracle_fused_f32     FUSED/fused.cpp:400-404              (Sddmm, then Spmm with double
 *                        accumulate, the scores rounded to float in between) plus a `scale` factor
 *                        the reference does not have: score = (float)acc * scale in fp32;
 *                        scale = 1.0f is exactly the reference.
 *   oracle_csr_check     SPMM/spmm-esimd-fromfile.cpp:36-61   (SanityCheck; returns which test failed
 *                        instead of throwing)
 * The *_omp variants run the same per-row loop bodies under `#pragma omp parallel for` over rows;
 * rows are independent, so their results are bit-identical to the single-thread ones.
 *
 * How each function is pinned (see tests/test_oracle_*.py):
 *   - oracle_sddmm_f32, oracle_spmm_f64acc, oracle_fused_f32(scale=1): bit-exact against the
 *     reference's own Sddmm / Spmm compiled from FUSED/fused.cpp (oracle/_ref) and against the
 *     fixtures under tests/golden/ that build wrote;
 *   - oracle_spmm_f32: bit-exact against SpmmEsimdCPU of FUSED/fused.cpp:218-303 (same fp32
 *     operation sequence per output element) and the same fixtures; plus closed forms
 *     (identity, all-ones rows, single-entry rows, empty rows), a dense float64 product, brute force
 *     on tiny inputs, linearity and nnz-splitting invariants;
 *   - oracle_fused_f32 with scale != 1: composition spmm_f64acc(sddmm * scale) and a dense float64
 *     ((Q K^T) .* mask * scale) V.
 *   - oracle_csr_check: hand-built malformed CSR cases, one per test of the reference's SanityCheck.
 * Build: see oracle/Makefile (gcc -O2, no -march flags, so no FMA contraction changes the rounding).
 */
#include <stddef.h>
#include <stdint.h>

/* C[i,j] = sum_l val[l] * B[col[l], j], float accumulator, l ascending. Empty rows give 0. */
void oracle_spmm_f32(int M, int N, const int* row_offsets, const int* col_indices,
                     const float* values, const float* B, float* C)
{
    for (int i = 0; i < M; ++i) {
        for (int j = 0; j < N; ++j) {
            float accum = 0.0f;
            for (int l = row_offsets[i]; l < row_offsets[i + 1]; ++l) {
                float a_val = values[l];
                int a_col = col_indices[l];
                accum += a_val * B[(size_t)a_col * N + j];
            }
            C[(size_t)i * N + j] = accum;
        }
    }
}

/* Same product with a double accumulator, rounded to float once per output element. */
void oracle_spmm_f64acc(int M, int N, const int* row_offsets, const int* col_indices,
                        const float* values, const float* B, float* C)
{
    for (int i = 0; i < M; ++i) {
        for (int j = 0; j < N; ++j) {
            double accum = 0.0;
            for (int l = row_offsets[i]; l < row_offsets[i + 1]; ++l) {
                float a_val = values[l];
                int a_col = col_indices[l];
                accum += (double)a_val * (double)B[(size_t)a_col * N + j];
            }
            C[(size_t)i * N + j] = (float)accum;
        }
    }
}

/* out[j] = dot(lhs[i,:], rhs[col[j],:]) over D, double accumulator, for each slot j of row i. */
void oracle_sddmm_f32(int M, int D, const int* row_offsets, const int* col_indices,
                      const float* lhs, const float* rhs, float* out_values)
{
    for (int i = 0; i < M; ++i) {
        for (int j = row_offsets[i]; j < row_offsets[i + 1]; ++j) {
            int idx_n = col_indices[j];
            double accumulator = 0.0;
            for (int l = 0; l < D; ++l) {
                accumulator += (double)lhs[(size_t)i * D + l] * (double)rhs[(size_t)idx_n * D + l];
            }
            out_values[j] = (float)accumulator;
        }
    }
}

/*
 * O = (S .* (Q Kmat^T) * scale) V. `scores` (nnz floats) is scratch supplied by the caller and
 * holds the fp32 scores on return.
 */
void oracle_fused_f32(int M, int D, const int* row_offsets, const int* col_indices,
                      const float* Q, const float* Kmat, const float* V, float scale,
                      float* scores, float* O)
{
    oracle_sddmm_f32(M, D, row_offsets, col_indices, Q, Kmat, scores);
    if (scale != 1.0f) {
        int nnz = row_offsets[M];
        for (int j = 0; j < nnz; ++j) scores[j] = scores[j] * scale;
    }
    oracle_spmm_f64acc(M, D, row_offsets, col_indices, scores, V, O);
}

/*
 * 0 if the CSR structure passes every test of the reference's SanityCheck, otherwise the number of
 * the first failing test: 1 nnz > M*K, 2 row_offsets[M] != nnz, 3 offsets decrease, 4 a row longer
 * than K, 5 a column index >= K. Two additions the reference leaves unchecked but its kernels
 * assume: 6 row_offsets[0] != 0, 7 a negative column index.
 */
int oracle_csr_check(int M, int K, int nnz, const int* row_offsets, const int* col_indices)
{
    if ((long long)nnz > (long long)M * (long long)K) return 1;
    if (row_offsets[M] != nnz) return 2;
    for (int i = 0; i < M; ++i) {
        if (row_offsets[i + 1] < row_offsets[i]) return 3;
        if (row_offsets[i + 1] - row_offsets[i] > K) return 4;
    }
    for (int i = 0; i < nnz; ++i) {
        if (col_indices[i] >= K) return 5;
    }
    if (row_offsets[0] != 0) return 6;
    for (int i = 0; i < nnz; ++i) {
        if (col_indices[i] < 0) return 7;
    }
    return 0;
}

/* ---- the same loops, rows spread over the host's cores (for the "all cores" timing only) ---- */

void oracle_spmm_f32_omp(int M, int N, const int* row_offsets, const int* col_indices,
                         const float* values, const float* B, float* C)
{
#pragma omp parallel for schedule(dynamic, 16)
    for (int i = 0; i < M; ++i) {
        for (int j = 0; j < N; ++j) {
            float accum = 0.0f;
            for (int l = row_offsets[i]; l < row_offsets[i + 1]; ++l) {
                accum += values[l] * B[(size_t)col_indices[l] * N + j];
            }
            C[(size_t)i * N + j] = accum;
        }
    }
}

void oracle_spmm_f64acc_omp(int M, int N, const int* row_offsets, const int* col_indices,
                            const float* values, const float* B, float* C)
{
#pragma omp parallel for schedule(dynamic, 16)
    for (int i = 0; i < M; ++i) {
        for (int j = 0; j < N; ++j) {
            double accum = 0.0;
            for (int l = row_offsets[i]; l < row_offsets[i + 1]; ++l) {
                accum += (double)values[l] * (double)B[(size_t)col_indices[l] * N + j];
            }
            C[(size_t)i * N + j] = (float)accum;
        }
    }
}

void oracle_sddmm_f32_omp(int M, int D, const int* row_offsets, const int* col_indices,
                          const float* lhs, const float* rhs, float* out_values)
{
#pragma omp parallel for schedule(dynamic, 16)
    for (int i = 0; i < M; ++i) {
        for (int j = row_offsets[i]; j < row_offsets[i + 1]; ++j) {
            int idx_n = col_indices[j];
            double accumulator = 0.0;
            for (int l = 0; l < D; ++l) {
                accumulator += (double)lhs[(size_t)i * D + l] * (double)rhs[(size_t)idx_n * D + l];
            }
            out_values[j] = (float)accumulator;
        }
    }
}

void oracle_fused_f32_omp(int M, int D, const int* row_offsets, const int* col_indices,
                          const float* Q, const float* Kmat, const float* V, float scale,
                          float* scores, float* O)
{
    oracle_sddmm_f32_omp(M, D, row_offsets, col_indices, Q, Kmat, scores);
    if (scale != 1.0f) {
        int nnz = row_offsets[M];
        for (int j = 0; j < nnz; ++j) scores[j] = scores[j] * scale;
    }
    oracle_spmm_f64acc_omp(M, D, row_offsets, col_indices, scores, V, O);
}

int oracle_omp_threads(void)
{
    int n = 1;
#ifdef _OPENMP
    extern int omp_get_max_threads(void);
    n = omp_get_max_threads();
#endif
    return n;
}
