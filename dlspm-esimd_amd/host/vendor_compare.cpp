// vendor_compare: libdlspm_hip next to rocSPARSE on the same device and the same seeded inputs.
// Takes the role the cuSPARSE and oneMKL harnesses play in the reference (CUSPARSE/spmm_fromfile.cu:175-234,
// CUSPARSE/sddmm_fromfile.cu:200-224, MKL/onemkl_test.hpp:320-471): a vendor-library baseline on the hardware the
// kernels run on. rocSPARSE is linked only into this program, never into the library. For each configuration it
// times rocsparse_spmm (every CSR algorithm, preprocess excluded) or rocsparse_sddmm, the fused configuration as
// rocsparse_sddmm -> scale -> rocsparse_spmm ("unfused vendor path", as MKL's FusedMM = gemm + sparse gemm), and
// the library's entry point, all as the minimum of `iters` launches bracketed by HIP events, and prints the
// relative Frobenius difference between the two results. Like the reference's comparators it checks itself: the
// exit status is 2 when the two results differ by more than --tol (1e-4), and `--dump <dir>` writes both results
// (cfg<id>_dlspm.f32, cfg<id>_rocsparse.f32) so that an external checker can hold each against its own gold.
#include <rocsparse/rocsparse.h>

#include "driver.hpp"

using namespace dlspm;

#define RS_CHECK(expr)                                                                              \
    do {                                                                                            \
        rocsparse_status s_ = (expr);                                                               \
        if (s_ != rocsparse_status_success)                                                         \
            throw std::runtime_error(std::string(#expr) + ": rocsparse status " + std::to_string((int)s_)); \
    } while (0)

template <typename F> static double min_ms(int warmup, int iters, F&& f)
{
    hipEvent_t e0, e1;
    DLSPM_HIP_CHECK(hipEventCreate(&e0));
    DLSPM_HIP_CHECK(hipEventCreate(&e1));
    double best = 1e30;
    for (int i = 0; i < warmup + iters; ++i) {
        DLSPM_HIP_CHECK(hipEventRecord(e0, nullptr));
        f();
        DLSPM_HIP_CHECK(hipEventRecord(e1, nullptr));
        DLSPM_HIP_CHECK(hipEventSynchronize(e1));
        float ms = 0;
        DLSPM_HIP_CHECK(hipEventElapsedTime(&ms, e0, e1));
        if (i >= warmup) best = std::min(best, (double)ms);
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    return best;
}

__global__ void scale_kernel(int n, float s, float* x)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) x[i] *= s;
}

struct AlgName { rocsparse_spmm_alg alg; const char* name; };
static const AlgName kSpmmAlgs[] = {{rocsparse_spmm_alg_default, "default"},
                                    {rocsparse_spmm_alg_csr, "csr"},
                                    {rocsparse_spmm_alg_csr_row_split, "csr_row_split"},
                                    {rocsparse_spmm_alg_csr_nnz_split, "csr_nnz_split"},
                                    {rocsparse_spmm_alg_csr_merge_path, "csr_merge_path"}};

// C = A_csr * B with rocSPARSE, every algorithm; returns the best time and leaves that algorithm's result in C
static double rocsparse_spmm_best(rocsparse_handle h, int M, int K, int N, int nnz, int* ro, int* ci, float* va, float* B,
                                  float* C, int warmup, int iters, std::string& best_name)
{
    rocsparse_spmat_descr A;
    rocsparse_dnmat_descr Bd, Cd;
    RS_CHECK(rocsparse_create_csr_descr(&A, M, K, nnz, ro, ci, va, rocsparse_indextype_i32, rocsparse_indextype_i32,
                                        rocsparse_index_base_zero, rocsparse_datatype_f32_r));
    RS_CHECK(rocsparse_create_dnmat_descr(&Bd, K, N, N, B, rocsparse_datatype_f32_r, rocsparse_order_row));
    RS_CHECK(rocsparse_create_dnmat_descr(&Cd, M, N, N, C, rocsparse_datatype_f32_r, rocsparse_order_row));
    const float alpha = 1.f, beta = 0.f;
    double best = 1e30;
    for (const auto& a : kSpmmAlgs) {
        size_t bytes = 0;
        if (rocsparse_spmm(h, rocsparse_operation_none, rocsparse_operation_none, &alpha, A, Bd, &beta, Cd,
                           rocsparse_datatype_f32_r, a.alg, rocsparse_spmm_stage_buffer_size, &bytes, nullptr) !=
            rocsparse_status_success) {
            std::printf("    rocsparse_spmm %-16s not available\n", a.name);
            continue;
        }
        DevBuf<char> tmp(bytes);
        if (rocsparse_spmm(h, rocsparse_operation_none, rocsparse_operation_none, &alpha, A, Bd, &beta, Cd,
                           rocsparse_datatype_f32_r, a.alg, rocsparse_spmm_stage_preprocess, &bytes, tmp.p) !=
            rocsparse_status_success) {
            std::printf("    rocsparse_spmm %-16s preprocess failed\n", a.name);
            continue;
        }
        bool ok = true;
        const double t = min_ms(warmup, iters, [&]() {
            ok = ok && rocsparse_spmm(h, rocsparse_operation_none, rocsparse_operation_none, &alpha, A, Bd, &beta, Cd,
                                      rocsparse_datatype_f32_r, a.alg, rocsparse_spmm_stage_compute, &bytes,
                                      tmp.p) == rocsparse_status_success;
        });
        if (!ok) {
            std::printf("    rocsparse_spmm %-16s failed\n", a.name);
            continue;
        }
        std::printf("    rocsparse_spmm %-16s %9.2f us  (workspace %zu bytes)\n", a.name, t * 1e3, bytes);
        if (t < best) {
            best = t;
            best_name = a.name;
        }
    }
    // leave the default algorithm's result in C for the comparison
    size_t bytes = 0;
    RS_CHECK(rocsparse_spmm(h, rocsparse_operation_none, rocsparse_operation_none, &alpha, A, Bd, &beta, Cd,
                            rocsparse_datatype_f32_r, rocsparse_spmm_alg_default, rocsparse_spmm_stage_buffer_size, &bytes,
                            nullptr));
    DevBuf<char> tmp(bytes);
    RS_CHECK(rocsparse_spmm(h, rocsparse_operation_none, rocsparse_operation_none, &alpha, A, Bd, &beta, Cd,
                            rocsparse_datatype_f32_r, rocsparse_spmm_alg_default, rocsparse_spmm_stage_preprocess, &bytes, tmp.p));
    RS_CHECK(rocsparse_spmm(h, rocsparse_operation_none, rocsparse_operation_none, &alpha, A, Bd, &beta, Cd,
                            rocsparse_datatype_f32_r, rocsparse_spmm_alg_default, rocsparse_spmm_stage_compute, &bytes, tmp.p));
    DLSPM_HIP_CHECK(hipDeviceSynchronize());
    (void)rocsparse_destroy_spmat_descr(A);
    (void)rocsparse_destroy_dnmat_descr(Bd);
    (void)rocsparse_destroy_dnmat_descr(Cd);
    return best;
}

// out = S .* (lhs * rhs^T) with rocSPARSE; rhs (K x D row-major) is handed over as a D x K column-major matrix
struct RsSddmm {
    rocsparse_handle h;
    rocsparse_dnmat_descr A, Bt;
    rocsparse_spmat_descr Cs;
    DevBuf<char> tmp;
    float alpha = 1.f, beta = 0.f;
    RsSddmm(rocsparse_handle h_, int M, int K, int D, int nnz, int* ro, int* ci, float* lhs, float* rhs, float* out) : h(h_)
    {
        RS_CHECK(rocsparse_create_dnmat_descr(&A, M, D, D, lhs, rocsparse_datatype_f32_r, rocsparse_order_row));
        RS_CHECK(rocsparse_create_dnmat_descr(&Bt, D, K, D, rhs, rocsparse_datatype_f32_r, rocsparse_order_column));
        RS_CHECK(rocsparse_create_csr_descr(&Cs, M, K, nnz, ro, ci, out, rocsparse_indextype_i32, rocsparse_indextype_i32,
                                            rocsparse_index_base_zero, rocsparse_datatype_f32_r));
        size_t bytes = 0;
        RS_CHECK(rocsparse_sddmm_buffer_size(h, rocsparse_operation_none, rocsparse_operation_none, &alpha, A, Bt, &beta, Cs,
                                             rocsparse_datatype_f32_r, rocsparse_sddmm_alg_default, &bytes));
        tmp = DevBuf<char>(bytes);
        RS_CHECK(rocsparse_sddmm_preprocess(h, rocsparse_operation_none, rocsparse_operation_none, &alpha, A, Bt, &beta, Cs,
                                            rocsparse_datatype_f32_r, rocsparse_sddmm_alg_default, tmp.p));
    }
    rocsparse_status run()
    {
        return rocsparse_sddmm(h, rocsparse_operation_none, rocsparse_operation_none, &alpha, A, Bt, &beta, Cs,
                               rocsparse_datatype_f32_r, rocsparse_sddmm_alg_default, tmp.p);
    }
    ~RsSddmm()
    {
        (void)rocsparse_destroy_dnmat_descr(A);
        (void)rocsparse_destroy_dnmat_descr(Bt);
        (void)rocsparse_destroy_spmat_descr(Cs);
    }
};

static double rel_frob(const std::vector<float>& ref, const std::vector<float>& x)
{
    return compare(ref, x).rel_frobenius;
}

int main(int argc, char** argv)
{
    try {
        int iters = 50, warmup = 10;
        double tol = 1e-4;
        std::string dump;
        bool all_ok = true;
        std::vector<int> cfgs = {1, 2, 3, 4, 5};
        for (int i = 1; i < argc; ++i) {
            const std::string a = argv[i];
            if (a == "--iters" && i + 1 < argc) iters = std::max(1, std::stoi(argv[++i]));
            else if (a == "--cfg" && i + 1 < argc) cfgs = {std::stoi(argv[++i])};
            else if (a == "--tol" && i + 1 < argc) tol = std::stod(argv[++i]);
            else if (a == "--dump" && i + 1 < argc) dump = argv[++i];
            else throw std::invalid_argument("Usage: vendor_compare [--cfg <id>] [--iters n] [--tol x] [--dump <dir>]");
        }
        print_device();
        rocsparse_handle h;
        RS_CHECK(rocsparse_create_handle(&h));
        std::printf("%-44s %12s %12s %8s %12s\n", "configuration", "dlspm us", "rocsparse us", "speedup", "rel.diff");
        for (int cfg : cfgs) {
            Problem p;
            if (!make_config(cfg, p)) throw std::invalid_argument("unknown configuration id");
            const int M = p.M, K = p.K, N = p.N, nnz = p.a.nnz();
            std::printf("%s  (M=%d K=%d N/D=%d nnz=%d)\n", p.name, M, K, N, nnz);
            DevBuf<int> ro(p.a.row_offsets), ci(p.a.col_indices);
            double t_ours = 0, t_vendor = 0, diff = 0;
            std::string alg = "default";
            std::vector<float> ours, vendor;
            if (p.op == kSpmm) {
                DevBuf<float> va(p.values), B(p.d0), C((size_t)M * N), Cv((size_t)M * N);
                t_ours = min_ms(warmup, iters, [&]() { (void)spmm_csr_f32(M, K, N, nnz, ro.p, ci.p, va.p, B.p, C.p, nullptr, 0, nullptr); });
                t_vendor = rocsparse_spmm_best(h, M, K, N, nnz, ro.p, ci.p, va.p, B.p, Cv.p, warmup, iters, alg);
                ours = C.to_host();
                vendor = Cv.to_host();
            } else if (p.op == kSddmm) {
                DevBuf<float> lhs(p.d0), rhs(p.d1), out((size_t)nnz), outv((size_t)nnz);
                DLSPM_HIP_CHECK(hipMemset(outv.p, 0, (size_t)nnz * sizeof(float)));
                t_ours = min_ms(warmup, iters, [&]() { (void)sddmm_csr_f32(M, K, N, nnz, ro.p, ci.p, lhs.p, rhs.p, out.p, nullptr, 0, nullptr); });
                RsSddmm rs(h, M, K, N, nnz, ro.p, ci.p, lhs.p, rhs.p, outv.p);
                t_vendor = min_ms(warmup, iters, [&]() { (void)rs.run(); });
                std::printf("    rocsparse_sddmm default          %9.2f us\n", t_vendor * 1e3);
                ours = out.to_host();
                vendor = outv.to_host();
            } else {
                DevBuf<float> Q(p.d0), Km(p.d1), V(p.d2), O((size_t)M * N), Ov((size_t)M * N), scores((size_t)nnz);
                DLSPM_HIP_CHECK(hipMemset(scores.p, 0, (size_t)nnz * sizeof(float)));
                t_ours = min_ms(warmup, iters, [&]() {
                    (void)fused_sddmm_spmm_f32(M, K, N, nnz, ro.p, ci.p, Q.p, Km.p, V.p, p.scale, O.p, nullptr, 0, nullptr);
                });
                RsSddmm rs(h, M, K, N, nnz, ro.p, ci.p, Q.p, Km.p, scores.p);
                const double t_sddmm = min_ms(warmup, iters, [&]() { (void)rs.run(); });
                const double t_scale = min_ms(warmup, iters, [&]() {
                    hipLaunchKernelGGL(scale_kernel, dim3(blocks_for(nnz)), dim3(256), 0, nullptr, nnz, 1.0f, scores.p);
                });
                (void)rs.run();
                hipLaunchKernelGGL(scale_kernel, dim3(blocks_for(nnz)), dim3(256), 0, nullptr, nnz, p.scale, scores.p);
                const double t_spmm = rocsparse_spmm_best(h, M, K, N, nnz, ro.p, ci.p, scores.p, V.p, Ov.p, warmup, iters, alg);
                std::printf("    unfused vendor path: rocsparse_sddmm %.2f us + scale %.2f us + rocsparse_spmm(%s) %.2f us\n",
                            t_sddmm * 1e3, t_scale * 1e3, alg.c_str(), t_spmm * 1e3);
                t_vendor = t_sddmm + t_scale + t_spmm;
                ours = O.to_host();
                vendor = Ov.to_host();
            }
            diff = rel_frob(vendor, ours);
            if (!(diff <= tol)) all_ok = false;
            if (!dump.empty()) {
                const std::string tag = "cfg" + std::to_string(cfg);
                dump_array(dump, (tag + "_dlspm.f32").c_str(), ours.data(), ours.size() * 4);
                dump_array(dump, (tag + "_rocsparse.f32").c_str(), vendor.data(), vendor.size() * 4);
            }
            std::printf("%-44s %12.2f %12.2f %7.2fx %12.3e   (best rocSPARSE algorithm: %s)\n\n", p.name, t_ours * 1e3,
                        t_vendor * 1e3, t_vendor / t_ours, diff, alg.c_str());
        }
        (void)rocsparse_destroy_handle(h);
        std::printf("vendor_compare %s (tolerance %g)\n", all_ok ? "PASS" : "FAIL", tol);
        return all_ok ? 0 : 2;
    } catch (std::exception& e) {
        std::cout << e.what() << std::endl;
        return 1;
    }
}
