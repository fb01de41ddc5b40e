// spmm_run: self-checking SpMM benchmark driver over libdlspm_hip (spmm_csr_f32).
// Takes the place of the reference's SpMM drivers: single synthetic matrix (SPMM/spmm-esimd-v1.cpp:281-466),
// in-process sweep (SPMM/spmm-esimd-allbenchs2.cpp:56-266), from file (SPMM/spmm-esimd-fromfile2.cpp:86-320) and
// the shell loop over DLMC files (SPMM/batch-run-spmm_fromfile:16-46). See driver.hpp for the shared parts.
#include <chrono>

#include "driver.hpp"

using namespace dlspm;

static bool run_case(const CaseSpec& s, const Options& opt)
{
    Csr a;
    std::vector<float> values, B;
    int N = s.N;
    if (s.kind == CaseSpec::kCfg) {
        Problem p;
        if (!make_config(s.cfg, p)) throw std::invalid_argument("unknown configuration id");
        if (p.op != kSpmm) throw std::invalid_argument(std::string(p.name) + " is not an SpMM configuration");
        std::cout << "configuration " << p.name << std::endl;
        a = std::move(p.a); values = std::move(p.values); B = std::move(p.d0); N = p.N;
    } else {
        if (s.kind == CaseSpec::kFile) {
            std::cout << "Filename = " << s.file << ", batchsize (=NSZ) = " << N << std::endl;
            a = load_smtx(s.file);
        } else {
            a = synthetic_pattern(s);
        }
        if (N < 1) throw std::invalid_argument("NSZ must be at least 1");
        values.resize(a.nnz());
        // value ranges as in the reference: rand()/RAND_MAX from file (SPMM/spmm-esimd-fromfile2.cpp:134),
        // times 0.01 in the synthetic sweep (SPMM/spmm-esimd-allbenchs2.cpp:74); B is rand()/RAND_MAX in both
        fill_uniform(s.seed ^ 0xA1, values.size(), 0.f, s.kind == CaseSpec::kFile ? 1.f : 0.01f, values.data());
        B.resize((size_t)a.K * N);
        fill_uniform(s.seed ^ 0xB2, B.size(), 0.f, 1.f, B.data());
    }
    const int M = a.M, K = a.K, nnz = a.nnz();
    std::printf("MSZ: %d, KSZ: %d, NSZ: %d, nnz: %d\n", M, K, N, nnz);

    DevBuf<int> ro_d(a.row_offsets), ci_d(a.col_indices);
    DevBuf<float> va_d(values), B_d(B), C_d((size_t)M * N), Cref_d((size_t)M * N);
    if (dlspm_csr_check(M, K, nnz, ro_d.p, ci_d.p, nullptr) != DLSPM_OK) throw std::invalid_argument("malformed CSR structure");
    DLSPM_HIP_CHECK(hipMemset(C_d.p, 0xFF, (size_t)M * N * sizeof(float)));  // NaN pattern: every element must be written

    // the caller owns the workspace, as it owns every other buffer. Once per matrix: one look at it (dlspm_analyze) and
    // the library's answer for this op and width (dlspm_advise) -- nothing, a hint, schedule memory, or a plan built here
    const PreparedCall pc = prepare_call(opt, DLSPM_OP_SPMM, M, K, N, nnz, ro_d.p, ci_d.p);
    const Timing t = time_launches(opt, [&](hipStream_t stream) {
        return spmm_csr_f32(M, K, N, nnz, ro_d.p, ci_d.p, va_d.p, B_d.p, C_d.p, pc.arg(), pc.size(), stream);
    });
    hipLaunchKernelGGL(check_spmm_kernel, dim3(blocks_for((long long)M * N)), dim3(256), 0, nullptr, M, N, ro_d.p, ci_d.p,
                       va_d.p, B_d.p, Cref_d.p);
    DLSPM_HIP_CHECK(hipGetLastError());
    DLSPM_HIP_CHECK(hipDeviceSynchronize());

    const std::vector<float> got = C_d.to_host(), ref = Cref_d.to_host();
    const Diff d = compare(ref, got);
    const bool intact = ro_d.to_host() == a.row_offsets && ci_d.to_host() == a.col_indices;
    report("spmm", kSpmm, M, K, N, nnz, t, d, intact, opt);

    const Accounting acc = account(kSpmm, M, K, N, nnz);
    const double gflops = acc.flops / (t.min_ms * 1e-3) * 1e-9;
    const double density = (double)nnz / ((double)M * K);
    if (!opt.csv.empty()) {
        std::ofstream csv(opt.csv, std::ios::app | std::ios::out);
        if (s.kind == CaseSpec::kFile)  // columns of SPMM/spmm-esimd-fromfile2.cpp:289-294
            csv << M << "," << N << "," << K << "," << density << "," << gflops << "," << d.max_diff << "," << acc.flops << std::endl;
        else                            // columns of SPMM/spmm-esimd-allbenchs2.cpp:221-226
            csv << M << "," << N << "," << K << "," << density << "," << gflops << "," << d.max_rel_diff << std::endl;
    }
    if (!opt.dump.empty()) {
        dump_array(opt.dump, "row_offsets.i32", a.row_offsets.data(), a.row_offsets.size() * 4);
        dump_array(opt.dump, "col_indices.i32", a.col_indices.data(), a.col_indices.size() * 4);
        dump_array(opt.dump, "values.f32", values.data(), values.size() * 4);
        dump_array(opt.dump, "B.f32", B.data(), B.size() * 4);
        dump_array(opt.dump, "C.f32", got.data(), got.size() * 4);
        std::ostringstream meta;
        meta << "{\"op\": \"spmm\", \"M\": " << M << ", \"K\": " << K << ", \"N\": " << N << ", \"nnz\": " << nnz << "}\n";
        dump_array(opt.dump, "meta.json", meta.str().data(), meta.str().size());
    }
    return intact && d.rel_frobenius <= opt.tol;
}

int main(int argc, char** argv)
{
    try {
        const Cli cli = parse_cli(argc, argv, "spmm_run", "batchsize");
        print_device();
        bool ok = true;
        for (size_t i = 0; i < cli.cases.size(); ++i) ok = run_case(cli.cases[i], case_options(cli.opt, i)) && ok;
        return ok ? 0 : 2;
    } catch (std::exception& e) {  // the reference prints the message and carries on to exit (…fromfile2.cpp:306-319)
        std::cout << e.what() << std::endl;
        return 1;
    }
}
