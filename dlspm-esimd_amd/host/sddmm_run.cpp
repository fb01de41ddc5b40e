// sddmm_run: self-checking SDDMM benchmark driver over libdlspm_hip (sddmm_csr_f32).
// Takes the place of the reference's SDDMM drivers: single synthetic matrix (SDDMM/sddmm-esimd-v2.cpp:132-371),
// in-process sweep (SDDMM/sddmm-esimd-allbench_v4.cpp:38-255), from file (SDDMM/sddmm-esimd-fromfile_v4.cpp:39-259)
// and the shell loop over DLMC files (SDDMM/batch-run-sddmm_fromfile). N on the command line is the inner
// (feature) dimension, as NSZ is in the reference's SDDMM files.
#include "driver.hpp"

using namespace dlspm;

static bool run_case(const CaseSpec& s, const Options& opt)
{
    Csr a;
    std::vector<float> lhs, rhs;
    int D = s.N;
    if (s.kind == CaseSpec::kCfg) {
        Problem p;
        if (!make_config(s.cfg, p)) throw std::invalid_argument("unknown configuration id");
        if (p.op != kSddmm) throw std::invalid_argument(std::string(p.name) + " is not an SDDMM configuration");
        std::cout << "configuration " << p.name << std::endl;
        a = std::move(p.a); lhs = std::move(p.d0); rhs = std::move(p.d1); D = p.N;
    } else {
        if (s.kind == CaseSpec::kFile) {
            std::cout << "Filename = " << s.file << ", batchsize (=NSZ) = " << D << std::endl;
            a = load_smtx(s.file);
        } else {
            a = synthetic_pattern(s);
        }
        if (D < 1) throw std::invalid_argument("NSZ must be at least 1");
        lhs.resize((size_t)a.M * D);
        rhs.resize((size_t)a.K * D);
        fill_uniform(s.seed ^ 0xB2, lhs.size(), 0.f, 1.f, lhs.data());  // rand()/RAND_MAX in the reference
        fill_uniform(s.seed ^ 0xC3, rhs.size(), 0.f, 1.f, rhs.data());
    }
    const int M = a.M, K = a.K, nnz = a.nnz();
    std::printf("MSZ: %d, KSZ: %d, NSZ: %d, nnz: %d\n", M, K, D, nnz);

    DevBuf<int> ro_d(a.row_offsets), ci_d(a.col_indices), rowof_d((size_t)nnz);
    DevBuf<float> lhs_d(lhs), rhs_d(rhs), out_d((size_t)nnz), ref_d((size_t)nnz);
    if (dlspm_csr_check(M, K, nnz, ro_d.p, ci_d.p, nullptr) != DLSPM_OK) throw std::invalid_argument("malformed CSR structure");
    DLSPM_HIP_CHECK(hipMemset(out_d.p, 0xFF, std::max(nnz, 1) * sizeof(float)));

    // SDDMM needs memory only for the slice boundaries of the column-sliced schedule or for a plan; otherwise the
    // argument only carries what dlspm_advise found out about the rows and columns
    const PreparedCall pc = prepare_call(opt, DLSPM_OP_SDDMM, M, K, D, nnz, ro_d.p, ci_d.p);
    const Timing t = time_launches(opt, [&](hipStream_t stream) {
        return sddmm_csr_f32(M, K, D, nnz, ro_d.p, ci_d.p, lhs_d.p, rhs_d.p, out_d.p, pc.arg(), pc.size(), stream);
    });
    hipLaunchKernelGGL(check_row_of_slot_kernel, dim3(blocks_for(M)), dim3(256), 0, nullptr, M, ro_d.p, rowof_d.p);
    hipLaunchKernelGGL(check_sddmm_kernel, dim3(blocks_for(nnz)), dim3(256), 0, nullptr, nnz, D, rowof_d.p, ci_d.p, lhs_d.p,
                       rhs_d.p, 1.0f, ref_d.p);
    DLSPM_HIP_CHECK(hipGetLastError());
    DLSPM_HIP_CHECK(hipDeviceSynchronize());

    const std::vector<float> got = out_d.to_host(), ref = ref_d.to_host();
    const Diff d = compare(ref, got);
    const bool intact = ro_d.to_host() == a.row_offsets && ci_d.to_host() == a.col_indices;
    report("sddmm", kSddmm, M, K, D, nnz, t, d, intact, opt);

    const Accounting acc = account(kSddmm, M, K, D, nnz);
    const double gflops = acc.flops / (t.min_ms * 1e-3) * 1e-9;
    const double density = (double)nnz / ((double)M * K);
    if (!opt.csv.empty()) {
        std::ofstream csv(opt.csv, std::ios::app | std::ios::out);
        if (s.kind == CaseSpec::kFile)  // columns of SDDMM/sddmm-esimd-fromfile_v4.cpp:236-241
            csv << M << "," << K << "," << D << "," << density << "," << gflops << "," << acc.flops << "," << d.max_diff << std::endl;
        else                            // columns of SDDMM/sddmm-esimd-allbench_v4.cpp:204-209 (calc_bw = application GB/s)
            csv << M << "," << K << "," << D << "," << density << "," << gflops << ","
                << acc.effective_B / (t.min_ms * 1e-3) * 1e-9 << ", " << d.max_diff << std::endl;
    }
    if (!opt.dump.empty()) {
        dump_array(opt.dump, "row_offsets.i32", a.row_offsets.data(), a.row_offsets.size() * 4);
        dump_array(opt.dump, "col_indices.i32", a.col_indices.data(), a.col_indices.size() * 4);
        dump_array(opt.dump, "lhs.f32", lhs.data(), lhs.size() * 4);
        dump_array(opt.dump, "rhs.f32", rhs.data(), rhs.size() * 4);
        dump_array(opt.dump, "out.f32", got.data(), got.size() * 4);
        std::ostringstream meta;
        meta << "{\"op\": \"sddmm\", \"M\": " << M << ", \"K\": " << K << ", \"N\": " << D << ", \"nnz\": " << nnz << "}\n";
        dump_array(opt.dump, "meta.json", meta.str().data(), meta.str().size());
    }
    return intact && d.rel_frobenius <= opt.tol;
}

int main(int argc, char** argv)
{
    try {
        const Cli cli = parse_cli(argc, argv, "sddmm_run", "NSZ");
        print_device();
        bool ok = true;
        for (size_t i = 0; i < cli.cases.size(); ++i) ok = run_case(cli.cases[i], case_options(cli.opt, i)) && ok;
        return ok ? 0 : 2;
    } catch (std::exception& e) {
        std::cout << e.what() << std::endl;
        return 1;
    }
}
