// fused_run: self-checking fused SDDMM->SpMM benchmark driver over libdlspm_hip (fused_sddmm_spmm_f32).
// Takes the place of the reference's FUSED/fused-esimd_cb.cpp main (:223-386; compile-time -DMSZ/-DKSZ/-DNSZ/-DSP,
// values rand()*0.01) and of FUSED/batch-run-fused, which recompiles it per shape. N on the command line is the
// feature dimension D; --scale sets the score factor (1 = the reference's semantics; --cfg 5 uses 1/8).
// The cross-check follows the reference's gold: Sddmm (double) -> fp32 scores -> Spmm (double), FUSED/fused.cpp:400-404.
#include "driver.hpp"

using namespace dlspm;

static float g_scale = 1.0f;

static bool run_case(const CaseSpec& s, const Options& opt)
{
    Csr a;
    std::vector<float> Q, Km, V;
    int D = s.N;
    float scale = g_scale;
    if (s.kind == CaseSpec::kCfg) {
        Problem p;
        if (!make_config(s.cfg, p)) throw std::invalid_argument("unknown configuration id");
        if (p.op != kFused) throw std::invalid_argument(std::string(p.name) + " is not a fused configuration");
        std::cout << "configuration " << p.name << std::endl;
        a = std::move(p.a); Q = std::move(p.d0); Km = std::move(p.d1); V = std::move(p.d2); D = p.N; scale = p.scale;
    } else {
        if (s.kind == CaseSpec::kFile) {
            std::cout << "Filename = " << s.file << ", batchsize (=NSZ) = " << D << std::endl;
            a = load_smtx(s.file);
        } else {
            a = synthetic_pattern(s);
        }
        if (D < 1) throw std::invalid_argument("NSZ must be at least 1");
        Q.resize((size_t)a.M * D);
        Km.resize((size_t)a.K * D);
        V.resize((size_t)a.K * D);
        fill_uniform(s.seed ^ 0xB2, Q.size(), 0.f, 0.01f, Q.data());  // rand()*0.01 in FUSED/fused-esimd_cb.cpp:270-284
        fill_uniform(s.seed ^ 0xC3, Km.size(), 0.f, 0.01f, Km.data());
        fill_uniform(s.seed ^ 0xD4, V.size(), 0.f, 0.01f, V.data());
    }
    const int M = a.M, K = a.K, nnz = a.nnz();
    std::printf("MSZ: %d, KSZ: %d, NSZ: %d, nnz: %d, scale: %g\n", M, K, D, nnz, scale);

    DevBuf<int> ro_d(a.row_offsets), ci_d(a.col_indices), rowof_d((size_t)nnz);
    DevBuf<float> Q_d(Q), K_d(Km), V_d(V), O_d((size_t)M * D), scores_d((size_t)nnz), ref_d((size_t)M * D);
    if (dlspm_csr_check(M, K, nnz, ro_d.p, ci_d.p, nullptr) != DLSPM_OK) throw std::invalid_argument("malformed CSR structure");
    DLSPM_HIP_CHECK(hipMemset(O_d.p, 0xFF, (size_t)M * D * sizeof(float)));

    const PreparedCall pc = prepare_call(opt, DLSPM_OP_FUSED, M, K, D, nnz, ro_d.p, ci_d.p);  // nothing for small, even problems
    const Timing t = time_launches(opt, [&](hipStream_t stream) {
        return fused_sddmm_spmm_f32(M, K, D, nnz, ro_d.p, ci_d.p, Q_d.p, K_d.p, V_d.p, scale, O_d.p, pc.arg(), pc.size(), stream);
    });
    hipLaunchKernelGGL(check_row_of_slot_kernel, dim3(blocks_for(M)), dim3(256), 0, nullptr, M, ro_d.p, rowof_d.p);
    hipLaunchKernelGGL(check_sddmm_kernel, dim3(blocks_for(nnz)), dim3(256), 0, nullptr, nnz, D, rowof_d.p, ci_d.p, Q_d.p, K_d.p,
                       scale, scores_d.p);
    hipLaunchKernelGGL(check_spmm_f64acc_kernel, dim3(blocks_for((long long)M * D)), dim3(256), 0, nullptr, M, D, ro_d.p, ci_d.p,
                       scores_d.p, V_d.p, ref_d.p);
    DLSPM_HIP_CHECK(hipGetLastError());
    DLSPM_HIP_CHECK(hipDeviceSynchronize());

    const std::vector<float> got = O_d.to_host(), ref = ref_d.to_host();
    const Diff d = compare(ref, got);
    const bool intact = ro_d.to_host() == a.row_offsets && ci_d.to_host() == a.col_indices;
    report("fused", kFused, M, K, D, nnz, t, d, intact, opt);

    if (!opt.csv.empty()) {
        const Accounting acc = account(kFused, M, K, D, nnz);
        std::ofstream csv(opt.csv, std::ios::app | std::ios::out);
        csv << M << "," << K << "," << D << "," << (double)nnz / ((double)M * K) << "," << acc.flops / (t.min_ms * 1e-3) * 1e-9
            << "," << d.max_diff << std::endl;
    }
    if (!opt.dump.empty()) {
        dump_array(opt.dump, "row_offsets.i32", a.row_offsets.data(), a.row_offsets.size() * 4);
        dump_array(opt.dump, "col_indices.i32", a.col_indices.data(), a.col_indices.size() * 4);
        dump_array(opt.dump, "Q.f32", Q.data(), Q.size() * 4);
        dump_array(opt.dump, "K.f32", Km.data(), Km.size() * 4);
        dump_array(opt.dump, "V.f32", V.data(), V.size() * 4);
        dump_array(opt.dump, "O.f32", got.data(), got.size() * 4);
        std::ostringstream meta;
        meta << "{\"op\": \"fused\", \"M\": " << M << ", \"K\": " << K << ", \"N\": " << D << ", \"nnz\": " << nnz
             << ", \"scale\": " << scale << "}\n";
        dump_array(opt.dump, "meta.json", meta.str().data(), meta.str().size());
    }
    return intact && d.rel_frobenius <= opt.tol;
}

int main(int argc, char** argv)
{
    try {
        std::vector<char*> rest;  // peel off --scale, which only this driver has
        for (int i = 0; i < argc; ++i) {
            if (std::string(argv[i]) == "--scale" && i + 1 < argc) g_scale = std::stof(argv[++i]);
            else rest.push_back(argv[i]);
        }
        const Cli cli = parse_cli((int)rest.size(), rest.data(), "fused_run", "NSZ");
        print_device();
        bool ok = true;
        for (size_t i = 0; i < cli.cases.size(); ++i) ok = run_case(cli.cases[i], case_options(cli.opt, i)) && ok;
        return ok ? 0 : 2;
    } catch (std::exception& e) {
        std::cout << e.what() << std::endl;
        return 1;
    }
}
