// Calls every entry point that does its work on the host -- the size queries, the advice, the launch descriptions --
// and, without a device, the compute entry points (which must answer with a status and touch nothing) over edge values
// and random sizes up to INT_MAX. No GPU needed. Run as it is, it shows that nothing crashes; built with the sanitizers
// it shows that no size computation overflows:
//   make -C tests/host_fuzz san     (compiles the library's sources once more, host side with ASan + UBSan, into
//                                    tests/host_fuzz/build/, and runs this program against that build)
#include <cstdio>
#include <cstdint>
#include <climits>
#include <random>
#include "../../include/dlspm_hip.h"
int main()
{
    std::mt19937_64 rng(1);
    const int edge[] = {0, 1, 2, 3, 4, 5, 63, 64, 65, 255, 256, 257, 511, 512, 2047, 2048, 2049, 4096, 65535, 65536, 1 << 20, (1 << 24) + 1, 1 << 30, INT_MAX - 1, INT_MAX};
    const int ne = sizeof(edge) / sizeof(edge[0]);
    long long calls = 0;
    // with a device in the machine the compute entry points would launch: they are called only where there is none
    const bool no_device = dlspm_device_info(nullptr, nullptr, nullptr) == DLSPM_E_NO_DEVICE;
    auto one = [&](int op, int M, int K, int W, int nnz, int longest) {
        volatile size_t b = dlspm_workspace_bytes(op, M, K, W, nnz);
        volatile int a = dlspm_workspace_advice(op, M, K, W, nnz, longest);
        volatile int p = dlspm_row_plan_advice(op, M, K, W, nnz, longest);
        int s = 0, r = 0;
        (void)dlspm_describe_slices(op, M, K, W, nnz, &s, &r);
        int shape[16] = {0};
        (void)dlspm_describe_launch(op, M, K, W, nnz, shape);
        (void)dlspm_describe_launch_rows(op, M, K, W, nnz, DLSPM_PASS_ROWS_EVEN, shape);
        (void)dlspm_describe_launch_rows(op, M, K, W, nnz, DLSPM_PASS_WORKSPACE, shape);
        (void)dlspm_describe_launch_rows(op, M, K, W, nnz, DLSPM_PASS_ROWS_SKEWED, shape);
        volatile size_t pb = dlspm_row_plan_bytes(M);
        volatile size_t cb = dlspm_row_plan_bytes_for(op, M, W);
        // the one-look advice on a matrix description of these sizes (any figures: it must answer or refuse, never crash)
        dlspm_matrix_info mi = {M, K, nnz, longest, (int)(nnz % 7), K / 3 + 1, (int)((unsigned)nnz % 8001u), (int)((unsigned)M % 8001u)};
        dlspm_call_plan cp;
        volatile int ad = dlspm_advise(op, W, &mi, &cp);
        (void)b; (void)a; (void)p; (void)pb; (void)cb; (void)ad;
        if (!no_device) { calls += 10; return; }
        // the compute entry points without a device and with pointers that must not be touched: a status, nothing else
        float* bad = reinterpret_cast<float*>(16);
        int* badi = reinterpret_cast<int*>(16);
        volatile int e1 = spmm_csr_f32(M, K, W, nnz, badi, badi, bad, bad, bad, nullptr, 0, nullptr);
        volatile int e2 = sddmm_csr_f32(M, K, W, nnz, badi, badi, bad, bad, bad, nullptr, DLSPM_HINT_ROWS_EVEN, nullptr);
        volatile int e3 = fused_sddmm_spmm_f32(M, K, W, nnz, badi, badi, bad, bad, bad, 0.5f, bad, bad, (size_t)longest | DLSPM_HINT_ROW_PLAN, nullptr);
        volatile int e4 = dlspm_row_plan_build(M, badi, bad, (size_t)nnz, nullptr);
        volatile int e5 = spmm_csr_f32_static(M, K, W, nnz, badi, badi, bad, bad, bad, nullptr);
        volatile int e6 = dlspm_row_plan_build_cut(M, badi, bad, (size_t)nnz, nullptr);
        volatile int e7 = sddmm_csr_f32(M, K, W, nnz, badi, badi, bad, bad, bad, bad, (size_t)longest | DLSPM_HINT_CUT_PLAN, nullptr);
        dlspm_matrix_info got;
        volatile int e8 = dlspm_analyze(M, K, nnz, badi, badi, nullptr, &got);
        (void)e1; (void)e2; (void)e3; (void)e4; (void)e5; (void)e6; (void)e7; (void)e8;
        calls += 18;
    };
    for (int op = 0; op < 4; ++op)
        for (int i = 0; i < ne; ++i)
            for (int j = 0; j < ne; ++j)
                for (int k = 0; k < ne; k += 2)
                    for (int l = 0; l < ne; l += 3) one(op, edge[i], edge[j], edge[k], edge[l], edge[(i + l) % ne]);
    for (int t = 0; t < 200000; ++t) {
        if (t % 1000 == 0) {  // the rules and plans as for devices of other sizes, and other cut rules
            dlspm_tuning tune;
            dlspm_tuning_default(&tune);
            const int units[] = {0, 8, 32, 64, 304, 1024};
            const int pcts[] = {0, 10, 33, 75, 100, 1000};
            tune.compute_units = units[rng() % 6];
            tune.cut_piece_pct = pcts[rng() % 6];
            tune.cut_longest_pct = pcts[rng() % 6];
            tune.rules_off = (int)(rng() % 2048);
            if (dlspm_set_tuning(&tune) != DLSPM_OK) return 1;
        }
        const int op = (int)(rng() % 3);
        const int M = (int)(rng() % (1u << (1 + rng() % 30)));
        const int K = (int)(rng() % (1u << (1 + rng() % 30)));
        const int W = (int)(rng() % (1u << (1 + rng() % 14)));
        const int nnz = (int)(rng() % (1u << (1 + rng() % 30)));
        const int longest = (int)(rng() % 3) == 0 ? -1 : (int)(rng() % (1u << (1 + rng() % 20)));
        one(op, M, K, W, nnz, longest);
    }
    std::printf("host_fuzz: %lld calls%s, nothing reported\n", calls, no_device ? " (compute entry points included: no device)" : "");
    return 0;
}
