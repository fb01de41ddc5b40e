// Shared plumbing of the three drivers (spmm_run, sddmm_run, fused_run): problem sources, device buffers,
// the timing loop, the on-device cross-check and the report.
//
// The drivers keep the call surface of the reference's self-checking benchmark programs:
//   single synthetic matrix   SPMM/spmm-esimd-v1.cpp:281-466 (shape by -DMSZ/-DKSZ/-DNSZ/-DSP)  ->  --shape M K N density
//   in-process sweep          SPMM/spmm-esimd-allbenchs2.cpp:56-266 (RunBenchmarkCase over the grid) ->  --sweep
//   from file                 SPMM/spmm-esimd-fromfile2.cpp:86-320 (`./app <file>.smtx <batchsize>`)  ->  <file>.smtx <N>
//   shell loop over DLMC      SPMM/batch-run-spmm_fromfile:16-46                                      ->  --batch <list>
// plus the five seeded benchmark configurations (--cfg 1..5). Per case they print what the reference prints
// (sizes, nnz, minimum kernel time over the timed launches, GFLOP/s with the reference's flop formula, checksums,
// largest difference) and, beyond it, median time, effective and algorithmic GB/s against the 8 TB/s HBM peak.
//
// Cross-check: the drivers do not contain a CPU implementation. The optimised kernel's output is compared on the
// device against check kernels that compute one output element per thread straight from the definition, with the
// accumulator types of the reference's gold loops (float for SpMM, SPMM/spmm-esimd-fromfile2.cpp:63-83; double for
// SDDMM and for both stages of the fused op, FUSED/fused.cpp:47-89). `--dump DIR` writes inputs and outputs as raw
// little-endian arrays so that an external checker can verify them as well.
#pragma once

#include <hip/hip_runtime.h>

#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <filesystem>
#include <fstream>
#include <iostream>
#include <sstream>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../include/dlspm_hip.h"
#include "gen.hpp"

namespace dlspm {

#define DLSPM_HIP_CHECK(expr)                                                                          \
    do {                                                                                               \
        hipError_t e_ = (expr);                                                                        \
        if (e_ != hipSuccess)                                                                          \
            throw std::runtime_error(std::string(#expr) + ": " + hipGetErrorString(e_));              \
    } while (0)

// ---- CSR validity, as the reference's SanityCheck (SPMM/spmm-esimd-fromfile2.cpp:36-61), same messages ----------
inline bool sanity_check(int M, int K, int nnz, const int* ro, const int* ci)
{
    if ((long long)nnz > (long long)M * K) throw std::invalid_argument("nnz is larger than matrix.");
    if (ro[M] != nnz) throw std::invalid_argument("a_row_offsets[MSZ] != nnz.");
    for (int i = 0; i < M; i++) {
        if (ro[i + 1] < ro[i]) throw std::invalid_argument("a_row_offsets[i+1] < a_row_offsets[i]");
        if (ro[i + 1] - ro[i] > K) throw std::invalid_argument("a_row_offsets[i + 1] - a_row_offsets[i] > KSZ");
    }
    for (int i = 0; i < nnz; i++) {
        if (ci[i] >= K) throw std::invalid_argument("a_column_indices[i] >= KSZ");
        if (ci[i] < 0) throw std::invalid_argument("a_column_indices[i] < 0");
    }
    if (ro[0] != 0) throw std::invalid_argument("a_row_offsets[0] != 0");
    return true;
}

// ---- .smtx loader: "M, K, nnz" then M+1 row offsets then nnz column indices (dlmc/README;
//      SPMM/spmm-esimd-fromfile2.cpp:106-137). Throws std::logic_error like the reference on a bad file. ---------
inline Csr load_smtx(const std::string& path)
{
    FILE* fp = std::fopen(path.c_str(), "r");
    if (fp == nullptr) throw std::logic_error("Error opening file!");
    Csr a;
    int nnz = 0;
    if (std::fscanf(fp, "%d,%d,%d", &a.M, &a.K, &nnz) != 3) {
        std::fclose(fp);
        throw std::logic_error("Something went wrong readin M, K, nnz");
    }
    if (a.M < 0 || a.K < 0 || nnz < 0) {
        std::fclose(fp);
        throw std::logic_error("Something went wrong readin M, K, nnz");
    }
    a.row_offsets.resize(a.M + 1);
    a.col_indices.resize(nnz);
    for (int i = 0; i < a.M + 1; i++)
        if (std::fscanf(fp, "%d", &a.row_offsets[i]) != 1) {
            std::fclose(fp);
            throw std::logic_error("Something went wrong reading row_offsets");
        }
    for (int i = 0; i < nnz; i++)
        if (std::fscanf(fp, "%d", &a.col_indices[i]) != 1) {
            std::fclose(fp);
            throw std::logic_error("Something went wrong reading column_indices");
        }
    std::fclose(fp);
    sanity_check(a.M, a.K, nnz, a.row_offsets.data(), a.col_indices.data());
    return a;
}

// ---- device buffers ---------------------------------------------------------------------------------------------
template <typename T> struct DevBuf {
    T* p = nullptr;
    size_t n = 0;
    DevBuf() = default;
    explicit DevBuf(size_t count) : n(count) { DLSPM_HIP_CHECK(hipMalloc(reinterpret_cast<void**>(&p), std::max<size_t>(count, 1) * sizeof(T))); }
    explicit DevBuf(const std::vector<T>& h) : DevBuf(h.size())
    {
        if (n) DLSPM_HIP_CHECK(hipMemcpy(p, h.data(), n * sizeof(T), hipMemcpyHostToDevice));
    }
    DevBuf(const DevBuf&) = delete;
    DevBuf& operator=(const DevBuf&) = delete;
    DevBuf(DevBuf&& o) noexcept : p(o.p), n(o.n) { o.p = nullptr; o.n = 0; }
    DevBuf& operator=(DevBuf&& o) noexcept
    {
        if (this != &o) { if (p) (void)hipFree(p); p = o.p; n = o.n; o.p = nullptr; o.n = 0; }
        return *this;
    }
    ~DevBuf() { if (p) (void)hipFree(p); }
    std::vector<T> to_host() const
    {
        std::vector<T> h(n);
        if (n) DLSPM_HIP_CHECK(hipMemcpy(h.data(), p, n * sizeof(T), hipMemcpyDeviceToHost));
        return h;
    }
};

// ---- check kernels: one output element per thread, straight from the definition ------------------------------------
__global__ void check_spmm_kernel(int M, int N, const int* ro, const int* ci, const float* va, const float* B, float* C)
{
    const long long t = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= (long long)M * N) return;
    const int i = (int)(t / N), j = (int)(t % N);
    float acc = 0.0f;
    for (int l = ro[i]; l < ro[i + 1]; ++l) acc += va[l] * B[(size_t)ci[l] * N + j];
    C[t] = acc;
}
__global__ void check_row_of_slot_kernel(int M, const int* ro, int* row_of)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= M) return;
    for (int l = ro[i]; l < ro[i + 1]; ++l) row_of[l] = i;
}
__global__ void check_sddmm_kernel(int nnz, int D, const int* row_of, const int* ci, const float* lhs, const float* rhs,
                                   float scale, float* out)
{
    const int j = blockIdx.x * blockDim.x + threadIdx.x;
    if (j >= nnz) return;
    const float* a = lhs + (size_t)row_of[j] * D;
    const float* b = rhs + (size_t)ci[j] * D;
    double acc = 0.0;
    for (int l = 0; l < D; ++l) acc += (double)a[l] * (double)b[l];
    float s = (float)acc;
    if (scale != 1.0f) s = s * scale;
    out[j] = s;
}
__global__ void check_spmm_f64acc_kernel(int M, int N, const int* ro, const int* ci, const float* va, const float* B, float* C)
{
    const long long t = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= (long long)M * N) return;
    const int i = (int)(t / N), j = (int)(t % N);
    double acc = 0.0;
    for (int l = ro[i]; l < ro[i + 1]; ++l) acc += (double)va[l] * (double)B[(size_t)ci[l] * N + j];
    C[t] = (float)acc;
}

inline unsigned blocks_for(long long n) { return (unsigned)std::max<long long>(1, (n + 255) / 256); }

// ---- comparison of two device-resident results, on the host ---------------------------------------------------------
struct Diff {
    double checksum_ref = 0, checksum_gpu = 0;  // mean of squares, as the reference prints
    double max_diff = 0, max_rel_diff = 0, rel_frobenius = 0;
    size_t maxi = 0;
    float ref_at_max = 0, gpu_at_max = 0;
};
inline Diff compare(const std::vector<float>& ref, const std::vector<float>& gpu)
{
    Diff d;
    double num = 0, den = 0;
    for (size_t i = 0; i < ref.size(); ++i) {
        d.checksum_ref += (double)ref[i] * ref[i];
        d.checksum_gpu += (double)gpu[i] * gpu[i];
        const double diff = std::fabs((double)ref[i] - (double)gpu[i]);
        const double mag = std::max(std::fabs((double)ref[i]), std::fabs((double)gpu[i]));
        if (mag > 0) d.max_rel_diff = std::max(d.max_rel_diff, diff / mag);
        if (diff > d.max_diff || !(diff == diff)) {
            d.max_diff = diff;
            d.maxi = i;
        }
        num += diff * diff;
        den += (double)ref[i] * ref[i];
    }
    if (!ref.empty()) {
        d.checksum_ref /= ref.size();
        d.checksum_gpu /= ref.size();
        d.ref_at_max = ref[d.maxi];
        d.gpu_at_max = gpu[d.maxi];
    }
    d.rel_frobenius = den > 0 ? std::sqrt(num / den) : (num > 0 ? INFINITY : 0.0);
    return d;
}

// ---- timing ----------------------------------------------------------------------------------------------------------
struct Timing {
    double min_ms = 0, median_ms = 0;
    double cold_min_ms = -1;  // with the caches flushed before every launch; -1 when not measured
    double graph_ms = -1;     // per launch inside a HIP graph of Options::graph launches (median replay); -1 when not measured
};
struct Options {
    int warmup = 5;
    int iters = 20;  // the reference keeps the minimum of 20 launches (SPMM/spmm-esimd-fromfile2.cpp:194-243)
    bool cold = false;
    int graph = 0;  // --graph n: also time a HIP graph of n launches, replayed five times (no event between the launches)
    // what to pass as `workspace`: by default what dlspm_advise says after one look at the matrix (dlspm_analyze);
    // --workspace: always the schedule memory of dlspm_workspace_bytes, --no-workspace: always NULL
    enum Workspace { kAuto, kAlways, kNever } workspace = kAuto;
    bool plan = true;  // build a row plan or a cut plan where dlspm_advise says so (--no-plan: never)
    std::string csv, dump;
    std::string dump_each;  // --dump-each DIR: every case dumps into its own sub-directory DIR/case_000, DIR/case_001, ...
    double tol = 1e-4;  // relative Frobenius error allowed between the kernel and the check kernel
};

// What this run passes as (workspace, workspace_bytes): one look at the matrix (dlspm_analyze, once per matrix structure)
// and the library's answer for the op and the width (dlspm_advise) -- nothing, a hint, schedule memory, a row plan or a
// cut plan -- allocated and, for the plans, built on the device here, with the time that took.
struct PreparedCall {
    DevBuf<char> memory{0};
    size_t hints = 0;
    int build = DLSPM_BUILD_NOTHING;
    void* arg() const { return memory.n ? memory.p : nullptr; }
    size_t size() const { return memory.n | hints; }
};
inline PreparedCall prepare_call(const Options& opt, int op, int M, int K, int width, int nnz, const int* row_offsets_dev,
                                 const int* col_indices_dev)
{
    PreparedCall pc;
    if (opt.workspace == Options::kNever || M <= 0 || nnz <= 0) return pc;
    dlspm_matrix_info mi;
    if (dlspm_analyze(M, K, nnz, row_offsets_dev, col_indices_dev, nullptr, &mi) != DLSPM_OK) throw std::runtime_error("dlspm_analyze failed");
    dlspm_call_plan cp{DLSPM_BUILD_NOTHING, 0, 0};
    if (opt.workspace == Options::kAlways) {
        cp.bytes = dlspm_workspace_bytes(op, M, K, width, nnz);
    } else {
        if (dlspm_advise(op, width, &mi, &cp) != DLSPM_OK) throw std::runtime_error("dlspm_advise failed");
        if (!opt.plan && cp.build != DLSPM_BUILD_NOTHING) {  // --no-plan: what the advice says without plans
            const int passing = dlspm_workspace_advice(op, M, K, width, nnz, mi.max_row_len);
            cp = dlspm_call_plan{DLSPM_BUILD_NOTHING, passing == DLSPM_PASS_WORKSPACE ? dlspm_workspace_bytes(op, M, K, width, nnz) : 0,
                                 passing == DLSPM_PASS_ROWS_EVEN ? DLSPM_HINT_ROWS_EVEN : 0};
        }
    }
    int slices = 0;
    (void)dlspm_describe_slices(op, M, K, width, nnz, &slices, nullptr);
    std::printf("rows: longest %d, mean %.1f, empty %d; columns: widest row %d, eighths span %.2f x K -> %s%s%s\n", mi.max_row_len,
                (double)nnz / M, mi.empty_rows, mi.max_col_span, mi.eighths_cover_permille * 1e-3,
                opt.workspace == Options::kAlways           ? "workspace passed (--workspace)"
                : cp.build == DLSPM_BUILD_CUT_PLAN          ? "a row above one and a half shares, cut plan (long rows handed out in pieces)"
                : cp.build == DLSPM_BUILD_ROW_PLAN          ? "uneven, row plan (one row per workgroup, handed out by length)"
                : (cp.hints & DLSPM_HINT_BANDED)            ? "banded, DLSPM_HINT_BANDED passed"
                : cp.bytes && slices > 0                    ? "dense operands beyond one L2, workspace passed (column-sliced schedule)"
                : cp.bytes                                  ? "uneven, workspace passed (flat schedule)"
                : (cp.hints & DLSPM_HINT_ROWS_EVEN)         ? "even, DLSPM_HINT_ROWS_EVEN passed"
                : (cp.hints & DLSPM_HINT_ROWS_SKEWED)       ? "long rows next to each other, fewer rows per workgroup"
                                                            : "nothing passed",
                (cp.hints & DLSPM_HINT_BANDED) && (cp.hints & DLSPM_HINT_ROWS_EVEN) ? " with DLSPM_HINT_ROWS_EVEN" : "",
                (cp.hints & DLSPM_HINT_ROWS_SKEWED) ? " with DLSPM_HINT_ROWS_SKEWED" : "");
    pc.memory = DevBuf<char>(cp.bytes);
    pc.hints = cp.hints;
    pc.build = cp.build;
    if (cp.bytes && cp.build == DLSPM_BUILD_NOTHING) std::printf("workspace: %zu bytes\n", cp.bytes);
    if (cp.build != DLSPM_BUILD_NOTHING) {
        // what the plan costs on the device: HIP events around the second of two builds (the first pays for loading the kernels)
        hipEvent_t e0, e1;
        DLSPM_HIP_CHECK(hipEventCreate(&e0));
        DLSPM_HIP_CHECK(hipEventCreate(&e1));
        float ms = 0;
        for (int rep = 0; rep < 2; ++rep) {
            DLSPM_HIP_CHECK(hipEventRecord(e0, nullptr));
            const int st = cp.build == DLSPM_BUILD_CUT_PLAN ? dlspm_row_plan_build_cut(M, row_offsets_dev, pc.memory.p, pc.memory.n, nullptr)
                                                            : dlspm_row_plan_build(M, row_offsets_dev, pc.memory.p, pc.memory.n, nullptr);
            if (st != DLSPM_OK) throw std::runtime_error("building the row plan failed");
            DLSPM_HIP_CHECK(hipEventRecord(e1, nullptr));
            DLSPM_HIP_CHECK(hipEventSynchronize(e1));
            DLSPM_HIP_CHECK(hipEventElapsedTime(&ms, e0, e1));
        }
        (void)hipEventDestroy(e0);
        (void)hipEventDestroy(e1);
        std::printf("%s: %zu bytes, built on the device in %.1f us (once per matrix)\n",
                    cp.build == DLSPM_BUILD_CUT_PLAN ? "cut plan" : "row plan", pc.memory.n, ms * 1e3);
    }
    return pc;
}

// `launch(stream)` enqueues one call of the op. Every launch is timed between its own pair of HIP events (the minimum is
// the reference's figure; the pair itself costs about 3 us that a sequence of launches does not pay); with --graph n the
// same launch is also captured n times into a HIP graph, whose replay is timed as a whole.
template <typename Launch> Timing time_launches(const Options& opt, Launch&& launch)
{
    hipEvent_t e0, e1;
    DLSPM_HIP_CHECK(hipEventCreate(&e0));
    DLSPM_HIP_CHECK(hipEventCreate(&e1));
    auto check = [](int st) {
        if (st != DLSPM_OK) throw std::runtime_error(std::string("libdlspm_hip: ") + dlspm_status_string(st));
    };
    auto one = [&]() {
        DLSPM_HIP_CHECK(hipEventRecord(e0, nullptr));
        const int st = launch(static_cast<hipStream_t>(nullptr));
        DLSPM_HIP_CHECK(hipEventRecord(e1, nullptr));
        DLSPM_HIP_CHECK(hipEventSynchronize(e1));
        check(st);
        float ms = 0;
        DLSPM_HIP_CHECK(hipEventElapsedTime(&ms, e0, e1));
        return (double)ms;
    };
    for (int i = 0; i < opt.warmup; ++i) one();
    std::vector<double> t;
    for (int i = 0; i < opt.iters; ++i) t.push_back(one());
    std::sort(t.begin(), t.end());
    Timing r;
    r.min_ms = t.front();
    r.median_ms = t[t.size() / 2];
    if (opt.cold) {  // the idea of SDDMM/tprint.cpp:256-265: stream a large buffer through the caches before each launch
        const size_t flush_bytes = size_t(1) << 30;
        DevBuf<char> flush(flush_bytes);
        double best = 1e30;
        for (int i = 0; i < std::max(3, opt.iters / 4); ++i) {
            DLSPM_HIP_CHECK(hipMemsetAsync(flush.p, i, flush_bytes, nullptr));
            best = std::min(best, one());
        }
        r.cold_min_ms = best;
    }
    if (opt.graph > 0) {
        constexpr int kReplays = 5;
        hipStream_t stream;
        hipGraph_t graph;
        hipGraphExec_t exec;
        DLSPM_HIP_CHECK(hipDeviceSynchronize());
        DLSPM_HIP_CHECK(hipStreamCreate(&stream));
        DLSPM_HIP_CHECK(hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal));
        int st = DLSPM_OK;
        for (int i = 0; i < opt.graph && st == DLSPM_OK; ++i) st = launch(stream);
        DLSPM_HIP_CHECK(hipStreamEndCapture(stream, &graph));
        check(st);
        DLSPM_HIP_CHECK(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0));
        DLSPM_HIP_CHECK(hipGraphLaunch(exec, stream));  // untimed: first-use set-up of the graph
        DLSPM_HIP_CHECK(hipStreamSynchronize(stream));
        hipEvent_t begin[kReplays], end[kReplays];
        for (int i = 0; i < kReplays; ++i) {
            DLSPM_HIP_CHECK(hipEventCreate(&begin[i]));
            DLSPM_HIP_CHECK(hipEventCreate(&end[i]));
        }
        for (int i = 0; i < kReplays; ++i) {  // enqueued back to back: a replay starts on a device that is at work
            DLSPM_HIP_CHECK(hipEventRecord(begin[i], stream));
            DLSPM_HIP_CHECK(hipGraphLaunch(exec, stream));
            DLSPM_HIP_CHECK(hipEventRecord(end[i], stream));
        }
        DLSPM_HIP_CHECK(hipStreamSynchronize(stream));
        std::vector<double> replay;
        for (int i = 0; i < kReplays; ++i) {
            float ms = 0;
            DLSPM_HIP_CHECK(hipEventElapsedTime(&ms, begin[i], end[i]));
            replay.push_back((double)ms / opt.graph);
            (void)hipEventDestroy(begin[i]);
            (void)hipEventDestroy(end[i]);
        }
        std::sort(replay.begin(), replay.end());
        r.graph_ms = replay[kReplays / 2];
        (void)hipGraphExecDestroy(exec);
        (void)hipGraphDestroy(graph);
        (void)hipStreamDestroy(stream);
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    return r;
}

// ---- report ------------------------------------------------------------------------------------------------------------
inline void dump_array(const std::string& dir, const char* name, const void* data, size_t bytes)
{
    std::ofstream f(dir + "/" + name, std::ios::binary);
    if (!f) throw std::logic_error("cannot write to dump directory " + dir);
    f.write(static_cast<const char*>(data), (std::streamsize)bytes);
}

inline void report(const char* opname, Op op, int M, int K, int N, int nnz, const Timing& t, const Diff& d, bool csr_intact,
                   const Options& opt)
{
    const Accounting a = account(op, M, K, N, nnz);
    const double s = t.min_ms * 1e-3;
    const double density = (M > 0 && K > 0) ? (double)nnz / ((double)M * K) : 0.0;
    std::printf("MSZ = %d KSZ = %d NSZ = %d SP = %f nnz = %d\n", M, K, N, density, nnz);
    std::printf("Total kernel time was %f ms.\n", t.min_ms);
    std::printf("GFLOPS:  %8.2f\n", a.flops / s * 1e-9);
    std::printf("median kernel time %f ms over %d launches (%d warm-up)\n", t.median_ms, opt.iters, opt.warmup);
    if (t.cold_min_ms >= 0) std::printf("cold-cache kernel time %f ms (1 GiB streamed through the caches before each launch)\n", t.cold_min_ms);
    if (t.graph_ms >= 0)
        std::printf("in a HIP graph of %d launches: %f ms per launch, GFLOPS: %8.2f (median of 5 replays)\n", opt.graph, t.graph_ms,
                    a.flops / (t.graph_ms * 1e-3) * 1e-9);
    std::printf("effective (application) bandwidth: %9.1f GB/s = %5.1f %% of 8000 GB/s HBM peak  [%.0f bytes]\n",
                a.effective_B / s * 1e-9, a.effective_B / s * 1e-9 / 80.0, a.effective_B);
    std::printf("algorithmic bandwidth:             %9.1f GB/s = %5.2f %% of 8000 GB/s HBM peak  [%.0f bytes]\n",
                a.algorithmic_B / s * 1e-9, a.algorithmic_B / s * 1e-9 / 80.0, a.algorithmic_B);
    std::cout.precision(7);
    std::cout << "checksum_ref = " << d.checksum_ref << std::endl;
    std::cout << "checksum_gpu = " << d.checksum_gpu << std::endl;
    std::cout << "maxi = " << d.maxi << " max_diff = " << d.max_diff << " max_rel_diff = " << d.max_rel_diff
              << " rel_frobenius = " << d.rel_frobenius << std::endl;
    std::cout << "output_ref[" << d.maxi << "] = " << d.ref_at_max << std::endl;
    std::cout << "output_gpu[" << d.maxi << "] = " << d.gpu_at_max << std::endl;
    std::cout << "csr structure after the call: " << (csr_intact ? "bit-identical" : "MODIFIED") << std::endl;
    const bool ok = csr_intact && d.rel_frobenius <= opt.tol;
    std::cout << opname << (ok ? " PASS" : " FAIL") << std::endl << "*********************************" << std::endl << std::endl;
}

// ---- command line -----------------------------------------------------------------------------------------------------------
struct CaseSpec {
    enum Kind { kCfg, kShape, kFile } kind = kCfg;
    int cfg = 0;
    int M = 0, K = 0, N = 0;
    double density = 0;
    double sigma = 0;  // > 0: row lengths lognormal around density*K with this sigma (skewed rows) instead of Bernoulli
    int band = 0;      // > 0: every row holds a band of this many columns around its diagonal position, plus
    int band_random = 0;  // ... this many columns anywhere (density is ignored): the pattern of sparse attention masks
    uint64_t seed = 1;
    std::string file;
};

// pattern of a --shape case
inline Csr synthetic_pattern(const CaseSpec& s)
{
    if (s.band > 0) return pattern_band_plus_random(s.seed, s.M, s.K, s.band, s.band_random);
    return s.sigma > 0 ? pattern_lognormal_rows(s.seed, s.M, s.K, s.density * s.K, s.sigma)
                       : pattern_bernoulli(s.seed, s.M, s.K, s.density);
}

// the grid of SPMM/spmm-esimd-allbenchs2.cpp:252-255 (same in SDDMM/sddmm-esimd-allbench_v4.cpp:241-244)
inline std::vector<CaseSpec> sputnik_grid(int max_m)
{
    const int Ms[] = {1024, 3072, 4096, 2048, 6144, 8192, 4096, 12288, 16384, 8192, 24576, 32768};
    const int Ks[] = {1024, 1024, 1024, 2048, 2048, 2048, 4096, 4096, 4096, 8192, 8192, 8192};
    const int Ns[] = {32, 128};
    const double SPs[] = {0.3, 0.2, 0.1};
    std::vector<CaseSpec> v;
    for (int N : Ns)
        for (int c = 0; c < 12; ++c)
            for (double sp : SPs) {
                if (Ms[c] > max_m) continue;
                CaseSpec s;
                s.kind = CaseSpec::kShape; s.M = Ms[c]; s.K = Ks[c]; s.N = N; s.density = sp;
                s.seed = 7000 + (uint64_t)v.size();
                v.push_back(s);
            }
    return v;
}

struct Cli {
    Options opt;
    std::vector<CaseSpec> cases;
};

// usage text shared by the three drivers; `app` is the program name, `width` what N means for it
inline std::string usage(const char* app, const char* width)
{
    std::ostringstream u;
    u << "Usage: " << app << " <filename>.smtx <" << width << ">            one matrix from a DLMC .smtx file\n"
      << "       " << app << " --batch <list>                      lines '<filename>.smtx <" << width << ">', '#' comments\n"
      << "       " << app << " --shape M K " << width << " density [--seed S] [--sigma s]   one synthetic matrix (Bernoulli pattern;\n"
      << "                                                     --sigma: lognormal row lengths, skewed;\n"
      << "                                                     --band w [--band-random r]: a band of w columns per row plus r anywhere)\n"
      << "       " << app << " --sweep [--max-m M]                  the 12 x {32,128} x {0.3,0.2,0.1} benchmark grid\n"
      << "       " << app << " --cfg <id>                           a seeded benchmark configuration (1..5)\n"
      << "options: --iters n (20)  --warmup n (5)  --cold  --graph n  --csv <file>  --dump <dir> | --dump-each <dir>  --tol x (1e-4)  --workspace | --no-workspace  --no-plan";
    return u.str();
}

inline Cli parse_cli(int argc, char** argv, const char* app, const char* width)
{
    Cli cli;
    std::vector<std::string> pos;
    int max_m = 1 << 30;
    bool sweep = false;
    auto need = [&](int& i, int n) {
        if (i + n >= argc) throw std::invalid_argument(usage(app, width));
    };
    for (int i = 1; i < argc; ++i) {
        const std::string a = argv[i];
        if (a == "--cfg") { need(i, 1); CaseSpec s; s.kind = CaseSpec::kCfg; s.cfg = std::stoi(argv[++i]); cli.cases.push_back(s); }
        else if (a == "--shape") {
            need(i, 4);
            CaseSpec s; s.kind = CaseSpec::kShape;
            s.M = std::stoi(argv[i + 1]); s.K = std::stoi(argv[i + 2]); s.N = std::stoi(argv[i + 3]); s.density = std::stod(argv[i + 4]);
            i += 4;
            cli.cases.push_back(s);
        }
        else if (a == "--seed") { need(i, 1); const uint64_t sd = std::stoull(argv[++i]); if (!cli.cases.empty()) cli.cases.back().seed = sd; }
        else if (a == "--sigma") { need(i, 1); const double sg = std::stod(argv[++i]); if (!cli.cases.empty()) cli.cases.back().sigma = sg; }
        else if (a == "--band") { need(i, 1); const int b = std::stoi(argv[++i]); if (!cli.cases.empty()) cli.cases.back().band = b; }
        else if (a == "--band-random") { need(i, 1); const int b = std::stoi(argv[++i]); if (!cli.cases.empty()) cli.cases.back().band_random = b; }
        else if (a == "--no-workspace") cli.opt.workspace = Options::kNever;
        else if (a == "--workspace") cli.opt.workspace = Options::kAlways;
        else if (a == "--no-plan") cli.opt.plan = false;
        else if (a == "--sweep") sweep = true;
        else if (a == "--max-m") { need(i, 1); max_m = std::stoi(argv[++i]); }
        else if (a == "--batch") {
            need(i, 1);
            std::ifstream f(argv[++i]);
            if (!f) throw std::logic_error("Error opening file!");
            std::string line;
            while (std::getline(f, line)) {
                if (line.empty() || line[0] == '#') continue;
                std::istringstream ls(line);
                CaseSpec s; s.kind = CaseSpec::kFile;
                if (!(ls >> s.file >> s.N)) throw std::logic_error("bad line in batch list: " + line);
                cli.cases.push_back(s);
            }
        }
        else if (a == "--iters") { need(i, 1); cli.opt.iters = std::max(1, std::stoi(argv[++i])); }
        else if (a == "--warmup") { need(i, 1); cli.opt.warmup = std::max(0, std::stoi(argv[++i])); }
        else if (a == "--graph") { need(i, 1); cli.opt.graph = std::max(0, std::stoi(argv[++i])); }
        else if (a == "--cold") cli.opt.cold = true;
        else if (a == "--csv") { need(i, 1); cli.opt.csv = argv[++i]; }
        else if (a == "--dump") { need(i, 1); cli.opt.dump = argv[++i]; }
        else if (a == "--dump-each") { need(i, 1); cli.opt.dump_each = argv[++i]; }
        else if (a == "--tol") { need(i, 1); cli.opt.tol = std::stod(argv[++i]); }
        else if (a.rfind("--", 0) == 0) throw std::invalid_argument(usage(app, width));
        else pos.push_back(a);
    }
    if (sweep) for (const auto& s : sputnik_grid(max_m)) cli.cases.push_back(s);
    if (!pos.empty()) {
        if (pos.size() != 2) throw std::invalid_argument(usage(app, width));  // the reference's `argc != 3`
        CaseSpec s; s.kind = CaseSpec::kFile; s.file = pos[0]; s.N = std::stoi(pos[1]);
        cli.cases.push_back(s);
    }
    if (cli.cases.empty()) throw std::invalid_argument(usage(app, width));
    return cli;
}

// Options of case number `index` of a run: with --dump-each every case dumps into a sub-directory of its own (created
// here), so that a sweep or a batch can be verified case by case from outside.
inline Options case_options(const Options& opt, size_t index)
{
    if (opt.dump_each.empty()) return opt;
    Options o = opt;
    char name[32];
    std::snprintf(name, sizeof name, "case_%03zu", index);
    o.dump = opt.dump_each + "/" + name;
    std::filesystem::create_directories(o.dump);
    return o;
}

inline void print_device()
{
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) {
        std::cout << "Running on: no HIP device visible, " << dlspm_version() << std::endl;
        return;
    }
    std::cout << "Running on " << prop.name << " (" << prop.gcnArchName << ", " << prop.multiProcessorCount << " CUs), "
              << dlspm_version() << std::endl;
}

}  // namespace dlspm
