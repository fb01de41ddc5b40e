// gather_probe: measures what the device can deliver for the access pattern the sparse kernels are made of --
// whole waves fetching 1 KiB dense rows at random positions of a table -- so that kernel times can be judged against
// a measured ceiling instead of the HBM number, which these cache-resident problems never touch.
//   sequential rows  : every wave walks consecutive 1 KiB rows (pure streaming from L2)
//   random rows      : every wave-load picks a pseudo-random row of the table (what SpMM does with B)
// Table sizes: 32 KiB (fits a CU's L1), 512 KiB (B of the 2048x512x256 benchmark; fits every XCD's L2),
// 8 MiB (exceeds an XCD's L2). Each wave issues 8 loads before it consumes them; 4096 waves x 32 rounds = 1.07 GB per
// launch, long enough that the launch itself (about 2 us) does not matter. Prints TB/s over the whole device and bytes
// per clock per CU at the reported engine clock.
#include "driver.hpp"

using namespace dlspm;

template <bool RANDOM>
__global__ __launch_bounds__(256) void probe_kernel(const float* __restrict__ table, float* out, int iters, unsigned rows_mask)
{
    const int lane = threadIdx.x & 63;
    const unsigned wave = blockIdx.x * 4 + (threadIdx.x >> 6);
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    unsigned h = wave * 2654435761u + 12345u;
    for (int it = 0; it < iters; ++it) {
        float4 v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            unsigned row;
            if (RANDOM) {
                h = h * 1664525u + 1013904223u;
                row = (h >> 8) & rows_mask;
            } else {
                row = (wave * iters * 8 + it * 8 + u) & rows_mask;
            }
            row = __builtin_amdgcn_readfirstlane(row);
            v[u] = *reinterpret_cast<const float4*>(table + (size_t)row * 256 + lane * 4);
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) { acc.x += v[u].x; acc.y += v[u].y; acc.z += v[u].z; acc.w += v[u].w; }
    }
    if (acc.x + acc.y + acc.z + acc.w == 12345.678f) out[0] = acc.x;  // keeps the loads alive, never true for this data
}

static double time_us(bool random, const float* table, float* out, int iters, unsigned mask)
{
    hipEvent_t e0, e1;
    DLSPM_HIP_CHECK(hipEventCreate(&e0));
    DLSPM_HIP_CHECK(hipEventCreate(&e1));
    const int reps = 200;
    auto launch = [&]() {
        if (random) hipLaunchKernelGGL(probe_kernel<true>, dim3(1024), dim3(256), 0, nullptr, table, out, iters, mask);
        else hipLaunchKernelGGL(probe_kernel<false>, dim3(1024), dim3(256), 0, nullptr, table, out, iters, mask);
    };
    for (int i = 0; i < 20; ++i) launch();
    double best = 1e30;
    for (int trial = 0; trial < 5; ++trial) {  // back-to-back launches between two events: per-launch time without event overhead
        DLSPM_HIP_CHECK(hipEventRecord(e0, nullptr));
        for (int i = 0; i < reps; ++i) launch();
        DLSPM_HIP_CHECK(hipEventRecord(e1, nullptr));
        DLSPM_HIP_CHECK(hipEventSynchronize(e1));
        float ms = 0;
        DLSPM_HIP_CHECK(hipEventElapsedTime(&ms, e0, e1));
        best = std::min(best, (double)ms * 1e3 / reps);
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    return best;
}

int main()
{
    try {
        print_device();
        int dev = 0, clock_khz = 0, cus = 0;
        DLSPM_HIP_CHECK(hipGetDevice(&dev));
        DLSPM_HIP_CHECK(hipDeviceGetAttribute(&clock_khz, hipDeviceAttributeClockRate, dev));
        DLSPM_HIP_CHECK(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
        std::vector<float> h((size_t)8192 * 256);
        fill_uniform(1, h.size(), -1.f, 1.f, h.data());
        DevBuf<float> table(h), out(4);
        const int rounds = 32;
        const double bytes = 1024.0 * 4 * rounds * 8 * 1024;  // waves x rounds x loads x 1 KiB
        std::printf("engine clock %.0f MHz, %d CUs; empty launch of the same grid: %.2f us\n", clock_khz / 1e3, cus,
                    time_us(true, table.p, out.p, 0, 511));
        struct Case { const char* name; bool random; unsigned mask; };
        const Case cases[] = {{"sequential 1 KiB rows, 512 KiB table", false, 511}, {"random 1 KiB rows,  32 KiB table (L1)", true, 31},
                              {"random 1 KiB rows, 512 KiB table (L2)", true, 511}, {"random 1 KiB rows,   8 MiB table (> one L2)", true, 8191}};
        for (const auto& c : cases) {
            const double t = time_us(c.random, table.p, out.p, rounds, c.mask);
            const double net = t * 1e-6;
            std::printf("%-46s %7.2f us per launch of %.0f MB -> %5.1f TB/s, %5.1f B/clk/CU\n", c.name, t, bytes / 1e6,
                        bytes / net / 1e12, bytes / net / cus / (clock_khz * 1e3));
        }
        return 0;
    } catch (std::exception& e) {
        std::cout << e.what() << std::endl;
        return 1;
    }
}
