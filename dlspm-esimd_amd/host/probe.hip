// libdlspm_probe.so: two measurement kernels for bench.py, behind a C ABI. Not part of libdlspm_hip and not used by it.
//   gather  what the device delivers for the access pattern the sparse kernels are made of -- whole waves fetching
//           1 KiB dense rows at random (or consecutive) positions of a table -- so that kernel times can be judged
//           against a measured ceiling instead of the HBM figure, which these cache-resident problems never touch.
//           Each wave issues 8 row loads before it consumes them, `iters` times: with 1024 workgroups of four waves and
//           iters = 32 one launch gathers 1.07 GB. rows_mask + 1 = rows of the table (a power of two): 512 rows = 512 KiB
//           fit every XCD's L2 (B of the 2048 x 512 x 256 benchmark), 8192 rows = 8 MiB do not.
//   copy    a plain float4 copy of known size: the kernel whose rocprofv3 FETCH_SIZE / WRITE_SIZE readings scale the
//           counters of the other kernels.
// The reference's nearest relative is the cache-flush copy kernel of SDDMM/tprint.cpp:65-72.
#include <hip/hip_runtime.h>
#include <stddef.h>

namespace {

template <bool RANDOM>
__global__ __launch_bounds__(256) void dlspm_probe_gather_kernel(const float* __restrict__ table, float* out, int iters,
                                                                 unsigned rows_mask)
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
        for (int u = 0; u < 8; ++u) {
            acc.x += v[u].x;
            acc.y += v[u].y;
            acc.z += v[u].z;
            acc.w += v[u].w;
        }
    }
    if (acc.x + acc.y + acc.z + acc.w == 12345.678f) out[0] = acc.x;  // keeps the loads alive, never true for this data
}

__global__ __launch_bounds__(256) void dlspm_probe_copy_kernel(const float4* __restrict__ src, float4* __restrict__ dst, size_t n4)
{
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += stride) dst[i] = src[i];
}

}  // namespace

extern "C" {

// One launch: `blocks` workgroups of four waves, every wave gathers iters x 8 rows of 256 floats from `table`
// ((rows_mask + 1) x 256 floats on the device). Returns the hipError_t of the launch as int (0 = ok).
int dlspm_probe_gather(const float* table, unsigned rows_mask, int iters, int random, int blocks, float* sink, void* stream)
{
    if (!table || !sink || iters < 0 || blocks < 1 || (rows_mask & (rows_mask + 1)) != 0) return (int)hipErrorInvalidValue;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (random) hipLaunchKernelGGL(dlspm_probe_gather_kernel<true>, dim3(blocks), dim3(256), 0, st, table, sink, iters, rows_mask);
    else hipLaunchKernelGGL(dlspm_probe_gather_kernel<false>, dim3(blocks), dim3(256), 0, st, table, sink, iters, rows_mask);
    return (int)hipGetLastError();
}

// dst[0 .. n) = src[0 .. n), n a multiple of 4, both 16-byte aligned: reads 4 n bytes, writes 4 n bytes.
int dlspm_probe_copy(const float* src, float* dst, size_t n, void* stream)
{
    if (!src || !dst || n % 4 != 0) return (int)hipErrorInvalidValue;
    hipLaunchKernelGGL(dlspm_probe_copy_kernel, dim3(4096), dim3(256), 0, static_cast<hipStream_t>(stream),
                       reinterpret_cast<const float4*>(src), reinterpret_cast<float4*>(dst), n / 4);
    return (int)hipGetLastError();
}

}  // extern "C"
