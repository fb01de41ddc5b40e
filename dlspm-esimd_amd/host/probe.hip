// libdlspm_probe.so: measurement legs of bench.py, behind a C ABI. Not part of libdlspm_hip and not used by it.
//   gather  what the device delivers for the access pattern the sparse kernels are made of -- whole waves fetching
//           1 KiB dense rows at random (or consecutive) positions of a table -- so that kernel times can be judged
//           against a measured ceiling instead of the HBM figure, which these cache-resident problems never touch.
//           Each wave issues 8 row loads before it consumes them, `iters` times: with 1024 workgroups of four waves and
//           iters = 32 one launch gathers 1.07 GB. rows_mask + 1 = rows of the table (a power of two): 512 rows = 512 KiB
//           fit every XCD's L2 (B of the 2048 x 512 x 256 benchmark), 8192 rows = 8 MiB do not.
//   copy    a plain float4 copy of known size: the kernel whose rocprofv3 FETCH_SIZE / WRITE_SIZE readings scale the
//           counters of the other kernels.
//   enqueue what a call of one of the three entry points costs the HOST when it is issued outside a graph, the way the
//           reference times its kernels (20 single launches, SPMM/spmm-esimd-fromfile2.cpp:194-243): n calls through
//           the function pointer, no synchronisation in between, wall time / n; and the same loop over an empty
//           kernel, which is what the HIP runtime's launch alone costs.
//   floor   what a launch costs the DEVICE before any arithmetic: an empty kernel of a given grid, and a kernel that only
//           walks the dependent loads every row-block kernel starts with (two row offsets -> 64 column indices -> one
//           1 KiB dense row -> one store). Timed by bench.py between the nodes of a HIP graph, like the ops themselves.
// The reference's nearest relative is the cache-flush copy kernel of SDDMM/tprint.cpp:65-72.
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <chrono>

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

__global__ void dlspm_probe_empty_kernel(int) {}

// depth 0: the row offsets only; 1: + 64 column indices per wave; 2: + the dense row of the first of them; 3: + the store
__global__ __launch_bounds__(256) void dlspm_probe_chain_kernel(int M, const int* __restrict__ ro, const int* __restrict__ ci,
                                                                const float* __restrict__ B, float* __restrict__ C, int depth)
{
    const int row = blockIdx.x % M, lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int rs = ro[row], re = ro[row + 1];
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    if (depth >= 1 && re > rs) {
        const int c = ci[min(rs + lane + 64 * w, re - 1)];
        if (depth >= 2) {
            const int first = __builtin_amdgcn_readfirstlane(c);
            acc = *reinterpret_cast<const float4*>(B + (size_t)first * 256 + lane * 4);
        } else {
            acc.x = (float)c;
        }
    }
    if ((depth >= 3 || acc.x == 12345.678f) && w == 0) *reinterpret_cast<float4*>(C + (size_t)row * 256 + lane * 4) = acc;
}

template <typename F> double per_call_us(int n, F&& call)
{
    const auto t0 = std::chrono::steady_clock::now();
    for (int i = 0; i < n; ++i) call();
    const auto t1 = std::chrono::steady_clock::now();
    return std::chrono::duration<double, std::micro>(t1 - t0).count() / (n > 0 ? n : 1);
}

}  // namespace

extern "C" {

typedef int (*dlspm_probe_spmm_fn)(int, int, int, int, const int*, const int*, const float*, const float*, float*, void*,
                                   size_t, void*);
typedef int (*dlspm_probe_sddmm_fn)(int, int, int, int, const int*, const int*, const float*, const float*, float*, void*,
                                    size_t, void*);
typedef int (*dlspm_probe_fused_fn)(int, int, int, int, const int*, const int*, const float*, const float*, const float*,
                                    float, float*, void*, size_t, void*);

// Host microseconds per call of n calls of `fn` (spmm_csr_f32 or an entry point of its signature) issued back to back on
// `stream` without synchronising; *status receives the last call's status. The caller synchronises afterwards.
double dlspm_probe_enqueue_spmm(void* fn, int n, int M, int K, int N, int nnz, const int* ro, const int* ci, const float* va,
                                const float* B, float* C, void* ws, size_t ws_bytes, void* stream, int* status)
{
    int st = 0;
    const double us = per_call_us(n, [&] { st = ((dlspm_probe_spmm_fn)fn)(M, K, N, nnz, ro, ci, va, B, C, ws, ws_bytes, stream); });
    if (status) *status = st;
    return us;
}
double dlspm_probe_enqueue_sddmm(void* fn, int n, int M, int K, int D, int nnz, const int* ro, const int* ci, const float* lhs,
                                 const float* rhs, float* out, void* ws, size_t ws_bytes, void* stream, int* status)
{
    int st = 0;
    const double us = per_call_us(n, [&] { st = ((dlspm_probe_sddmm_fn)fn)(M, K, D, nnz, ro, ci, lhs, rhs, out, ws, ws_bytes, stream); });
    if (status) *status = st;
    return us;
}
double dlspm_probe_enqueue_fused(void* fn, int n, int M, int K, int D, int nnz, const int* ro, const int* ci, const float* Q,
                                 const float* Km, const float* V, float scale, float* O, void* ws, size_t ws_bytes, void* stream,
                                 int* status)
{
    int st = 0;
    const double us = per_call_us(n, [&] { st = ((dlspm_probe_fused_fn)fn)(M, K, D, nnz, ro, ci, Q, Km, V, scale, O, ws, ws_bytes, stream); });
    if (status) *status = st;
    return us;
}
// the same loop over an empty kernel: the launch cost of the runtime by itself
double dlspm_probe_enqueue_empty(int n, void* stream)
{
    return per_call_us(n, [&] { hipLaunchKernelGGL(dlspm_probe_empty_kernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream), 0); });
}

// One launch of the floor kernels. depth < 0: the empty kernel with `workgroups` x `threads`; depth 0 ... 3: the chain kernel
// (256 threads) over a CSR matrix of M rows whose column indices are < the rows of B (B and C have 256 floats per row, C has M rows).
int dlspm_probe_floor(int workgroups, int threads, int depth, int M, const int* ro, const int* ci, const float* B, float* C,
                      void* stream)
{
    if (workgroups < 1 || depth > 3) return (int)hipErrorInvalidValue;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (depth < 0) {
        if (threads < 1 || threads > 1024) return (int)hipErrorInvalidValue;
        hipLaunchKernelGGL(dlspm_probe_empty_kernel, dim3(workgroups), dim3(threads), 0, st, 0);
    } else {
        if (M < 1 || !ro || !ci || !B || !C) return (int)hipErrorInvalidValue;
        hipLaunchKernelGGL(dlspm_probe_chain_kernel, dim3(workgroups), dim3(256), 0, st, M, ro, ci, B, C, depth);
    }
    return (int)hipGetLastError();
}

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
