// Column-sliced schedule, the two passes around the main kernel (SpMM and the fused op):
//   before: where each CSR row is cut by the slice boundaries (one lower-bound search per row and boundary);
//   after:  the output is the sum of the slices' partial rows, added in slice order.
// The reference has no counterpart: its kernels gather the rows of B by column index as they come
// (SPMM/spmmesimd2.hpp:63-147).
#include "common.hpp"
#include "launch.hpp"

namespace dlspm {

// 32 lanes per row, lane p <- first position of the row whose column is >= p * K / slices (p = 0: the row's start,
// p >= slices: its end). Columns that ascend inside a row (every generator and file format here) make these the
// exact cuts; for any other order the running maximum still makes them a partition of the row, so the result of the
// op stays right and only the locality is lost. bounds[p][row], p = 0 .. slices.
__global__ __launch_bounds__(256) void slice_bounds_kernel(int M, int K, int slices, const int* __restrict__ row_offsets,
                                                           const int* __restrict__ col_indices, int* __restrict__ bounds)
{
    const int lane = threadIdx.x & 63;
    const int p = threadIdx.x & 31;
    const int row = blockIdx.x * 8 + (threadIdx.x >> 5);
    const int r = min(row, M - 1);  // every lane stays in the exchange below
    const int rs = row_offsets[r];
    const int re = row_offsets[r + 1];
    int lb = p == 0 ? rs : re;
    if (p > 0 && p < slices) {
        const int cut = (int)((long long)p * K / slices);
        int lo = rs, hi = re;
        while (lo < hi) {
            const int mid = lo + ((hi - lo) >> 1);
            if (col_indices[mid] < cut) lo = mid + 1;
            else hi = mid;
        }
        lb = lo;
    }
#pragma unroll
    for (int d = 1; d < 32; d *= 2) {
        const int y = lane_get(lb, p >= d ? lane - d : lane);
        lb = max(lb, y);
    }
    if (row < M && p <= slices) bounds[(size_t)p * M + row] = lb;
}

hipError_t slice_bounds_launch(int M, int K, int slices, const int* row_offsets, const int* col_indices, int* bounds,
                               hipStream_t stream)
{
    if (slices < 1 || slices > 31) return hipErrorInvalidValue;
    const unsigned blocks = (unsigned)ceil_div(M, 8);
    hipLaunchKernelGGL(slice_bounds_kernel, dim3(blocks), dim3(256), 0, stream, M, K, slices, row_offsets, col_indices,
                       bounds);
    return hipGetLastError();
}

// out[i] = partial[0][i] + partial[1][i] + ... in that order (VEC floats per thread and step)
template <int VEC>
__global__ __launch_bounds__(256) void slice_sum_kernel(long long count, int slices, const float* __restrict__ partial,
                                                        float* __restrict__ out)
{
    using VecT = Vec<VEC>;
    const long long stride = (long long)gridDim.x * blockDim.x * VEC;
    for (long long i = ((long long)blockIdx.x * blockDim.x + threadIdx.x) * VEC; i < count; i += stride) {
        VecT sum = VecT::gload(partial + i);
        for (int s = 1; s < slices; ++s) sum.add(VecT::gload(partial + (size_t)s * count + i));
        sum.gstore(out + i);
    }
}

hipError_t slice_sum_launch(long long count, int slices, const float* partial, float* out, hipStream_t stream)
{
    if (count <= 0) return hipSuccess;
    const bool vec4 = count % 4 == 0;  // whole float4 steps (dwordx4 accesses need only dword alignment)
    const long long threads = vec4 ? count / 4 : count;
    const long long want = (threads + 255) / 256;
    const unsigned blocks = (unsigned)(want < (1 << 16) ? want : (1 << 16));
    if (vec4) hipLaunchKernelGGL((slice_sum_kernel<4>), dim3(blocks), dim3(256), 0, stream, count, slices, partial, out);
    else hipLaunchKernelGGL((slice_sum_kernel<1>), dim3(blocks), dim3(256), 0, stream, count, slices, partial, out);
    return hipGetLastError();
}

}  // namespace dlspm
