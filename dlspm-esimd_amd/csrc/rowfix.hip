// Second pass of the flat schedule (SpMM and the fused kernel): rows whose nonzeros were spread over several
// waves are the sum of those waves' partial rows, added here in wave order; rows without nonzeros become zeros.
#include "common.hpp"
#include "launch.hpp"

namespace dlspm {

// One wave per row. `partial[unit][k][N]`: k = 0 is the row that began before the unit's range (or exactly at its
// start and runs past its end), k = 1 the row that begins inside the range and continues after it.
template <int VEC>
__global__ __launch_bounds__(kFlatWaves * 64) void row_fixup_kernel(int M, int N, int chunk,
                                                                     const int* __restrict__ row_offsets,
                                                                     const float* __restrict__ partial,
                                                                     float* __restrict__ out)
{
    using VecT = Vec<VEC>;
    const int lane = threadIdx.x & 63;
    const int r = blockIdx.x * kFlatWaves + (int)__builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    if (r >= M) return;
    const int rs = __builtin_amdgcn_readfirstlane(row_offsets[r]);
    const int re = __builtin_amdgcn_readfirstlane(row_offsets[r + 1]);
    float* orow = out + (size_t)r * N;
    if (rs == re) {
        for (int col = lane * VEC; col < N; col += kWave * VEC) VecT::zero().gstore(orow + min(col, N - VEC));
        return;
    }
    const int ul = rs / chunk;
    const int uh = (re - 1) / chunk;
    if (ul == uh) return;  // the row lies inside one wave's range: that wave stored it
    for (int col = lane * VEC; col < N; col += kWave * VEC) {
        const int c = min(col, N - VEC);  // the last lane of a row moves back to the row's last VEC floats
        VecT sum = VecT::zero();
        for (int u = ul; u <= uh; ++u) {
            const int k = (u == ul && (long long)u * chunk != rs) ? 1 : 0;
            sum.add(VecT::gload(partial + ((size_t)u * 2 + k) * N + c));
        }
        sum.gstore(orow + c);
    }
}

hipError_t row_fixup_launch(int M, int N, int chunk, const int* row_offsets, const float* partial, float* out,
                            hipStream_t stream)
{
    const unsigned blocks = (unsigned)ceil_div(M, kFlatWaves);
    if (N >= 4)
        hipLaunchKernelGGL((row_fixup_kernel<4>), dim3(blocks), dim3(kFlatWaves * 64), 0, stream, M, N, chunk, row_offsets,
                           partial, out);
    else
        hipLaunchKernelGGL((row_fixup_kernel<1>), dim3(blocks), dim3(kFlatWaves * 64), 0, stream, M, N, chunk, row_offsets,
                           partial, out);
    return hipGetLastError();
}

}  // namespace dlspm
