// 2-d transpose y(n,m) = x(m,n)', column-major: the device side of `permutedims(x)` for matrices, which the
// reference takes from CUDA.jl / cublasSgeam (src/knetarrays/reshape.jl:18, src/knetarrays/linalg.jl:92-113) and
// uses for softmax over dims=2 (src/ops20_gpu/softmax.jl:19-20).
// 64x64 tiles go through LDS (row pitch 65 to keep the transposed reads off a single bank) so that both the
// global reads and the global writes are contiguous along lanes.  HBM roofline: 2*sizeof(T)*m*n.
#pragma once
#include "knet8_device.h"

namespace knet8 {

constexpr int kTrTile = 64;

template <typename T>
__global__ __launch_bounds__(256) void transpose_kernel(int m, int n, const T* __restrict__ x, T* __restrict__ y) {
  __shared__ T tile[kTrTile][kTrTile + 1];
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;  // 64 x 4
  const long i0 = (long)blockIdx.x * kTrTile, j0 = (long)blockIdx.y * kTrTile;
#pragma unroll
  for (int q = 0; q < kTrTile / 4; q++) {
    const int r = ty + q * 4;
    const long i = i0 + tx, j = j0 + r;
    if (i < m && j < n) tile[r][tx] = x[i + j * (long)m];
  }
  __syncthreads();
#pragma unroll
  for (int q = 0; q < kTrTile / 4; q++) {
    const int r = ty + q * 4;
    const long j = j0 + tx, i = i0 + r;
    if (i < m && j < n) y[j + i * (long)n] = tile[tx][r];
  }
}

template <typename T> inline void launch_transpose(hipStream_t stream, int m, int n, const T* x, T* y) {
  if (m <= 0 || n <= 0) return;
  const dim3 grid((unsigned)((m + kTrTile - 1) / kTrTile), (unsigned)((n + kTrTile - 1) / kTrTile));
  hipLaunchKernelGGL((transpose_kernel<T>), grid, dim3(256), 0, stream, m, n, x, y);
}

}  // namespace knet8
