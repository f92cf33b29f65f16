// 2-d transpose y(n,m) = x(m,n)', column-major: the device side of `permutedims(x)` for matrices, which the
// reference takes from CUDA.jl / cublasSgeam (src/knetarrays/reshape.jl:18, src/knetarrays/linalg.jl:92-113) and
// uses for softmax over dims=2 (src/ops20_gpu/softmax.jl:19-20).
// 64x64 tiles go through LDS (row pitch 65 to keep the transposed reads off a single bank) so that both the
// global reads and the global writes are contiguous along lanes.  HBM roofline: 2*sizeof(T)*m*n.
#pragma once
#include "knet8_device.h"
#include "knet8_runtime.h"

namespace knet8 {

constexpr int kTrTile = 64;

// `batch` matrices one after the other (x viewed as (m, n, batch) -> y as (n, m, batch)): the permutation (2,1,3), used to bring a
// softmax over a middle dimension down to contiguous columns.  One linear grid index covers (tile row, tile column, batch), so no
// grid dimension can overflow.
template <typename T>
__global__ __launch_bounds__(256) void transpose_kernel(int m, int n, long tiles_m, long tiles_n, const T* __restrict__ x, T* __restrict__ y) {
  __shared__ T tile[kTrTile][kTrTile + 1];
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;  // 64 x 4
  const long per = tiles_m * tiles_n;
  const long bz = blockIdx.x / per, rem = blockIdx.x - bz * per;
  const long i0 = (rem % tiles_m) * kTrTile, j0 = (rem / tiles_m) * kTrTile;
  const T* xb = x + bz * (long)m * n;
  T* yb = y + bz * (long)m * n;
#pragma unroll
  for (int q = 0; q < kTrTile / 4; q++) {
    const int r = ty + q * 4;
    const long i = i0 + tx, j = j0 + r;
    if (i < m && j < n) tile[r][tx] = xb[i + j * (long)m];
  }
  __syncthreads();
#pragma unroll
  for (int q = 0; q < kTrTile / 4; q++) {
    const int r = ty + q * 4;
    const long j = j0 + tx, i = i0 + r;
    if (i < m && j < n) yb[j + i * (long)n] = tile[tx][r];
  }
}

// Skinny matrices (one side of at most 32): 64x64 tiles would leave most lanes idle.  A workgroup takes a chunk of c = 4096/small
// whole columns (SMALL_M: m is the small side) or rows (n is the small side) -- contiguous on the side where the matrix is
// skinny -- through LDS; the other side moves in contiguous runs of c elements.  The LDS pitch c+1 is odd: no bank conflicts.
constexpr int kTrSkinny = 32, kTrChunkElems = 4096;
template <typename T, bool SMALL_M>
__global__ __launch_bounds__(256) void transpose_skinny_kernel(int m, int n, int c, long chunks, const T* __restrict__ x, T* __restrict__ y) {
  __shared__ T buf[kTrChunkElems + kTrSkinny + 64];
  const long bz = blockIdx.x / chunks, ch = blockIdx.x - bz * chunks;
  const T* xb = x + bz * (long)m * n;
  T* yb = y + bz * (long)m * n;
  const int pitch = c + 1;
  if (SMALL_M) {
    const long j0 = ch * c;
    const int cc = (int)(n - j0 < c ? n - j0 : c), cnt = cc * m;
    for (int t = threadIdx.x; t < cnt; t += 256) buf[(t % m) * pitch + t / m] = xb[j0 * m + t];          // contiguous read
    __syncthreads();
    for (int t = threadIdx.x; t < cnt; t += 256) yb[j0 + (t % cc) + (long)(t / cc) * n] = buf[(t / cc) * pitch + t % cc];
  } else {
    const long i0 = ch * c;
    const int cc = (int)(m - i0 < c ? m - i0 : c), cnt = cc * n;
    for (int t = threadIdx.x; t < cnt; t += 256) buf[(t / cc) * pitch + t % cc] = xb[i0 + (t % cc) + (long)(t / cc) * m];
    __syncthreads();
    for (int t = threadIdx.x; t < cnt; t += 256) yb[i0 * n + t] = buf[(t % n) * pitch + t / n];           // contiguous write
  }
}

template <typename T> inline void launch_transpose(hipStream_t stream, int m, int n, const T* x, T* y, int batch = 1) {
  if (m <= 0 || n <= 0 || batch <= 0) return;
  const int small = m < n ? m : n, large = m < n ? n : m;
  if (small <= kTrSkinny && large > kTrTile) {
    const int c = kTrChunkElems / small;
    const long chunks = ((long)large + c - 1) / c;
    const long blocks = chunks * batch;
    if (blocks > 0x7fffffffL) { record_error("transpose: too many chunks"); return; }
    if (m <= n) hipLaunchKernelGGL((transpose_skinny_kernel<T, true>), dim3((unsigned)blocks), dim3(256), 0, stream, m, n, c, chunks, x, y);
    else hipLaunchKernelGGL((transpose_skinny_kernel<T, false>), dim3((unsigned)blocks), dim3(256), 0, stream, m, n, c, chunks, x, y);
    return;
  }
  const long tiles_m = (m + kTrTile - 1) / kTrTile, tiles_n = (n + kTrTile - 1) / kTrTile;
  const long blocks = tiles_m * tiles_n * batch;
  if (blocks > 0x7fffffffL) { record_error("transpose: too many tiles"); return; }
  hipLaunchKernelGGL((transpose_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, stream, m, n, tiles_m, tiles_n, x, y);
}

}  // namespace knet8
