// Chunked transpose for skinny matrices, y(n,m) = x(m,n)' column-major with one side of at most 32 (optionally `batch`
// matrices one after the other): the short-side case of the permutation kernels in knet8_permute.h, which cover everything else.
// Callers: transpose_S / permute213_S / permutedims_S, i.e. `permutedims` of the reference (src/knetarrays/reshape.jl:18-33) and
// its softmax over dims=2 (src/ops20_gpu/softmax.jl:19-20).  HBM roofline: 2*sizeof(T)*m*n.
#pragma once
#include "knet8_device.h"
#include "knet8_runtime.h"

namespace knet8 {

constexpr int kTrTile = 64;

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

template <typename T> inline void launch_transpose_skinny(hipStream_t stream, int m, int n, const T* x, T* y, int batch) {
  const int small = m < n ? m : n, large = m < n ? n : m;
  const int c = kTrChunkElems / small;
  const long chunks = ((long)large + c - 1) / c;
  const long blocks = chunks * batch;
  if (blocks > 0x7fffffffL) { record_error("transpose: too many chunks"); return; }
  if (m <= n) hipLaunchKernelGGL((transpose_skinny_kernel<T, true>), dim3((unsigned)blocks), dim3(256), 0, stream, m, n, c, chunks, x, y);
  else hipLaunchKernelGGL((transpose_skinny_kernel<T, false>), dim3((unsigned)blocks), dim3(256), 0, stream, m, n, c, chunks, x, y);
}

}  // namespace knet8
