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

// Either side of a chunk is R runs of L contiguous elements, `stride` apart in global memory (R = 1: one contiguous range).
// All 256 lanes walk the R*L elements as one flat range; 16-byte accesses when L, the stride and the base address allow
// (a vector then never straddles two runs), element by element otherwise.  `at(run, pos)` is the element's place in LDS.
template <typename T, typename At>
__device__ __forceinline__ void skinny_load(const T* g, int R, int L, long stride, T* buf, At at) {
  constexpr int NV = Vec16<T>::N;
  typedef typename Vec16<T>::type V;
  const int cnt = R * L;
  if (L % NV == 0 && stride % NV == 0 && aligned16(g)) {
    for (int t = threadIdx.x * NV; t < cnt; t += 256 * NV) {
      const int r = t / L, q = t - r * L;
      const V v = ld_stream(reinterpret_cast<const V*>(g + r * stride + q));
#pragma unroll
      for (int e = 0; e < NV; e++) buf[at(r, q + e)] = v[e];
    }
  } else {
    for (int t = threadIdx.x; t < cnt; t += 256) {
      const int r = t / L, q = t - r * L;
      buf[at(r, q)] = __builtin_nontemporal_load(g + r * stride + q);
    }
  }
}
template <typename T, typename At>
__device__ __forceinline__ void skinny_store(T* g, int R, int L, long stride, const T* buf, At at) {
  constexpr int NV = Vec16<T>::N;
  typedef typename Vec16<T>::type V;
  const int cnt = R * L;
  if (L % NV == 0 && stride % NV == 0 && aligned16(g)) {
    for (int t = threadIdx.x * NV; t < cnt; t += 256 * NV) {
      const int r = t / L, q = t - r * L;
      V v;
#pragma unroll
      for (int e = 0; e < NV; e++) v[e] = buf[at(r, q + e)];
      st_stream(reinterpret_cast<V*>(g + r * stride + q), v);
    }
  } else {
    for (int t = threadIdx.x; t < cnt; t += 256) {
      const int r = t / L, q = t - r * L;
      __builtin_nontemporal_store(buf[at(r, q)], g + r * stride + q);
    }
  }
}

template <typename T, bool SMALL_M>
__global__ __launch_bounds__(256) void transpose_skinny_kernel(int m, int n, int c, long chunks, const T* __restrict__ x, T* __restrict__ y) {
  __shared__ T buf[kTrChunkElems + kTrSkinny + 64];
  const long bz = blockIdx.x / chunks, ch = blockIdx.x - bz * chunks;
  const T* xb = x + bz * (long)m * n;
  T* yb = y + bz * (long)m * n;
  const int pitch = c + 1;
  if (SMALL_M) {
    // x: cc whole columns of m elements = one contiguous range; y: m runs of cc elements, one per row.  LDS: buf[i][j]
    const long j0 = ch * c;
    const int cc = (int)(n - j0 < c ? n - j0 : c);
    skinny_load(xb + j0 * m, 1, cc * m, 0, buf, [=](int, int q) { return (q % m) * pitch + q / m; });
    __syncthreads();
    skinny_store(yb + j0, m, cc, (long)n, buf, [=](int r, int q) { return r * pitch + q; });
  } else {
    // x: n runs of cc elements, one per column; y: cc whole rows of n elements = one contiguous range.  LDS: buf[j][i]
    const long i0 = ch * c;
    const int cc = (int)(m - i0 < c ? m - i0 : c);
    skinny_load(xb + i0, n, cc, (long)m, buf, [=](int r, int q) { return r * pitch + q; });
    __syncthreads();
    skinny_store(yb + i0 * n, 1, cc * n, 0, buf, [=](int, int q) { return (q % n) * pitch + q / n; });
  }
}

template <typename T> inline void launch_transpose_skinny(hipStream_t stream, int m, int n, const T* x, T* y, int batch) {
  const int small = m < n ? m : n, large = m < n ? n : m;
  int c = kTrChunkElems / small;
  c -= c % 4;   // chunk boundaries stay on 16-byte boundaries when the matrix allows vectors at all
  const long chunks = ((long)large + c - 1) / c;
  const long blocks = chunks * batch;
  if (blocks > 0x7fffffffL) { record_error("transpose: too many chunks"); return; }
  if (m <= n) hipLaunchKernelGGL((transpose_skinny_kernel<T, true>), dim3((unsigned)blocks), dim3(256), 0, stream, m, n, c, chunks, x, y);
  else hipLaunchKernelGGL((transpose_skinny_kernel<T, false>), dim3((unsigned)blocks), dim3(256), 0, stream, m, n, c, chunks, x, y);
}

}  // namespace knet8
