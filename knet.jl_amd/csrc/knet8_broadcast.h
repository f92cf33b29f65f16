// General N-d broadcasting z = f(x, y): every operand is addressed through per-dimension element strides, a broadcast
// dimension having stride 0 (src/libknet8/cuda16.jl:10-88 for 3-5 dims with strides by value, cuda17.jl:25-64 for more
// dims with the strides in device arrays; the caller is src/knetarrays/binary.jl:96-125 with get_strides, :214-231).
//
// The reference decomposes every output index with one division per dimension.  Here the strides-by-value entry points
// first collapse neighbouring dimensions that both operands walk contiguously (or both broadcast), which turns the usual
// cases -- (8,8,16,4).+(8,8,1,4), NCHW bias -- into 2 or 3 effective dimensions, and when the first collapsed dimension
// is a multiple of the 16-byte vector a lane handles one whole vector of z (one index decomposition per 4 floats, a vector
// load where the operand's first stride is 1, one scalar load where it is 0).  HBM roofline: sizeof(T) * (N_z + N_x + N_y)
// (broadcast operands are re-read from cache).
#pragma once
#include "knet8_device.h"
#include "knet8_elementwise.h"
#include "knet8_runtime.h"

namespace knet8 {

constexpr int kBcastMaxRank = 5;

struct BcastDims {
  int rank;
  unsigned dim[kBcastMaxRank];
  int sx[kBcastMaxRank];
  int sy[kBcastMaxRank];
};

// Collapse: dims (fastest first) with element strides of x and y (0 = broadcast) and the contiguous strides of z.
// Dimensions of size 1 vanish; dimension k+1 merges into k when, for both operands, stride[k+1] == stride[k]*dim[k]
// (this covers 0 == 0*dim: both steps broadcast).
inline BcastDims bcast_collapse(int nd, const long* dim, const int* sx, const int* sy) {
  BcastDims d;
  d.rank = 0;
  for (int k = 0; k < nd; k++) {
    if (dim[k] == 1) continue;
    if (d.rank > 0) {
      const int p = d.rank - 1;
      if ((long)sx[k] == (long)d.sx[p] * d.dim[p] && (long)sy[k] == (long)d.sy[p] * d.dim[p]) {
        d.dim[p] *= (unsigned)dim[k];
        continue;
      }
    }
    d.dim[d.rank] = (unsigned)dim[k];
    d.sx[d.rank] = sx[k];
    d.sy[d.rank] = sy[k];
    d.rank++;
  }
  if (d.rank == 0) { d.rank = 1; d.dim[0] = 1; d.sx[0] = 0; d.sy[0] = 0; }
  for (int k = d.rank; k < kBcastMaxRank; k++) { d.dim[k] = 1; d.sx[k] = 0; d.sy[k] = 0; }
  return d;
}

// Item i covers NV consecutive elements of z along the first collapsed dimension (dim[0] % NV == 0).
template <typename T, typename F, int NV>
__global__ __launch_bounds__(kEwBlock) void ew_bcast_nd_kernel(unsigned nitems, BcastDims d, const T* x, const T* y, T* z, F f) {
  typedef typename Vec16<T>::type V;
  const unsigned i = blockIdx.x * kEwBlock + threadIdx.x;
  if (i >= nitems) return;
  const unsigned d0 = d.dim[0] / NV;
  unsigned rem = i / d0;
  const unsigned c0 = (i - rem * d0) * NV;
  long ix = (long)c0 * d.sx[0], iy = (long)c0 * d.sy[0];
#pragma unroll
  for (int k = 1; k < kBcastMaxRank; k++) {
    if (k < d.rank) {
      const unsigned q = rem / d.dim[k];
      const unsigned c = rem - q * d.dim[k];
      rem = q;
      ix += (long)c * d.sx[k];
      iy += (long)c * d.sy[k];
    }
  }
  if (NV > 1) {
    V a, b, r;
    if (d.sx[0] == 1) a = *reinterpret_cast<const V*>(x + ix);
    else {
      const T s = x[ix];
#pragma unroll
      for (int e = 0; e < NV; e++) a[e] = s;
    }
    if (d.sy[0] == 1) b = *reinterpret_cast<const V*>(y + iy);
    else {
      const T s = y[iy];
#pragma unroll
      for (int e = 0; e < NV; e++) b[e] = s;
    }
#pragma unroll
    for (int e = 0; e < NV; e++) r[e] = f(a[e], b[e]);
    st_stream(reinterpret_cast<V*>(z + (long)i * NV), r);
  } else {
    z[i] = f(x[ix], y[iy]);
  }
}

// Strides by value (the _16_3/_16_4/_16_5 entry points).  The sizes of z follow from its strides and N.
template <typename T, typename F>
inline void launch_bcast_nd(hipStream_t stream, int nd, const int* sx, const int* sy, const int* sz, long n, const T* x, const T* y, T* z, F f) {
  if (n <= 0) return;
  if (nd < 1 || nd > kBcastMaxRank) { record_error("broadcast: 1 to 5 dimensions expected"); return; }
  long dim[kBcastMaxRank];
  for (int k = 0; k < nd; k++) {
    const long hi = (k + 1 < nd) ? sz[k + 1] : n;
    if (sz[k] <= 0 || hi % sz[k] != 0) { record_error("broadcast: the strides of z are not those of a contiguous array"); return; }
    dim[k] = hi / sz[k];
  }
  if (sz[0] != 1) { record_error("broadcast: z must be contiguous"); return; }
  const BcastDims d = bcast_collapse(nd, dim, sx, sy);
  constexpr int N = Vec16<T>::N;
  // the vector path needs every collapsed step of a unit-stride operand to keep 16-byte alignment: its higher strides are
  // multiples of N whenever dim[0] is, because they are products of the operand's own leading sizes
  bool vec = (d.dim[0] % N == 0) && aligned16(z) && (d.sx[0] == 0 || d.sx[0] == 1) && (d.sy[0] == 0 || d.sy[0] == 1);
  if (d.sx[0] == 1) vec = vec && aligned16(x);
  if (d.sy[0] == 1) vec = vec && aligned16(y);
  for (int k = 1; k < d.rank && vec; k++) {
    if (d.sx[0] == 1 && d.sx[k] % N != 0) vec = false;
    if (d.sy[0] == 1 && d.sy[k] % N != 0) vec = false;
  }
  const long nitems = vec ? n / N : n;
  const unsigned grid = (unsigned)((nitems + kEwBlock - 1) / kEwBlock);
  if (vec) hipLaunchKernelGGL((ew_bcast_nd_kernel<T, F, N>), dim3(grid), dim3(kEwBlock), 0, stream, (unsigned)nitems, d, x, y, z, f);
  else hipLaunchKernelGGL((ew_bcast_nd_kernel<T, F, 1>), dim3(grid), dim3(kEwBlock), 0, stream, (unsigned)nitems, d, x, y, z, f);
}

// Strides in device arrays (the _17 entry point, more than 5 dims): no collapsing (it would need the strides on the host,
// i.e. a blocking copy); the index is decomposed from the slowest dimension down, as the reference does.
template <typename T, typename F>
__global__ __launch_bounds__(kEwBlock) void ew_bcast17_kernel(const T* x, const T* y, T* z, const int* sx, const int* sy, const int* sz, int n, int nd, F f) {
  const long base = (long)blockIdx.x * (kEwBlock * 4) + threadIdx.x;
#pragma unroll
  for (int u = 0; u < 4; u++) {
    const long i = base + u * kEwBlock;
    if (i < n) {
      unsigned rem = (unsigned)i;
      long ix = 0, iy = 0;
      for (int k = nd - 1; k >= 0; k--) {
        const unsigned s = (unsigned)sz[k];
        const unsigned c = rem / s;
        rem -= c * s;
        ix += (long)c * sx[k];
        iy += (long)c * sy[k];
      }
      z[i] = f(x[ix], y[iy]);
    }
  }
}

template <typename T, typename F>
inline void launch_bcast17(hipStream_t stream, const T* x, const T* y, T* z, const int* sx, const int* sy, const int* sz, int n, int nd, F f) {
  if (n <= 0 || nd <= 0) return;
  const long grid = ((long)n + kEwBlock * 4 - 1) / (kEwBlock * 4);
  hipLaunchKernelGGL((ew_bcast17_kernel<T, F>), dim3((unsigned)grid), dim3(kEwBlock), 0, stream, x, y, z, sx, sy, sz, n, nd, f);
}

}  // namespace knet8
