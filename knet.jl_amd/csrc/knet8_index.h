// Index kernels.  First: gather / scatter-add on 1-based int32 linear indices: the device side of `x[indices]` and of its
// gradient (src/libknet8/cuda1.jl:342-362; callers src/knetarrays/getindex.jl:217-220,291-298 and
// src/autograd_gpu/addto.jl:59-65).  n is the number of indices (one per instance on the nll path), so
// these are latency-, not bandwidth-bound; one lane per index.
#pragma once
#include "knet8_device.h"

namespace knet8 {

template <typename T> __global__ __launch_bounds__(256) void getents_kernel(long n, const int* ents, const T* x, T* y) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i < n) y[i] = x[(long)ents[i] - 1];
}

// Hardware floating-point atomic add (global_atomic_add_f32 / _f64).  When the indices are unique, as
// they are for nll (one labelled entry per column), the result does not depend on the order of arrival.
template <typename T> __global__ __launch_bounds__(256) void addents_kernel(long n, const int* ents, T* x, const T* y) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i < n) unsafeAtomicAdd(x + ((long)ents[i] - 1), y[i]);
}

template <typename T> __global__ __launch_bounds__(256) void setents_kernel(long n, const int* ents, T* x, const T* y) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i < n) x[(long)ents[i] - 1] = y[i];
}

template <typename T> inline void launch_getents(hipStream_t s, long n, const int* ents, const T* x, T* y) {
  if (n > 0) hipLaunchKernelGGL((getents_kernel<T>), dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, n, ents, x, y);
}
template <typename T> inline void launch_addents(hipStream_t s, long n, const int* ents, T* x, const T* y) {
  if (n > 0) hipLaunchKernelGGL((addents_kernel<T>), dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, n, ents, x, y);
}
template <typename T> inline void launch_setents(hipStream_t s, long n, const int* ents, T* x, const T* y) {
  if (n > 0) hipLaunchKernelGGL((setents_kernel<T>), dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, n, ents, x, y);
}


template <typename T> __global__ __launch_bounds__(256) void setent1_kernel(long n, const int* ents, T* x, T v) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i < n) x[(long)ents[i] - 1] = v;
}
template <typename T> inline void launch_setent1(hipStream_t s, long n, const int* ents, T* x, T v) {
  if (n > 0) hipLaunchKernelGGL((setent1_kernel<T>), dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, n, ents, x, v);
}

// ---- whole columns / rows of a matrix by 1-based int32 index ---------------------------------------------
// x is xrows x xcols column-major; `cols` (`rows`) holds the selected columns (rows); y is the xrows x ncols
// (nrows x xcols) matrix of the selection (src/libknet8/cuda1.jl:234-341; callers src/knetarrays/getindex.jl:235-271
// for x[:,i] / x[i,:], src/autograd_gpu/addto.jl:67-83 for the gradient of an embedding lookup).
// MODE 0: y = x[sel]; 1: x[sel] = y; 2: x[sel] += y (hardware atomic add, so repeated indices accumulate);
// 3: x[sel] = v.  Bit-exact index work; with repeated indices MODE 1 keeps one of the writers and MODE 2 adds in
// arrival order, as in the reference.
// Columns are contiguous: a lane moves NV consecutive rows of one column (16 bytes when xrows % NV == 0 and the
// operands are aligned), so a column copy streams like a plain copy (MODE 2 has a kernel of its own below).  HBM roofline: 2*sizeof(T) per selected element.
template <typename T, int MODE, int NV>
__global__ __launch_bounds__(256) void cols_kernel(long nitems, int xrows, const int* cols, T* x, T* y, T v) {
  typedef typename Vec16<T>::type V;
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= nitems) return;
  const unsigned per = (unsigned)xrows / NV;
  const unsigned col = (unsigned)(i / per);
  const unsigned row = ((unsigned)i - col * per) * NV;
  T* xp = x + ((long)cols[col] - 1) * xrows + row;
  T* yp = y + i * NV;
  if (NV > 1) {
    if (MODE == 0) *reinterpret_cast<V*>(yp) = *reinterpret_cast<const V*>(xp);
    else if (MODE == 1) *reinterpret_cast<V*>(xp) = *reinterpret_cast<const V*>(yp);
    else if (MODE == 2) {
      const V t = *reinterpret_cast<const V*>(yp);
#pragma unroll
      for (int e = 0; e < NV; e++) unsafeAtomicAdd(xp + e, t[e]);
    } else {
      V t;
#pragma unroll
      for (int e = 0; e < NV; e++) t[e] = v;
      *reinterpret_cast<V*>(xp) = t;
    }
  } else {
    if (MODE == 0) *yp = *xp;
    else if (MODE == 1) *xp = *yp;
    else if (MODE == 2) unsafeAtomicAdd(xp, *yp);
    else *xp = v;
  }
}

// x[:, cols] += y, the gradient of an embedding lookup: one element per lane, so that every atomic instruction of a wave covers 64 consecutive elements of one
// column (of two where the wave crosses a column boundary).  The atomic units work on whole cache lines: a wave whose lanes are 16 bytes apart -- the layout of
// the copies above -- sends them four times as many lines per instruction.  Measured, fp32: x(512,32000) with 2048 columns selected 16.8 us with the 16-byte
// layout, 5.3 with this one (the bytes at the elementwise rate: 5.3); (1024,50257) with 4096 columns 56.8 -> 15.1; (768,50257) with 16384 columns 166.7 -> 41.7,
// and with the repeated indices of a Zipf-distributed vocabulary (additions to one address are carried out one after the other) 470 -> 118.  Two, four or eight
// elements per lane, 64 apart, are 2-15 % slower than one.
template <typename T, typename I>
__global__ __launch_bounds__(256) void cols_add_kernel(I n, I xrows, const int* cols, T* x, const T* y) {
  const I k = (I)blockIdx.x * 256 + threadIdx.x;
  if (k >= n) return;
  const I col = k / xrows, row = k - col * xrows;
  unsafeAtomicAdd(x + ((long)cols[col] - 1) * (long)xrows + (long)row, __builtin_nontemporal_load(y + k));
}

template <typename T, int MODE>
inline void launch_cols(hipStream_t s, int xrows, int xcols, int ncols, const int* cols, T* x, T* y, T v) {
  if (ncols <= 0 || xrows <= 0 || xcols <= 0) return;
  constexpr int N = Vec16<T>::N;
  if (MODE == 2) {
    const long n = (long)xrows * ncols;
    const dim3 grid((unsigned)((n + 255) / 256));
    if (n + 256 < (1L << 32)) hipLaunchKernelGGL((cols_add_kernel<T, unsigned>), grid, dim3(256), 0, s, (unsigned)n, (unsigned)xrows, cols, x, y);
    else hipLaunchKernelGGL((cols_add_kernel<T, unsigned long>), grid, dim3(256), 0, s, (unsigned long)n, (unsigned long)xrows, cols, x, y);
    return;
  }
  const bool vec = (xrows % N == 0) && aligned16(x) && (MODE == 3 || aligned16(y));
  const long nitems = (long)xrows * ncols / (vec ? N : 1);
  const dim3 grid((unsigned)((nitems + 255) / 256));
  if (vec) hipLaunchKernelGGL((cols_kernel<T, MODE, N>), grid, dim3(256), 0, s, nitems, xrows, cols, x, y, v);
  else hipLaunchKernelGGL((cols_kernel<T, MODE, 1>), grid, dim3(256), 0, s, nitems, xrows, cols, x, y, v);
}

// Rows are strided: lanes run along the selected rows of one column (y contiguous, x gathered within the column).
template <typename T, int MODE>
__global__ __launch_bounds__(256) void rows_kernel(long n, int xrows, int nrows, const int* rows, T* x, T* y, T v) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const unsigned col = (unsigned)(i / (unsigned)nrows);
  const unsigned row = (unsigned)i - col * (unsigned)nrows;
  T* xp = x + ((long)rows[row] - 1) + (long)col * xrows;
  if (MODE == 0) y[i] = *xp;
  else if (MODE == 1) *xp = y[i];
  else if (MODE == 2) unsafeAtomicAdd(xp, y[i]);
  else *xp = v;
}

template <typename T, int MODE>
inline void launch_rows(hipStream_t s, int xrows, int xcols, int nrows, const int* rows, T* x, T* y, T v) {
  if (nrows <= 0 || xrows <= 0 || xcols <= 0) return;
  const long n = (long)nrows * xcols;
  hipLaunchKernelGGL((rows_kernel<T, MODE>), dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, n, xrows, nrows, rows, x, y, v);
}

// ---- rectangular blocks: y[row + col*incy] = x[row + col*incx] over nrows x ncols units ---------------------
// xcopy counts in bytes (src/libknet8/cuda1.jl:130-165; the caller scales rows and steps by sizeof(T),
// src/knetarrays/getindex.jl:656-660,697-700): the widest unit (16, 8, 4 or 1 bytes) that divides the row length, both
// steps and both addresses is moved per lane.  xfill counts in elements (cuda1.jl:107-128).
template <typename U>
__global__ __launch_bounds__(256) void xcopy_kernel(long n, unsigned nrows, const U* x, long incx, U* y, long incy) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const unsigned col = (unsigned)(i / nrows);
  const unsigned row = (unsigned)i - col * nrows;
  y[row + col * incy] = x[row + col * incx];
}

inline void launch_xcopy(hipStream_t s, int nrows, int ncols, const void* x, int incx, void* y, int incy) {
  if (nrows <= 0 || ncols <= 0) return;
  const uintptr_t bits = (uintptr_t)nrows | (uintptr_t)(unsigned)incx | (uintptr_t)(unsigned)incy | reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y);
  const int unit = (bits % 16 == 0) ? 16 : (bits % 8 == 0) ? 8 : (bits % 4 == 0) ? 4 : 1;
  const long n = (long)(nrows / unit) * ncols;
  const dim3 grid((unsigned)((n + 255) / 256));
#define KNET8_XCOPY(U) hipLaunchKernelGGL((xcopy_kernel<U>), grid, dim3(256), 0, s, n, (unsigned)(nrows / unit), static_cast<const U*>(x), (long)(incx / unit), static_cast<U*>(y), (long)(incy / unit))
  if (unit == 16) KNET8_XCOPY(uint4);
  else if (unit == 8) KNET8_XCOPY(uint2);
  else if (unit == 4) KNET8_XCOPY(unsigned);
  else KNET8_XCOPY(unsigned char);
#undef KNET8_XCOPY
}

template <typename T>
__global__ __launch_bounds__(256) void xfill_kernel(long n, unsigned nrows, T v, T* y, long incy) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const unsigned col = (unsigned)(i / nrows);
  const unsigned row = (unsigned)i - col * nrows;
  y[row + col * incy] = v;
}
template <typename T> inline void launch_xfill(hipStream_t s, int nrows, int ncols, T v, T* y, int incy) {
  if (nrows <= 0 || ncols <= 0) return;
  const long n = (long)nrows * ncols;
  hipLaunchKernelGGL((xfill_kernel<T>), dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, n, (unsigned)nrows, v, y, (long)incy);
}

// ---- concatenation -----------------------------------------------------------------------------------------
// icat: y[:,col] = x[col][0:nrows] where x is a HOST array of ncols device pointers (src/libknet8/cuda1.jl:167-207).
// The reference allocates a device copy of the pointer list, copies it synchronously and frees it on every call; here
// the pointers travel as kernel arguments, 32 columns per launch: no allocation and no blocking copy.
constexpr int kIcatChunk = 32;
template <typename T> struct IcatPtrs { const T* p[kIcatChunk]; };
template <typename T>
__global__ __launch_bounds__(256) void icat_kernel(int nrows, IcatPtrs<T> src, T* y) {
  const T* xc = src.p[blockIdx.y];
  T* yc = y + (long)blockIdx.y * nrows;
  for (long r = (long)blockIdx.x * 256 + threadIdx.x; r < nrows; r += (long)gridDim.x * 256) yc[r] = xc[r];
}
template <typename T> inline void launch_icat(hipStream_t s, int nrows, int ncols, T** x, T* y) {
  if (nrows <= 0 || ncols <= 0) return;
  unsigned gx = (unsigned)((nrows + 255) / 256);
  if (gx > 1024) gx = 1024;
  for (int c0 = 0; c0 < ncols; c0 += kIcatChunk) {
    const int nc = ncols - c0 < kIcatChunk ? ncols - c0 : kIcatChunk;
    IcatPtrs<T> src;
    for (int k = 0; k < kIcatChunk; k++) src.p[k] = k < nc ? x[c0 + k] : nullptr;
    hipLaunchKernelGGL((icat_kernel<T>), dim3(gx, (unsigned)nc), dim3(256), 0, s, nrows, src, y + (long)c0 * nrows);
  }
}

// concat: y[starts[a] + i] = x[a][i], i < lengths[a]; starts, lengths and the pointer list x are DEVICE arrays
// (src/libknet8/cuda1.jl:503-530).  The lengths are unknown on the host, so every array gets a fixed number of
// workgroups that stride over it (the reference gives each array one workgroup).
constexpr int kConcatSplit = 16;
template <typename T>
__global__ __launch_bounds__(256) void concat_kernel(const int* starts, const int* lengths, T* const* x, T* y) {
  const int a = blockIdx.x;
  const long n = lengths[a], off = starts[a];
  const T* xa = x[a];
  for (long i = (long)blockIdx.y * 256 + threadIdx.x; i < n; i += (long)kConcatSplit * 256) y[off + i] = xa[i];
}
template <typename T> inline void launch_concat(hipStream_t s, int narrays, const int* starts, const int* lengths, T** x, T* y) {
  if (narrays <= 0) return;
  hipLaunchKernelGGL((concat_kernel<T>), dim3((unsigned)narrays, kConcatSplit), dim3(256), 0, s, starts, lengths, x, y);
}

}  // namespace knet8
