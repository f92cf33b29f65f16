// Gather / scatter-add on 1-based int32 linear indices: the device side of `x[indices]` and of its
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

}  // namespace knet8
