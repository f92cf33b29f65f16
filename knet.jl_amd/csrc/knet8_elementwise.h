// Elementwise kernel family: out[i] = f(a[i] [, b[i] [, c[i]]]) over a flat length-n array.
//
// Replaces the reference's fixed <<<256,256>>> scalar grid-stride loops (src/libknet8/cuda1.jl:13-38,
// cuda01.jl:11-25, cuda11.jl:12-28, cuda111.jl:12-29, relu.jl:8-38) with a one-shot grid of
// 256-thread workgroups in which every lane moves one 16-byte vector per operand with the
// non-temporal hint.  Measured on MI355X this shape (many small workgroups, one dwordx4 per lane per
// stream, no loop) sustains the highest 2R+1W bandwidth; persistent grid-stride variants were slower.
//
// HBM roofline: (NIN+1)*sizeof(T) algorithmic bytes per element.
#pragma once
#include "knet8_device.h"

namespace knet8 {

constexpr int kEwBlock = 256;

template <typename T, int NIN, typename F> struct EwApply;
template <typename T, typename F> struct EwApply<T, 0, F> {
  __device__ static __forceinline__ T go(const F& f, T, T, T) { return f(); }
};
template <typename T, typename F> struct EwApply<T, 1, F> {
  __device__ static __forceinline__ T go(const F& f, T a, T, T) { return f(a); }
};
template <typename T, typename F> struct EwApply<T, 2, F> {
  __device__ static __forceinline__ T go(const F& f, T a, T b, T) { return f(a, b); }
};
template <typename T, typename F> struct EwApply<T, 3, F> {
  __device__ static __forceinline__ T go(const F& f, T a, T b, T c) { return f(a, b, c); }
};

// Vector path.  Operands are congruent modulo 16 bytes: after `head` scalar elements every pointer
// is 16-byte aligned.  Elements [head, head + nvec*N) go through vectors; the `head` leading and the
// trailing (n - tail0) elements are handled as scalars by the first lanes of workgroup 0.
template <typename T, int NIN, typename F>
__global__ __launch_bounds__(kEwBlock) void ew_vec_kernel(long nvec, int head, long tail0, long n, const T* a, const T* b,
                                                          const T* c, T* out, F f KNET8_TL_PARAM) {
  KNET8_TL_BEGIN
  typedef typename Vec16<T>::type V;
  constexpr int N = Vec16<T>::N;
  const long i = (long)blockIdx.x * kEwBlock + threadIdx.x;
  if (i < nvec) {
    const long e = head + i * N;
    V va, vb, vc, r;
    if (NIN >= 1) va = ld_stream(reinterpret_cast<const V*>(a + e));
    if (NIN >= 2) vb = ld_stream(reinterpret_cast<const V*>(b + e));
    if (NIN >= 3) vc = ld_stream(reinterpret_cast<const V*>(c + e));
#pragma unroll
    for (int k = 0; k < N; k++)
      r[k] = EwApply<T, NIN, F>::go(f, NIN >= 1 ? va[k] : T(0), NIN >= 2 ? vb[k] : T(0), NIN >= 3 ? vc[k] : T(0));
    st_stream(reinterpret_cast<V*>(out + e), r);
  }
  if (blockIdx.x == 0) {
    long e = -1;
    if ((int)threadIdx.x < head) e = threadIdx.x;
    else if (threadIdx.x >= kWave && tail0 + (threadIdx.x - kWave) < n) e = tail0 + (threadIdx.x - kWave);
    if (e >= 0)
      out[e] = EwApply<T, NIN, F>::go(f, NIN >= 1 ? a[e] : T(0), NIN >= 2 ? b[e] : T(0), NIN >= 3 ? c[e] : T(0));
  }
  KNET8_TL_END
}

// Scalar path for operands whose addresses differ modulo 16 bytes (sub-array views that start at
// arbitrary element offsets).  Lanes still read consecutive elements, four per thread.
template <typename T, int NIN, typename F>
__global__ __launch_bounds__(kEwBlock) void ew_scalar_kernel(long n, const T* a, const T* b, const T* c, T* out, F f) {
  const long base = (long)blockIdx.x * (kEwBlock * 4) + threadIdx.x;
  T ra[4], rb[4], rc[4];
#pragma unroll
  for (int u = 0; u < 4; u++) {
    const long e = base + u * kEwBlock;
    if (e < n) {
      if (NIN >= 1) ra[u] = a[e];
      if (NIN >= 2) rb[u] = b[e];
      if (NIN >= 3) rc[u] = c[e];
    }
  }
#pragma unroll
  for (int u = 0; u < 4; u++) {
    const long e = base + u * kEwBlock;
    if (e < n)
      out[e] = EwApply<T, NIN, F>::go(f, NIN >= 1 ? ra[u] : T(0), NIN >= 2 ? rb[u] : T(0), NIN >= 3 ? rc[u] : T(0));
  }
}

template <typename T, int NIN, typename F>
inline void launch_ew(hipStream_t stream, long n, const T* a, const T* b, const T* c, T* out, F f) {
  if (n <= 0) return;
  constexpr int N = Vec16<T>::N;
  const uintptr_t mo = reinterpret_cast<uintptr_t>(out) & 15u;
  bool congruent = (mo % sizeof(T)) == 0;
  if (NIN >= 1) congruent = congruent && ((reinterpret_cast<uintptr_t>(a) & 15u) == mo);
  if (NIN >= 2) congruent = congruent && ((reinterpret_cast<uintptr_t>(b) & 15u) == mo);
  if (NIN >= 3) congruent = congruent && ((reinterpret_cast<uintptr_t>(c) & 15u) == mo);
  if (congruent) {
    long head = mo ? (long)((16u - mo) / sizeof(T)) : 0;
    if (head > n) head = n;
    const long nvec = (n - head) / N;
    const long tail0 = head + nvec * N;
    long grid = (nvec + kEwBlock - 1) / kEwBlock;
    if (grid < 1) grid = 1;
    hipLaunchKernelGGL((ew_vec_kernel<T, NIN, F>), dim3((unsigned)grid), dim3(kEwBlock), 0, stream, nvec, (int)head, tail0, n,
                       a, b, c, out, f KNET8_TL_ARG);
  } else {
    const long grid = (n + kEwBlock * 4 - 1) / (kEwBlock * 4);
    hipLaunchKernelGGL((ew_scalar_kernel<T, NIN, F>), dim3((unsigned)grid), dim3(kEwBlock), 0, stream, n, a, b, c, out, f);
  }
}

// z = f(x[.], y[.]) where each operand is either full size or a vector along one dimension of the
// result: element i of the result reads x[(i/sx)%nx] (src/libknet8/cuda12.jl:18-27).  Used for the
// forward bias add; HBM roofline 2*sizeof(T) per element (the vector operand stays in cache).
template <typename T, typename F>
__global__ __launch_bounds__(kEwBlock) void ew_bcast12_kernel(long n, const T* x, int sx, int nx, const T* y, int sy, int ny,
                                                              T* z, F f) {
  // n is a 32-bit int at the ABI: index arithmetic in 32 bits (a 64-bit division costs several times more than the memory access)
  const unsigned base = blockIdx.x * (kEwBlock * 4) + threadIdx.x;
  const unsigned un = (unsigned)n, unx = (unsigned)nx, uny = (unsigned)ny, usx = (unsigned)sx, usy = (unsigned)sy;
#pragma unroll
  for (int u = 0; u < 4; u++) {
    const unsigned i = base + u * kEwBlock;
    if (i < un) {
      const T xi = (unx == un ? x[i] : usx == 1 ? x[i % unx] : unx == 1 ? x[0] : x[(i / usx) % unx]);
      const T yi = (uny == un ? y[i] : usy == 1 ? y[i % uny] : uny == 1 ? y[0] : y[(i / usy) % uny]);
      z[i] = f(xi, yi);
    }
  }
}

// Fast path of the vector broadcast for the shapes the MLP path produces: one operand is the full array, the
// other a vector along a single dimension, everything 16-byte aligned and the vector's stride or length a
// multiple of the lanes of a 16-byte access.  XFULL says which operand is the full one (operand order matters
// for sub/div).  s == 1: the vector runs along the contiguous dimension, so the four elements of an access
// take four consecutive vector entries (one aligned 16-byte load of the vector, which stays in cache);
// s > 1: all four elements of an access share one vector entry.
template <typename T, typename F, bool XFULL>
__global__ __launch_bounds__(kEwBlock) void ew_bias_vec_kernel(long nvec, const T* full, const T* vec, int s, int nv, T* z, F f) {
  typedef typename Vec16<T>::type V;
  constexpr int N = Vec16<T>::N;
  const long i = (long)blockIdx.x * kEwBlock + threadIdx.x;
  if (i >= nvec) return;
  const long e = i * N;
  const V a = ld_stream(reinterpret_cast<const V*>(full + e));
  V b;
  if (s == 1) {
    b = *reinterpret_cast<const V*>(vec + ((unsigned)e % (unsigned)nv));  // n is a 32-bit int at the ABI: 32-bit division
  } else {
    const T bv = vec[((unsigned)e / (unsigned)s) % (unsigned)nv];
#pragma unroll
    for (int k = 0; k < N; k++) b[k] = bv;
  }
  V r;
#pragma unroll
  for (int k = 0; k < N; k++) r[k] = XFULL ? f(a[k], b[k]) : f(b[k], a[k]);
  st_stream(reinterpret_cast<V*>(z + e), r);
}

// The same with a vector of any length and stride (1001 classes, a vocabulary of 50257): the full-size operand still moves in 16-byte accesses over
// the flat array, the vector's entries are fetched one by one (they stay in cache) with the position in the vector carried along instead of divided
// out per element.  The last n % N elements are done by workgroup 0.  (Measured on (1001, 8380) fp32: 18.0 -> 13.7 us.)
template <typename T, typename F, bool XFULL>
__global__ __launch_bounds__(kEwBlock) void ew_bias_gather_kernel(long nvec, long n, const T* full, const T* vec, unsigned s, unsigned nv, T* z, F f) {
  typedef typename Vec16<T>::type V;
  constexpr int N = Vec16<T>::N;
  const long i = (long)blockIdx.x * kEwBlock + threadIdx.x;
  if (i < nvec) {
    const long e = i * N;
    const V a = ld_stream(reinterpret_cast<const V*>(full + e));
    const unsigned q = (unsigned)e / s;      // n is a 32-bit int at the ABI: 32-bit division
    unsigned p = (unsigned)e - q * s, idx = q % nv;
    V r;
#pragma unroll
    for (int k = 0; k < N; k++) {
      const T bv = vec[idx];
      r[k] = XFULL ? f(a[k], bv) : f(bv, a[k]);
      if (++p == s) { p = 0; if (++idx == nv) idx = 0; }
    }
    st_stream(reinterpret_cast<V*>(z + e), r);
  }
  if (blockIdx.x == 0) {
    const long e = nvec * N + threadIdx.x;
    if (e < n) {
      const T bv = vec[((unsigned)e / s) % nv];
      z[e] = XFULL ? f(full[e], bv) : f(bv, full[e]);
    }
  }
}

template <typename T, typename F>
inline void launch_bcast12(hipStream_t stream, long n, const T* x, int sx, int nx, const T* y, int sy, int ny, T* z, F f) {
  if (n <= 0) return;
  constexpr int N = Vec16<T>::N;
  const bool xfull = (nx == n), yfull = (ny == n);
  if (xfull != yfull && n % N == 0 && aligned16(x) && aligned16(y) && aligned16(z)) {
    const int s = xfull ? sy : sx, nv = xfull ? ny : nx;
    const bool fits = (s == 1) ? (nv % N == 0) : (s % N == 0);
    if (fits && nv > 1) {
      const long nvec = n / N, grid = (nvec + kEwBlock - 1) / kEwBlock;
      if (xfull)
        hipLaunchKernelGGL((ew_bias_vec_kernel<T, F, true>), dim3((unsigned)grid), dim3(kEwBlock), 0, stream, nvec, x, y, s, nv, z, f);
      else
        hipLaunchKernelGGL((ew_bias_vec_kernel<T, F, false>), dim3((unsigned)grid), dim3(kEwBlock), 0, stream, nvec, y, x, s, nv, z, f);
      return;
    }
  }
  if (xfull != yfull && n >= 4 * N && n < (1L << 32)) {
    const T* full = xfull ? x : y;
    const T* vec = xfull ? y : x;
    const int s = xfull ? sy : sx, nv = xfull ? ny : nx;
    if (aligned16(full) && aligned16(z) && s >= 1 && nv >= 1) {
      const long nvec = n / N, grid = (nvec + kEwBlock - 1) / kEwBlock;
      if (xfull)
        hipLaunchKernelGGL((ew_bias_gather_kernel<T, F, true>), dim3((unsigned)grid), dim3(kEwBlock), 0, stream, nvec, n, full, vec, (unsigned)s, (unsigned)nv, z, f);
      else
        hipLaunchKernelGGL((ew_bias_gather_kernel<T, F, false>), dim3((unsigned)grid), dim3(kEwBlock), 0, stream, nvec, n, full, vec, (unsigned)s, (unsigned)nv, z, f);
      return;
    }
  }
  const long grid = (n + kEwBlock * 4 - 1) / (kEwBlock * 4);
  hipLaunchKernelGGL((ew_bcast12_kernel<T, F>), dim3((unsigned)grid), dim3(kEwBlock), 0, stream, n, x, sx, nx, y, sy, ny, z, f);
}

// In-place update of NARR same-length arrays: v[k] = element of array k; f(v) rewrites some of them; the arrays
// whose bit is set in WMASK are stored back.  One pass over every array instead of the axpy!/lmul!/broadcast
// chains of the optimizers (src/train20/update.jl:513-570).  HBM roofline: (NARR + popcount(WMASK))*sizeof(T)
// bytes per element.  Vector path when every array is 16-byte aligned, scalar otherwise; the last n % N
// elements are done as scalars by workgroup 0.
template <typename T, int NARR, unsigned WMASK, typename F>
__global__ __launch_bounds__(kEwBlock) void ew_update_vec_kernel(long nvec, long n, T* a0, T* a1, T* a2, T* a3, F f) {
  typedef typename Vec16<T>::type V;
  constexpr int N = Vec16<T>::N;
  T* arr[4] = {a0, a1, a2, a3};
  const long i = (long)blockIdx.x * kEwBlock + threadIdx.x;
  if (i < nvec) {
    V in[NARR];
#pragma unroll
    for (int k = 0; k < NARR; k++) in[k] = ld_stream(reinterpret_cast<const V*>(arr[k] + i * N));
#pragma unroll
    for (int e = 0; e < N; e++) {
      T v[NARR];
#pragma unroll
      for (int k = 0; k < NARR; k++) v[k] = in[k][e];
      f(v);
#pragma unroll
      for (int k = 0; k < NARR; k++) in[k][e] = v[k];
    }
#pragma unroll
    for (int k = 0; k < NARR; k++)
      if (WMASK & (1u << k)) st_stream(reinterpret_cast<V*>(arr[k] + i * N), in[k]);
  }
  if (blockIdx.x == 0) {
    const long e = nvec * N + threadIdx.x;
    if (e < n) {
      T v[NARR];
#pragma unroll
      for (int k = 0; k < NARR; k++) v[k] = arr[k][e];
      f(v);
#pragma unroll
      for (int k = 0; k < NARR; k++)
        if (WMASK & (1u << k)) arr[k][e] = v[k];
    }
  }
}

template <typename T, int NARR, unsigned WMASK, typename F>
__global__ __launch_bounds__(kEwBlock) void ew_update_scalar_kernel(long n, T* a0, T* a1, T* a2, T* a3, F f) {
  T* arr[4] = {a0, a1, a2, a3};
  const long e = (long)blockIdx.x * kEwBlock + threadIdx.x;
  if (e >= n) return;
  T v[NARR];
#pragma unroll
  for (int k = 0; k < NARR; k++) v[k] = arr[k][e];
  f(v);
#pragma unroll
  for (int k = 0; k < NARR; k++)
    if (WMASK & (1u << k)) arr[k][e] = v[k];
}

template <typename T, int NARR, unsigned WMASK, typename F>
inline void launch_update(hipStream_t stream, long n, T* a0, T* a1, T* a2, T* a3, F f) {
  if (n <= 0) return;
  constexpr int N = Vec16<T>::N;
  T* arr[4] = {a0, a1, a2, a3};
  bool al = true;
  for (int k = 0; k < NARR; k++) al = al && aligned16(arr[k]);
  if (al) {
    const long nvec = n / N;
    long grid = (nvec + kEwBlock - 1) / kEwBlock;
    if (grid < 1) grid = 1;
    hipLaunchKernelGGL((ew_update_vec_kernel<T, NARR, WMASK, F>), dim3((unsigned)grid), dim3(kEwBlock), 0, stream, nvec, n, a0, a1, a2, a3, f);
  } else {
    const long grid = (n + kEwBlock - 1) / kEwBlock;
    hipLaunchKernelGGL((ew_update_scalar_kernel<T, NARR, WMASK, F>), dim3((unsigned)grid), dim3(kEwBlock), 0, stream, n, a0, a1, a2, a3, f);
  }
}

}  // namespace knet8
