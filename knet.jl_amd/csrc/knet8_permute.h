// N-d permutedims: y = permutedims(x, perm), column-major, y dims d[perm[0]], d[perm[1]], ...  The device side of
// `permutedims(B::KnetArray, perm)` / `permutedims!`, which the reference hands to CUDA.jl through a CuArray view
// (src/knetarrays/reshape.jl:18-29).  A pure data movement: 2*sizeof(T) bytes per element, bit-exact.
//
// The host reduces the problem first: dimensions of size 1 vanish and neighbouring dimensions of x that stay neighbours in the
// same order in y merge into one.  What remains is one of
//   * nothing to permute: one contiguous copy;
//   * the fastest dimension stays the fastest (`rows` kernel): whole runs of d0 elements move, read contiguously, as 16-byte
//     vectors when d0 and both addresses allow it;
//   * another dimension p becomes the fastest (`tile` kernel): TM x TN tiles of the (dim 0, dim p) plane go through LDS so that
//     reads run along dim 0 and writes along dim p, both contiguous; every other dimension is a batch index with its own stride
//     on either side.  The tile is 64x64 with 16-byte global accesses wherever alignment allows (reads matter: +30 %), or
//     16x256 / 4x1024 (and the mirror images) when one of the two dimensions is short; a plain batched 2-d transpose with a side
//     of at most 32 takes the chunked kernel of knet8_transpose.h instead.  Runs of 8 or 16 bytes that stay in place are moved
//     as single wide elements.
// transpose_S and permute213_S (softmax over a non-leading dimension, src/ops20_gpu/softmax.jl:19-20) are the same machinery.
#pragma once
#include "knet8_device.h"
#include "knet8_runtime.h"
#include "knet8_transpose.h"

namespace knet8 {

constexpr int kPermMaxDims = 8;

struct PermPlan {
  int m;                      // dimensions after collapsing, in x order
  int d[kPermMaxDims];        // sizes
  int sx[kPermMaxDims];       // element strides in x (contiguous: sx[0] = 1)
  int sy[kPermMaxDims];       // element stride in y of the same dimension
};

// Returns false (with `why`) if the arguments are not a permutation problem the kernels accept.
inline bool perm_plan(int nd, const int* dims, const int* perm, PermPlan& p, long& total, const char*& why) {
  if (nd < 1 || nd > kPermMaxDims) { why = "permutedims: 1 to 8 dimensions"; return false; }
  bool seen[kPermMaxDims] = {false};
  for (int i = 0; i < nd; i++) {
    if (perm[i] < 1 || perm[i] > nd || seen[perm[i] - 1]) { why = "permutedims: no valid permutation of dimensions"; return false; }
    seen[perm[i] - 1] = true;
    if (dims[i] < 0) { why = "permutedims: negative dimension"; return false; }
  }
  total = 1;
  for (int i = 0; i < nd; i++) {
    total *= dims[i];
    if (total >= (1L << 31)) { why = "permutedims: more than 2^31-1 elements"; return false; }   // checked as it grows: no overflow
  }
  long sxl[kPermMaxDims], syl[kPermMaxDims], ys = 1, xs = 1;
  for (int k = 0; k < nd; k++) { sxl[k] = xs; xs *= dims[k]; }
  for (int i = 0; i < nd; i++) { syl[perm[i] - 1] = ys; ys *= dims[perm[i] - 1]; }
  p.m = 0;
  for (int k = 0; k < nd; k++) {
    if (dims[k] == 1) continue;
    if (p.m > 0 && syl[k] == (long)p.sy[p.m - 1] * p.d[p.m - 1]) {   // follows its predecessor on both sides: one dimension
      p.d[p.m - 1] *= dims[k];
      continue;
    }
    p.d[p.m] = dims[k]; p.sx[p.m] = (int)sxl[k]; p.sy[p.m] = (int)syl[k];
    p.m++;
  }
  return true;
}

template <typename T, int NV> struct PermVec { typedef typename Vec16<T>::type type; };
template <typename T> struct PermVec<T, 1> { typedef T type; };

// Fastest dimension unchanged.  One lane moves one unit (NV elements of a run); `u0` units per run.
template <typename T, int NV>
__global__ __launch_bounds__(256) void permute_rows_kernel(PermPlan p, int u0, unsigned units, const T* __restrict__ x, T* __restrict__ y) {
  typedef typename PermVec<T, NV>::type V;
  const unsigned u = blockIdx.x * 256u + threadIdx.x;
  if (u >= units) return;
  unsigned rest = u / (unsigned)u0;
  const unsigned i0 = (u - rest * (unsigned)u0) * NV;
  unsigned yo = i0;
#pragma unroll
  for (int k = 1; k < kPermMaxDims; k++) {
    if (k < p.m) {
      const unsigned q = rest / (unsigned)p.d[k];
      yo += (rest - q * (unsigned)p.d[k]) * (unsigned)p.sy[k];
      rest = q;
    }
  }
  if (NV > 1) {
    const V v = ld_stream(reinterpret_cast<const V*>(x + (size_t)u * NV));
    st_stream(reinterpret_cast<V*>(y + yo), v);
  } else {
    y[yo] = __builtin_nontemporal_load(x + u);
  }
}

// Dimension P of x becomes the fastest of y.  Tile: TM elements along dim 0, TN along dim P; 256 lanes.
template <typename T, int TM, int TN>
__global__ __launch_bounds__(256) void permute_tile_kernel(PermPlan p, int P, unsigned tiles0, unsigned tilesp, const T* __restrict__ x, T* __restrict__ y) {
  __shared__ T tile[TN][TM + 1];
  unsigned b = blockIdx.x;
  const unsigned t0 = b % tiles0; b /= tiles0;
  const unsigned tp = b % tilesp; b /= tilesp;
  size_t xb = 0, yb = 0;       // offsets of this batch element (every dimension but 0 and P)
#pragma unroll
  for (int k = 1; k < kPermMaxDims; k++) {
    if (k < p.m && k != P) {
      const unsigned q = b / (unsigned)p.d[k];
      const unsigned r = b - q * (unsigned)p.d[k];
      xb += (size_t)r * p.sx[k];
      yb += (size_t)r * p.sy[k];
      b = q;
    }
  }
  const int d0 = p.d[0], dp = p.d[P];
  const size_t sxp = p.sx[P], sy0 = p.sy[0];
  constexpr int PASSES = TM * TN / 256;
#pragma unroll
  for (int q = 0; q < PASSES; q++) {          // lanes along dim 0: contiguous reads
    const int e = q * 256 + threadIdx.x;
    const int tx = e % TM, r = e / TM;
    const int i = t0 * TM + tx, j = tp * TN + r;
    if (i < d0 && j < dp) tile[r][tx] = __builtin_nontemporal_load(x + xb + i + j * sxp);
  }
  __syncthreads();
#pragma unroll
  for (int q = 0; q < PASSES; q++) {          // lanes along dim P: contiguous writes
    const int e = q * 256 + threadIdx.x;
    const int tx = e % TN, r = e / TN;
    const int j = tp * TN + tx, i = t0 * TM + r;
    if (i < d0 && j < dp) __builtin_nontemporal_store(tile[tx][r], y + yb + j + i * sy0);
  }
}

// The 64x64 tile with 16-byte global accesses on the side(s) that allow them (VR: reads along dim 0, VW: writes along dim P):
// NV elements per lane and access instead of one.  LDS holds scalars (pitch 65), so either side can be scalar or vector.
template <typename T, bool VR, bool VW>
__global__ __launch_bounds__(256) void permute_tile64_kernel(PermPlan p, int P, unsigned tiles0, unsigned tilesp, const T* __restrict__ x, T* __restrict__ y, bool diag) {
  constexpr int TS = 64, NV = Vec16<T>::N;
  typedef typename Vec16<T>::type V;
  __shared__ T tile[TS][TS + 1];
  // With `diag` tiles are numbered along a diagonal of the (dim 0, dim P) plane: workgroups that run at the same time then differ
  // in both coordinates, which keeps their reads AND their writes spread over the memory channels when a stride is a multiple of
  // 4 KB ((4096,8192) fp32 transpose, cold: 60 -> 49 us; without such strides the plain order is 5-10 % faster).
  unsigned b = blockIdx.x;
  const unsigned t0 = b % tiles0; b /= tiles0;
  const unsigned tp = (b % tilesp + (diag ? t0 : 0u)) % tilesp; b /= tilesp;
  size_t xb = 0, yb = 0;
#pragma unroll
  for (int k = 1; k < kPermMaxDims; k++) {
    if (k < p.m && k != P) {
      const unsigned q = b / (unsigned)p.d[k];
      const unsigned r = b - q * (unsigned)p.d[k];
      xb += (size_t)r * p.sx[k];
      yb += (size_t)r * p.sy[k];
      b = q;
    }
  }
  const int d0 = p.d[0], dp = p.d[P];
  const size_t sxp = p.sx[P], sy0 = p.sy[0];
  if (VR) {
    constexpr int LX = TS / NV;                    // lanes along dim 0
#pragma unroll
    for (int q = 0; q < TS * LX / 256; q++) {
      const int e = q * 256 + threadIdx.x;
      const int tx = (e % LX) * NV, r = e / LX;
      const int i = t0 * TS + tx, j = tp * TS + r;
      if (i < d0 && j < dp) {                      // d0 % NV == 0: a vector is inside or outside as a whole
        const V v = ld_stream(reinterpret_cast<const V*>(x + xb + i + j * sxp));
#pragma unroll
        for (int c = 0; c < NV; c++) tile[r][tx + c] = v[c];
      }
    }
  } else {
#pragma unroll
    for (int q = 0; q < TS * TS / 256; q++) {
      const int e = q * 256 + threadIdx.x;
      const int tx = e % TS, r = e / TS;
      const int i = t0 * TS + tx, j = tp * TS + r;
      if (i < d0 && j < dp) tile[r][tx] = __builtin_nontemporal_load(x + xb + i + j * sxp);
    }
  }
  __syncthreads();
  if (VW) {
    constexpr int LX = TS / NV;                    // lanes along dim P
#pragma unroll
    for (int q = 0; q < TS * LX / 256; q++) {
      const int e = q * 256 + threadIdx.x;
      const int tx = (e % LX) * NV, r = e / LX;
      const int j = tp * TS + tx, i = t0 * TS + r;
      if (i < d0 && j < dp) {
        V v;
#pragma unroll
        for (int c = 0; c < NV; c++) v[c] = tile[tx + c][r];
        st_stream(reinterpret_cast<V*>(y + yb + j + i * sy0), v);
      }
    }
  } else {
#pragma unroll
    for (int q = 0; q < TS * TS / 256; q++) {
      const int e = q * 256 + threadIdx.x;
      const int tx = e % TS, r = e / TS;
      const int j = tp * TS + tx, i = t0 * TS + r;
      if (i < d0 && j < dp) __builtin_nontemporal_store(tile[tx][r], y + yb + j + i * sy0);
    }
  }
}

// Runs the reduced problem `p` (strides and sizes in units of E) with the kernel its shape asks for.
template <typename E>
inline void perm_dispatch(hipStream_t stream, const PermPlan& p, long total, const E* x, E* y) {
  if (p.sy[0] == 1) {
    constexpr int N = sizeof(E) < 16 ? 16 / sizeof(E) : 1;
    bool vec = N > 1 && aligned16(x) && aligned16(y) && p.d[0] % N == 0;
    for (int k = 1; k < p.m && vec; k++) vec = p.sy[k] % N == 0;
    const int nv = vec ? N : 1;
    const int u0 = p.d[0] / nv;
    const unsigned units = (unsigned)(total / nv);
    const unsigned grid = (units + 255u) / 256u;
    if constexpr (N > 1) {
      if (vec) { hipLaunchKernelGGL((permute_rows_kernel<E, N>), dim3(grid), dim3(256), 0, stream, p, u0, units, x, y); return; }
    }
    hipLaunchKernelGGL((permute_rows_kernel<E, 1>), dim3(grid), dim3(256), 0, stream, p, u0, units, x, y);
    return;
  }
  int P = 1;
  while (P < p.m && p.sy[P] != 1) P++;
  if (P >= p.m) { record_error("permutedims: internal plan error"); return; }
  const int d0 = p.d[0], dp = p.d[P];
  const long batch = total / ((long)d0 * dp);
  if constexpr (sizeof(E) <= 8) {
    // a plain (batched) matrix transpose with a short side: whole chunks of columns or rows per workgroup
    const bool plain = P == 1 && (p.m == 2 || (p.m == 3 && p.sx[2] == d0 * dp && p.sy[2] == d0 * dp));
    const int small = d0 < dp ? d0 : dp, large = d0 < dp ? dp : d0;
    if (plain && small <= kTrSkinny && large > kTrTile) { launch_transpose_skinny<E>(stream, d0, dp, x, y, (int)batch); return; }
  }
#define KNET8_PERM_TILE(TM, TN) do { \
    const long t0 = (d0 + (TM) - 1) / (TM), tp = (dp + (TN) - 1) / (TN); \
    const long blocks = t0 * tp * batch; \
    if (blocks > 0x7fffffffL) { record_error("permutedims: too many tiles"); return; } \
    hipLaunchKernelGGL((permute_tile_kernel<E, TM, TN>), dim3((unsigned)blocks), dim3(256), 0, stream, p, P, (unsigned)t0, (unsigned)tp, x, y); \
  } while (0)
  if constexpr (sizeof(E) <= 8) {
    if (d0 <= 4 && dp > 64) KNET8_PERM_TILE(4, 1024);
    else if (d0 <= 16 && dp > 64) KNET8_PERM_TILE(16, 256);
    else if (dp <= 4 && d0 > 64) KNET8_PERM_TILE(1024, 4);
    else if (dp <= 16 && d0 > 64) KNET8_PERM_TILE(256, 16);
    else {
      // every stride of x but dim 0's is a multiple of d0, every stride of y but dim P's a multiple of dp: vectors stay aligned
      constexpr int N = 16 / sizeof(E);
      const bool vr = aligned16(x) && d0 % N == 0, vw = aligned16(y) && dp % N == 0;
      // strides of 4 KB multiples on either side alias the memory channels: number the tiles along a diagonal then
      const bool diag = ((size_t)p.sx[P] * sizeof(E)) % 4096 == 0 || ((size_t)p.sy[0] * sizeof(E)) % 4096 == 0;
      const long t0 = (d0 + 63) / 64, tp = (dp + 63) / 64;
      const long blocks = t0 * tp * batch;
      if (blocks > 0x7fffffffL) { record_error("permutedims: too many tiles"); return; }
#define KNET8_PERM_T64(VR, VW) hipLaunchKernelGGL((permute_tile64_kernel<E, VR, VW>), dim3((unsigned)blocks), dim3(256), 0, stream, p, P, (unsigned)t0, (unsigned)tp, x, y, diag)
      if (vr && vw) KNET8_PERM_T64(true, true); else if (vr) KNET8_PERM_T64(true, false); else if (vw) KNET8_PERM_T64(false, true); else KNET8_PERM_T64(false, false);
#undef KNET8_PERM_T64
    }
  } else {   // 16-byte units: a quarter of the elements per tile keeps the LDS footprint
    if (d0 <= 4 && dp > 32) KNET8_PERM_TILE(4, 256);
    else if (dp <= 4 && d0 > 32) KNET8_PERM_TILE(256, 4);
    else KNET8_PERM_TILE(32, 32);
  }
#undef KNET8_PERM_TILE
}

template <typename T>
inline void launch_permutedims(hipStream_t stream, int nd, const int* dims, const int* perm, const T* x, T* y) {
  PermPlan p;
  long total = 0;
  const char* why = nullptr;
  if (dims == nullptr || perm == nullptr) { record_error("permutedims: null dims or perm"); return; }
  if (!perm_plan(nd, dims, perm, p, total, why)) { record_error(why); return; }
  if (total == 0) return;
  if (p.m <= 1) {   // nothing moves
    if (hipMemcpyAsync(y, x, (size_t)total * sizeof(T), hipMemcpyDeviceToDevice, stream) != hipSuccess) record_error("permutedims: copy failed");
    return;
  }
  // A short fastest dimension that stays in place (runs of 8 or 16 bytes: pairs, quadruples) would be moved in pieces of that
  // size.  Seen as one wide element the run disappears from the problem and the next dimension takes its role, tiles and all.
  const size_t run = (size_t)p.d[0] * sizeof(T);
  if (p.sy[0] == 1 && p.m >= 3 && (run == 16 || (run == 8 && sizeof(T) < 8)) &&
      reinterpret_cast<uintptr_t>(x) % run == 0 && reinterpret_cast<uintptr_t>(y) % run == 0) {
    PermPlan q;
    q.m = p.m - 1;
    for (int k = 1; k < p.m; k++) { q.d[k - 1] = p.d[k]; q.sx[k - 1] = p.sx[k] / p.d[0]; q.sy[k - 1] = p.sy[k] / p.d[0]; }
    if (run == 16) {
      typedef typename Vec16<float>::type W;
      perm_dispatch<W>(stream, q, total / p.d[0], reinterpret_cast<const W*>(x), reinterpret_cast<W*>(y));
    } else {
      perm_dispatch<double>(stream, q, total / p.d[0], reinterpret_cast<const double*>(x), reinterpret_cast<double*>(y));
    }
    return;
  }
  perm_dispatch<T>(stream, p, total, x, y);
}

// y(n, m, batch) = permutedims(x(m, n, batch), (2, 1, 3)): the matrix transpose and its batched form.
template <typename T> inline void launch_transpose(hipStream_t stream, int m, int n, const T* x, T* y, int batch = 1) {
  if (m <= 0 || n <= 0 || batch <= 0) return;
  const int dims[3] = {m, n, batch}, perm[3] = {2, 1, 3};
  launch_permutedims<T>(stream, 3, dims, perm, x, y);
}

}  // namespace knet8
