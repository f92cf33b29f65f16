// Backward pass of one small dense layer y = f(W*x + b) in a single launch.  No libknet8 counterpart: the reference runs it as
// reluback (src/ops20_gpu/activation.jl:30-37), sum(dz;dims=2) (src/knetarrays/reduction.jl:21-77) and two gemm! calls
// (dW = dz*x', dx = W'*dz: src/knetarrays/linalg.jl:11-18,26-52) -- four dependent launches of a few microseconds each, which
// for the 784-64-10 MLP is most of the backward step.
//
// With dz = f'(y) .* dy formed on the fly while the tiles are loaded (relu: y > 0 ? dy : 0, the reluback of the reference), the
// workgroups of one grid split into two jobs: 32x32 tiles of dW = dz*x' (the tiles of the first block column also add up the rows
// of dz they walk: db) and 32x32 tiles of dx = W'*dz.  dz is never written.  Sums run in a fixed order: deterministic results;
// against the separate launches they differ only in the order of summation.
// Only for products the small-matrix GEMM would take (gemm_is_small); larger layers keep the separate launches.
#pragma once
#include "knet8_device.h"
#include "knet8_gemm_small.h"
#include "knet8_runtime.h"

namespace knet8 {

template <typename T>
__global__ __launch_bounds__(256) void dense_back_kernel(int act, int m, int n, int k, const T* __restrict__ W, const T* __restrict__ x,
                                                         const T* __restrict__ y, const T* __restrict__ dy, T* __restrict__ dW,
                                                         T* __restrict__ db, T* __restrict__ dx, int tiles_w, int tiles_w_m, int tiles_x_m) {
  constexpr int TS = kGsTile;
  __shared__ T As[TS][TS + 1];  // As[kk][i] = A(i0+i, k0+kk)
  __shared__ T Bs[TS][TS + 1];  // Bs[kk][j] = B(k0+kk, j0+j)
  const bool job_w = (int)blockIdx.x < tiles_w;
  // C (M x N) = A (M x K) * B (K x N):  job_w: dW (m x k) = dz (m x n) * x' (n x k);  else dx (k x n) = W' (k x m) * dz (m x n)
  const int M = job_w ? m : k, N = job_w ? k : n, K = job_w ? n : m;
  const int tile = job_w ? (int)blockIdx.x : (int)blockIdx.x - tiles_w;
  const int tm = job_w ? tiles_w_m : tiles_x_m;
  const int i0 = (tile % tm) * TS, j0 = (tile / tm) * TS;
  const int t = threadIdx.x, tx = t & 15, ty = t >> 4;
  const int lo = t & 31, hi = t >> 5;  // loader coordinates: `lo` runs along the contiguous axis of the operand
  auto dz_at = [&](int i, int j) -> T {   // dz(i, j), i < m, j < n
    const T g = dy[i + (long)j * m];
    if (act == 1) return y[i + (long)j * m] > T(0) ? g : T(0);
    return g;
  };
  T acc[2][2] = {{T(0), T(0)}, {T(0), T(0)}};
  T rowsum = T(0);
  const bool sums = job_w && j0 == 0 && db != nullptr;
  // global -> registers for kDepth k steps at once (zero outside the matrices): the inner dimension here is a batch size or a layer
  // width, usually at most 4*32, so that every load of the tile is in flight before the first multiply -- the arithmetic of a
  // step is far shorter than a memory round trip, a one-step lookahead would pay the latency once per step
  constexpr int kDepth = 4;
  T ga[kDepth][4], gb[kDepth][4];
  for (int kg = 0; kg < K; kg += kDepth * TS) {
#pragma unroll
    for (int s = 0; s < kDepth; s++) {
      const int k0 = kg + s * TS;
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const int h = hi + 8 * r;
        if (job_w) {
          { const int i = i0 + lo, kk = k0 + h; ga[s][r] = (i < m && kk < n) ? dz_at(i, kk) : T(0); }               // dz: contiguous along i
          { const int j = j0 + lo, kk = k0 + h; gb[s][r] = (j < k && kk < n) ? x[j + (long)kk * k] : T(0); }          // x' : x(j, kk), contiguous along j
        } else {
          { const int kk = k0 + lo, i = i0 + h; ga[s][r] = (i < k && kk < m) ? W[kk + (long)i * m] : T(0); }          // W' : W(kk, i), contiguous along kk
          { const int kk = k0 + lo, j = j0 + h; gb[s][r] = (j < n && kk < m) ? dz_at(kk, j) : T(0); }                 // dz: contiguous along kk
        }
      }
    }
#pragma unroll
    for (int s = 0; s < kDepth; s++) {
      if (kg + s * TS >= K) break;      // uniform across the workgroup
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const int h = hi + 8 * r;
        if (job_w) { As[h][lo] = ga[s][r]; Bs[h][lo] = gb[s][r]; }
        else       { As[lo][h] = ga[s][r]; Bs[lo][h] = gb[s][r]; }
      }
      __syncthreads();
      if (sums) {   // all 256 lanes: lane (i = t % 32, part = t / 32) adds the four kk of its part; parts meet at the end
#pragma unroll
        for (int q = 0; q < TS / 8; q++) rowsum = rowsum + As[hi * (TS / 8) + q][lo];   // zero beyond n: adds nothing
      }
#pragma unroll
      for (int kk = 0; kk < TS; kk++) {
        const T a0 = As[kk][tx], a1 = As[kk][tx + 16], b0 = Bs[kk][ty], b1 = Bs[kk][ty + 16];
        acc[0][0] = kfma(a0, b0, acc[0][0]); acc[1][0] = kfma(a1, b0, acc[1][0]); acc[0][1] = kfma(a0, b1, acc[0][1]); acc[1][1] = kfma(a1, b1, acc[1][1]);
      }
      __syncthreads();
    }
  }
  T* C = job_w ? dW : dx;
#pragma unroll
  for (int a = 0; a < 2; a++)
#pragma unroll
    for (int b = 0; b < 2; b++) {
      const int i = i0 + tx + 16 * a, j = j0 + ty + 16 * b;
      if (i < M && j < N) C[i + (long)j * M] = acc[a][b];
    }
  if (sums) {     // the eight parts of each row, in part order
    T* part = &Bs[0][0];
    part[hi * TS + lo] = rowsum;     // every lane is past its last read of Bs (barrier at the end of the loop)
    __syncthreads();
    if (t < TS && i0 + t < m) {
      T r = T(0);
#pragma unroll
      for (int q = 0; q < 8; q++) r = r + part[q * TS + t];
      db[i0 + t] = r;
    }
  }
}

// 0: done.  1: not applicable (a product too large for the small kernels, or db wanted without dW): nothing was launched and the
// caller takes the separate launches.  -1: bad arguments (recorded).
template <typename T>
inline int launch_dense_back(hipStream_t stream, int act, int m, int n, int k, const T* W, const T* x, const T* y, const T* dy, T* dW, T* db, T* dx) {
  if (act != 0 && act != 1) { record_error("dense_back: act must be 0 (none) or 1 (relu)"); return -1; }
  if (m <= 0 || n <= 0 || k <= 0) return 0;
  if (dy == nullptr || (act == 1 && y == nullptr) || (dW != nullptr && x == nullptr) || (dx != nullptr && W == nullptr)) {
    record_error("dense_back: missing operand");
    return -1;
  }
  if (!gemm_is_small(m, k, n) || !gemm_is_small(k, n, m) || (db != nullptr && dW == nullptr)) return 1;
  const int tw_m = (m + kGsTile - 1) / kGsTile, tw_n = (k + kGsTile - 1) / kGsTile;
  const int tx_m = (k + kGsTile - 1) / kGsTile, tx_n = (n + kGsTile - 1) / kGsTile;
  const int tiles_w = dW ? tw_m * tw_n : 0, tiles_x = dx ? tx_m * tx_n : 0;
  if (tiles_w + tiles_x == 0) return 0;
  hipLaunchKernelGGL((dense_back_kernel<T>), dim3((unsigned)(tiles_w + tiles_x)), dim3(256), 0, stream, act, m, n, k, W, x, y, dy, dW, db, dx,
                     tiles_w, tw_m, tx_m);
  return 0;
}

}  // namespace knet8
