// Backward pass of one small dense layer y = f(W*x + b) in a single launch.  No libknet8 counterpart: the reference runs it as
// reluback (src/ops20_gpu/activation.jl:30-37), sum(dz;dims=2) (src/knetarrays/reduction.jl:21-77) and two gemm! calls
// (dW = dz*x', dx = W'*dz: src/knetarrays/linalg.jl:11-18,26-52) -- four dependent launches of a few microseconds each, which
// for the 784-64-10 MLP is most of the backward step.
//
// With dz = f'(y) .* dy formed on the fly while the tiles are loaded (relu: y > 0 ? dy : 0, the reluback of the reference), the
// workgroups of one grid split into two jobs: 16x16 tiles of dW = dz*x' (the tiles of the first block column also add up the rows
// of dz they walk: db) and 16x16 tiles of dx = W'*dz.  dz is never written.  Sums run in a fixed order: deterministic results;
// against the separate launches they differ only in the order of summation.
// Only for layers of up to about 6e7 flop per product; larger ones keep the separate launches (the entry point returns 1).
#pragma once
#include "knet8_device.h"
#include "knet8_gemm_small.h"
#include "knet8_runtime.h"

namespace knet8 {

// Tile and workgroup shape: 16x16 outputs per tile, four waves per workgroup, wave w taking the w-th slice of the inner dimension
// (2x2 outputs per lane); the four partial tiles meet in LDS.  The inner dimension of either product is a batch size or a layer
// width: with at most 128 of it every wave runs a single 32-deep step, all its loads in flight at once.
constexpr int kDbTile = 16, kDbWaves = 4;

template <typename T>
__global__ __launch_bounds__(kDbWaves * kWave) void dense_back_kernel(int act, int m, int n, int k, const T* __restrict__ W, const T* __restrict__ x,
                                                                      const T* __restrict__ y, const T* __restrict__ dy, T* __restrict__ dW,
                                                                      T* __restrict__ db, T* __restrict__ dx, int tiles_w, int tiles_w_m, int tiles_x_m,
                                                                      int kslice_w, int kslice_x) {
  constexpr int TS = kDbTile, KT = kGsTile, KS = kDbWaves;
  constexpr int R = TS * KT / kWave;   // operand elements a lane stages per step (8)
  __shared__ T As[KS][KT][TS + 1];     // As[w][kk][i] = A(i0+i, k0+kk) of wave w's current step
  __shared__ T Bs[KS][KT][TS + 1];     // Bs[w][kk][j] = B(k0+kk, j0+j)
  __shared__ T rs[KS][4][TS];          // row-sum parts
  const bool job_w = (int)blockIdx.x < tiles_w;
  // C (M x N) = A (M x K) * B (K x N):  job_w: dW (m x k) = dz (m x n) * x' (n x k);  else dx (k x n) = W' (k x m) * dz (m x n)
  const int M = job_w ? m : k, N = job_w ? k : n, K = job_w ? n : m;
  const int tile = job_w ? (int)blockIdx.x : (int)blockIdx.x - tiles_w;
  const int tm = job_w ? tiles_w_m : tiles_x_m;
  const int kslice = job_w ? kslice_w : kslice_x;
  const int i0 = (tile % tm) * TS, j0 = (tile / tm) * TS;
  const int w = threadIdx.x / kWave, l = threadIdx.x & (kWave - 1);
  const int tx = l & 7, ty = l >> 3;                      // outputs (tx + 8a, ty + 8b), a, b = 0..1
  const int lo_t = l & (TS - 1), hi_t = l / TS;           // operand contiguous along the tile edge: kk = hi_t + 4r
  const int lo_k = l & (KT - 1), hi_k = l / KT;           // operand contiguous along the inner dimension: edge index = hi_k + 2r
  const int kbeg = w * kslice;
  int kend = kbeg + kslice;
  if (kend > K) kend = K;
  auto dz_at = [&](int i, int j) -> T {   // dz(i, j), i < m, j < n
    const T g = dy[i + (long)j * m];
    if (act == 1) return y[i + (long)j * m] > T(0) ? g : T(0);
    return g;
  };
  T acc[2][2] = {{T(0), T(0)}, {T(0), T(0)}};
  T rowsum = T(0);
  const bool sums = job_w && j0 == 0 && db != nullptr;
  T ga[R], gb[R];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int r = 0; r < R; r++) {
      if (job_w) {
        { const int i = i0 + lo_t, kk = k0 + hi_t + (kWave / TS) * r; ga[r] = (i < m && kk < kend) ? dz_at(i, kk) : T(0); }          // dz(i, kk): contiguous along i
        { const int j = j0 + lo_t, kk = k0 + hi_t + (kWave / TS) * r; gb[r] = (j < k && kk < kend) ? x[j + (long)kk * k] : T(0); }     // x'(kk, j) = x(j, kk): along j
      } else {
        { const int kk = k0 + lo_k, i = i0 + hi_k + (kWave / KT) * r; ga[r] = (i < k && kk < kend) ? W[kk + (long)i * m] : T(0); }     // W'(i, kk) = W(kk, i): along kk
        { const int kk = k0 + lo_k, j = j0 + hi_k + (kWave / KT) * r; gb[r] = (j < n && kk < kend) ? dz_at(kk, j) : T(0); }            // dz(kk, j): along kk
      }
    }
  };
  fetch(kbeg);
  for (int k0 = kbeg; k0 < kbeg + kslice; k0 += KT) {     // every wave runs the same number of steps: the barriers line up
#pragma unroll
    for (int r = 0; r < R; r++) {
      if (job_w) { As[w][hi_t + (kWave / TS) * r][lo_t] = ga[r]; Bs[w][hi_t + (kWave / TS) * r][lo_t] = gb[r]; }
      else       { As[w][lo_k][hi_k + (kWave / KT) * r] = ga[r]; Bs[w][lo_k][hi_k + (kWave / KT) * r] = gb[r]; }
    }
    __syncthreads();
    if (k0 + KT < kbeg + kslice) fetch(k0 + KT);
    if (sums) {   // lane (i = l % 16, part = l / 16) adds the eight kk of its part of this wave's slice (zero beyond n: adds nothing)
#pragma unroll
      for (int q = 0; q < KT / 4; q++) rowsum = rowsum + As[w][hi_t * (KT / 4) + q][lo_t];
    }
#pragma unroll 8
    for (int kk = 0; kk < KT; kk++) {
      const T a0 = As[w][kk][tx], a1 = As[w][kk][tx + 8], b0 = Bs[w][kk][ty], b1 = Bs[w][kk][ty + 8];
      acc[0][0] = kfma(a0, b0, acc[0][0]); acc[1][0] = kfma(a1, b0, acc[1][0]); acc[0][1] = kfma(a0, b1, acc[0][1]); acc[1][1] = kfma(a1, b1, acc[1][1]);
    }
    __syncthreads();
  }
  // partial tiles into LDS (each wave reuses its own staging area), summed in wave order; row-sum parts likewise
  T* mine = &As[w][0][0];
#pragma unroll
  for (int a = 0; a < 2; a++)
#pragma unroll
    for (int b = 0; b < 2; b++) mine[(ty + 8 * b) * TS + tx + 8 * a] = acc[a][b];
  if (sums) rs[w][hi_t][lo_t] = rowsum;
  __syncthreads();
  T* C = job_w ? dW : dx;
  {
    const int o = threadIdx.x;   // 256 lanes, 256 outputs
    T sum = T(0);
#pragma unroll
    for (int q = 0; q < KS; q++) sum += (&As[q][0][0])[o];
    const int i = i0 + (o & (TS - 1)), j = j0 + o / TS;
    if (i < M && j < N) C[i + (long)j * M] = sum;
  }
  if (sums && threadIdx.x < TS && i0 + (int)threadIdx.x < m) {
    T r = T(0);
#pragma unroll
    for (int q = 0; q < KS; q++)
#pragma unroll
      for (int part = 0; part < 4; part++) r = r + rs[q][part][threadIdx.x];
    db[i0 + threadIdx.x] = r;
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
  // both products have 2*m*n*k flop; measured against reluback_biasgrad + two gemm launches (us): 64x100x784 5.6/14.5, 256^3 8.4/14.5,
  // 300^3 12.5/21.6, 512x128x512 16.4/16.2, 512^3 32.5/27.4 -- one launch wins up to about 6e7 flop
  if (2.0 * m * n * (double)k > 6.0e7 || (long)m * k > 262144 || (long)k * n > 262144 || (db != nullptr && dW == nullptr)) return 1;
  const int tw_m = (m + kDbTile - 1) / kDbTile, tw_n = (k + kDbTile - 1) / kDbTile;
  const int tx_m = (k + kDbTile - 1) / kDbTile, tx_n = (n + kDbTile - 1) / kDbTile;
  const int tiles_w = dW ? tw_m * tw_n : 0, tiles_x = dx ? tx_m * tx_n : 0;
  if (tiles_w + tiles_x == 0) return 0;
  // inner dimension per wave, in whole 32-deep steps
  auto slice = [](int K) { const int steps = (K + kGsTile - 1) / kGsTile; return ((steps + kDbWaves - 1) / kDbWaves) * kGsTile; };
  hipLaunchKernelGGL((dense_back_kernel<T>), dim3((unsigned)(tiles_w + tiles_x)), dim3(kDbWaves * kWave), 0, stream, act, m, n, k, W, x, y, dy, dW, db, dx,
                     tiles_w, tw_m, tx_m, slice(n), slice(m));
  return 0;
}

}  // namespace knet8
