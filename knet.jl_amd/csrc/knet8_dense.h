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

// Tile and workgroup shape: 16x16 outputs per tile on the matrix cores (v_mfma_*_16x16x4, operands straight from global memory as in
// gemm_mfma_kernel), four waves per workgroup, wave w taking the w-th slice of the inner dimension; the four partial tiles meet in
// LDS.  The inner dimension of either product is a batch size or a layer width: with at most 256 of it a wave has at most four
// 16-deep steps, all its loads in flight at once.
constexpr int kDbTile = 16, kDbWaves = 4;

template <typename T>
__global__ __launch_bounds__(kDbWaves * kWave) void dense_back_kernel(int act, int m, int n, int k, const T* __restrict__ W, const T* __restrict__ x,
                                                                      const T* __restrict__ y, const T* __restrict__ dy, T* __restrict__ dW,
                                                                      T* __restrict__ db, T* __restrict__ dx, int tiles_w, int tiles_w_m, int tiles_x_m,
                                                                      int kslice_w, int kslice_x, bool vecw, bool vecz) {
  constexpr int TS = kDbTile, KS = kDbWaves;
  __shared__ T part[KS][TS * TS];      // part[w][j*16 + i]
  __shared__ T rs[KS][4][TS];          // row-sum parts
  const bool job_w = (int)blockIdx.x < tiles_w;
  // C (M x N) = A (M x K) * B (K x N):  job_w: dW (m x k) = dz (m x n) * x' (n x k);  else dx (k x n) = W' (k x m) * dz (m x n)
  const int M = job_w ? m : k, N = job_w ? k : n, K = job_w ? n : m;
  const int tile = job_w ? (int)blockIdx.x : (int)blockIdx.x - tiles_w;
  const int tm = job_w ? tiles_w_m : tiles_x_m;
  const int kslice = job_w ? kslice_w : kslice_x;
  const int i0 = (tile % tm) * TS, j0 = (tile / tm) * TS;
  const int w = threadIdx.x / kWave, l = threadIdx.x & (kWave - 1);
  const int r16 = l & 15, kq = l >> 4;   // lane supplies A(i0 + r16, kk) and B(kk, j0 + r16) for kk = 4*kq .. 4*kq + 3 of each 16-deep step
  const int kbeg = w * kslice;
  int kend = kbeg + kslice;
  if (kend > K) kend = K;
  const int i = i0 + r16, j = j0 + r16;
  const bool iok = i < M, jok = j < N;
  const bool relu = act == 1;
  typename Mfma16<T>::Acc acc = {T(0), T(0), T(0), T(0)};
  T rowsum = T(0);
  const bool sums = job_w && j0 == 0 && db != nullptr;
  if (job_w) {
    // A(i, kk) = dz(i, kk) and B(kk, j) = x(j, kk): both contiguous along the tile edge
    const T* gp = dy + (iok ? i : 0);
    const T* yp = relu ? y + (iok ? i : 0) : nullptr;
    const T* xp = x + (jok ? j : 0);
#pragma unroll 2
    for (int kc = kbeg; kc < kend; kc += 16) {
      T a[4], b[4];
#pragma unroll
      for (int c = 0; c < 4; c++) {
        const int kk = kc + 4 * kq + c;
        const bool kok = kk < kend;
        T g = (iok && kok) ? gp[(long)kk * m] : T(0);
        if (relu && iok && kok) g = yp[(long)kk * m] > T(0) ? g : T(0);
        a[c] = g;
        b[c] = (jok && kok) ? xp[(long)kk * k] : T(0);
      }
      if (sums) rowsum = rowsum + ((a[0] + a[1]) + (a[2] + a[3]));   // zero beyond n: adds nothing
#pragma unroll
      for (int c = 0; c < 4; c++) acc = Mfma16<T>::run(a[c], b[c], acc);
    }
  } else {
    // A(i, kk) = W(kk, i) and B(kk, j) = dz(kk, j): both contiguous along the inner dimension
    const T* wp = W + (long)(iok ? i : 0) * m;
    const T* gp = dy + (long)(jok ? j : 0) * m;
    const T* yp = relu ? y + (long)(jok ? j : 0) * m : nullptr;
#pragma unroll 2
    for (int kc = kbeg; kc < kend; kc += 16) {
      T a[4], b[4];
      mfma_load4<T, true>(a, wp, 1, kc + 4 * kq, kend, iok, vecw);
      mfma_load4<T, true>(b, gp, 1, kc + 4 * kq, kend, jok, vecz);
      if (relu) {
        T yy[4];
        mfma_load4<T, true>(yy, yp, 1, kc + 4 * kq, kend, jok, vecz);
#pragma unroll
        for (int c = 0; c < 4; c++) b[c] = yy[c] > T(0) ? b[c] : T(0);   // masked-out lanes hold zeros in both
      }
#pragma unroll
      for (int c = 0; c < 4; c++) acc = Mfma16<T>::run(a[c], b[c], acc);
    }
  }
  // partial tiles into LDS, summed in wave order; row-sum parts likewise
#pragma unroll
  for (int r = 0; r < 4; r++) part[w][r16 * TS + Mfma16<T>::row(r, kq)] = acc[r];
  if (sums) rs[w][kq][r16] = rowsum;
  __syncthreads();
  T* C = job_w ? dW : dx;
  {
    const int o = threadIdx.x;   // 256 lanes, 256 outputs
    T sum = T(0);
#pragma unroll
    for (int q = 0; q < KS; q++) sum += part[q][o];
    const int oi = i0 + (o & (TS - 1)), oj = j0 + o / TS;
    if (oi < M && oj < N) C[oi + (long)oj * M] = sum;
  }
  if (sums && threadIdx.x < TS && i0 + (int)threadIdx.x < m) {
    T r = T(0);
#pragma unroll
    for (int q = 0; q < KS; q++)
#pragma unroll
      for (int pq = 0; pq < 4; pq++) r = r + rs[q][pq][threadIdx.x];
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
  // inner dimension per wave, in whole 16-deep steps
  auto slice = [](int K) { const int steps = (K + 15) / 16; return ((steps + kDbWaves - 1) / kDbWaves) * 16; };
  // 16-byte (fp64: 32-byte) loads along the inner dimension of dx = W'*dz need columns of W, dy and y that start on such a boundary
  const bool vecw = W != nullptr && mfma_vec_ok(W, m);
  const bool vecz = mfma_vec_ok(dy, m) && (act != 1 || mfma_vec_ok(y, m));
  hipLaunchKernelGGL((dense_back_kernel<T>), dim3((unsigned)(tiles_w + tiles_x)), dim3(kDbWaves * kWave), 0, stream, act, m, n, k, W, x, y, dy, dW, db, dx,
                     tiles_w, tw_m, tx_m, slice(n), slice(m), vecw, vecz);
  return 0;
}

}  // namespace knet8
