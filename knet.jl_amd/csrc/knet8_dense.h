// Backward pass of one small dense layer y = f(W*x + b) in a single launch.  No libknet8 counterpart: the reference runs it as
// reluback (src/ops20_gpu/activation.jl:30-37), sum(dz;dims=2) (src/knetarrays/reduction.jl:21-77) and two gemm! calls
// (dW = dz*x', dx = W'*dz: src/knetarrays/linalg.jl:11-18,26-52) -- four dependent launches of a few microseconds each, which
// for the 784-64-10 MLP is most of the backward step.
//
// With dz = f'(y) .* dy formed on the fly while the tiles are loaded (relu: y > 0 ? dy : 0, the reluback of the reference), the
// workgroups of one grid split into two jobs: 16x16 tiles of dW = dz*x' (the tiles of the first block column also add up the rows
// of dz they walk: db) and 16x16 tiles of dx = W'*dz.  dz is never written.  Sums run in a fixed order: deterministic results;
// against the separate launches they differ only in the order of summation.
// Only for layers of up to about 2.7e8 flop per product; larger ones keep the separate launches (the entry point returns 1).
//
// The output layer of a classifier (at most 16 classes) can take its dz from the loss instead: with the scores z = W*x + b and the
// labels, dz = scale * (softmax(z) - onehot(label)) per column is formed while the tiles are loaded -- a column's classes sit in the
// sixteen lanes that load it -- and the per-column loss -logsoftmax(z)[label] is written on the way (nll_logsoftmax_back_S of the
// reference-side chain nll -> logsoftmax -> getindex, src/ops20/loss.jl:37-41, folded into the layer's backward launch).
#pragma once
#include "knet8_device.h"
#include "knet8_gemm_small.h"
#include "knet8_runtime.h"
#include "knet8_softmax.h"

namespace knet8 {

// Tile and workgroup shape: 16x16 outputs per tile on the matrix cores (v_mfma_*_16x16x4, operands straight from global memory as in
// gemm_mfma_kernel), eight waves per workgroup, wave w taking the w-th slice of the inner dimension; the partial tiles meet in
// LDS.  The inner dimension of either product is a batch size or a layer width: with at most 256 of it a wave has at most two
// 16-deep steps, all its loads in flight at once (64x100x784 layer: 5.0 us with four waves, 3.9 us with eight).
constexpr int kDbTile = 16, kDbWaves = 8;

// All-reduce over the 16 lanes of a DPP row (lanes 16q .. 16q+15) by rotations within the row: four full-rate ALU operations, no LDS
// traffic (a shuffle through ds_bpermute costs a dependent LDS round trip per step, and the loss form below needs eight per column).
template <int N> __device__ __forceinline__ float row_ror(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x120 + N, 0xf, 0xf, false));
}
template <int N> __device__ __forceinline__ double row_ror(double v) {
  const long long b = __builtin_bit_cast(long long, v);
  const int lo = __builtin_amdgcn_update_dpp(0, (int)b, 0x120 + N, 0xf, 0xf, false);
  const int hi = __builtin_amdgcn_update_dpp(0, (int)(b >> 32), 0x120 + N, 0xf, 0xf, false);
  return __builtin_bit_cast(double, ((long long)hi << 32) | (unsigned int)lo);
}
template <typename T> __device__ __forceinline__ T row16_max(T v) {
  T o;
  o = row_ror<8>(v); v = v > o ? v : o;
  o = row_ror<4>(v); v = v > o ? v : o;
  o = row_ror<2>(v); v = v > o ? v : o;
  o = row_ror<1>(v); v = v > o ? v : o;
  return v;
}
template <typename T> __device__ __forceinline__ T row16_sum(T v) {
  v = v + row_ror<8>(v);
  v = v + row_ror<4>(v);
  v = v + row_ror<2>(v);
  v = v + row_ror<1>(v);
  return v;
}

// dz of one score for the loss form: e = exp(z - max) of the lane's score, sum the column's sum of them.  fp32 takes the hardware
// reciprocal (1 ulp) instead of the division sequence: 0.4 us of a 5 us kernel whose waves have nothing to hide ALU latency behind.
__device__ __forceinline__ float nll_rcp(float s) { return __builtin_amdgcn_rcpf(s); }
__device__ __forceinline__ double nll_rcp(double s) { return 1.0 / s; }
template <typename T>
__device__ __forceinline__ T nll_dz(T e, T sum, int lab, int cls, T scale) {
  if (lab == 0) return T(0);
  return ((cls + 1 == lab) ? -scale : T(0)) + e * (nll_rcp(sum) * scale);
}

// MODE 0: y and dy are the layer's output and its gradient.  MODE 1 (loss form): y holds the scores, dy is unused, dz comes from
// (labels, scale) and the per-column loss goes to `loss` (m <= 16: a column's classes fit one tile edge).  MODE 2 (head form): as 1, but
// the scores are not read: every workgroup first computes the scores of the columns it needs, z = W*x + bias, into LDS (all n
// columns for a tile of dW, its own sixteen for a tile of dx) -- the output layer's forward product rides in its backward launch.
template <typename T> struct DenseHead { static constexpr int kCols = 32768 / (int)sizeof(T) / kDbTile; };   // 32 KB of scores in LDS

template <typename T, int MODE>
__global__ __launch_bounds__(kDbWaves * kWave) void dense_back_kernel(int act, int m, int n, int k, const T* __restrict__ W, const T* __restrict__ x,
                                                                      const T* __restrict__ y, const T* __restrict__ dy, T* __restrict__ dW,
                                                                      T* __restrict__ db, T* __restrict__ dx, int tiles_w, int tiles_w_m, int tiles_x_m,
                                                                      int kslice_w, int kslice_x, bool vecw, bool vecz, const int* __restrict__ labels, T scale,
                                                                      T* __restrict__ loss, T* __restrict__ mean, const T* __restrict__ bias, T* __restrict__ zout) {
  constexpr int TS = kDbTile, KS = kDbWaves;
  constexpr bool NLL = MODE >= 1, HEAD = MODE == 2;
  __shared__ T zs[HEAD ? DenseHead<T>::kCols * TS : 1];   // zs[column * 16 + class]
  __shared__ T part[KS][TS * TS];      // part[w][j*16 + i]
  __shared__ T rs[KS][4][TS];          // row-sum parts
  __shared__ T ls[KS];                 // loss parts
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
  T rowsum = T(0), lacc = T(0);
  const bool first = job_w && j0 == 0;          // the tiles that walk all of dz once: row sums and, in the loss form, the losses
  const bool sums = first && db != nullptr;
  const T ninf = T(-INFINITY);
  // Head form: the scores of the columns this workgroup needs, into LDS.  Called once by every wave (it contains a barrier), after the
  // loads of the second phase that do not depend on the scores have been issued, so that the two memory round trips overlap.
  auto compute_scores = [&]() {
    const int c0 = job_w ? 0 : j0;
    const int c1 = job_w ? n : (j0 + TS < n ? j0 + TS : n);
    const bool rok = r16 < m;                       // lane's class row of W
    for (int t = w; 16 * t < c1 - c0; t += KS) {   // one wave per tile of sixteen columns
      const int col = c0 + 16 * t + r16;
      const bool cok = col < c1;
      const T* wp = W + (rok ? r16 : 0);
      const T* xp = x + (long)(cok ? col : 0) * k;
      typename Mfma16<T>::Acc za = {T(0), T(0), T(0), T(0)};
#pragma unroll 4
      for (int kc = 0; kc < k; kc += 16) {
        T a[4], b[4];
        mfma_load4<T, false>(a, wp, m, kc + 4 * kq, k, rok, false);   // W(class, kk): contiguous along the classes
        mfma_load4<T, true>(b, xp, 1, kc + 4 * kq, k, cok, vecz);     // x(kk, col): contiguous along kk
#pragma unroll
        for (int c = 0; c < 4; c++) za = Mfma16<T>::run(a[c], b[c], za);
      }
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const int row = Mfma16<T>::row(r, kq);
        zs[(16 * t + r16) * TS + row] = (row < m && cok) ? za[r] + bias[row] : ninf;
      }
    }
    __syncthreads();
    if (first && zout != nullptr)
      for (long o = threadIdx.x; o < (long)m * n; o += KS * kWave) zout[o] = zs[(o / m) * TS + (o % m)];
  };
  if (job_w) {
    // A(i, kk) = dz(i, kk) and B(kk, j) = x(j, kk): both contiguous along the tile edge
    const T* gp = NLL ? nullptr : dy + (iok ? i : 0);
    const T* yp = relu ? y + (iok ? i : 0) : nullptr;
    const T* xp = x + (jok ? j : 0);
    if (NLL) {
      // Loads first, for the step after the current one: the losses' stores and the label lanes' branch would otherwise sit between
      // one column's loads and the next's, and a wave would pay a memory round trip per column instead of one per slice.
      constexpr int CH = 2, NC = 4 * CH;   // 16-deep steps per fetch: a slice of up to 32 columns is one memory round trip
      T zn[NC], xn[NC];
      int ln[NC];
      auto col = [&](int kc, int c) { return kc + 16 * (c / 4) + 4 * kq + (c & 3); };
      auto fetch = [&](int kc) {
#pragma unroll
        for (int c = 0; c < NC; c++) {
          const int kk = col(kc, c);
          const bool kok = kk < kend;
          if (HEAD) zn[c] = (iok && kok) ? zs[kk * TS + i] : ninf;
          else zn[c] = (iok && kok) ? y[i + (long)kk * m] : ninf;
          ln[c] = kok ? labels[kk] : 0;
          xn[c] = (jok && kok) ? xp[(long)kk * k] : T(0);
        }
      };
      if (HEAD) {   // labels and x of the first step first, the scores' product behind them, then the scores from LDS
#pragma unroll
        for (int c = 0; c < NC; c++) {
          const int kk = col(kbeg, c);
          const bool kok = kk < kend;
          ln[c] = kok ? labels[kk] : 0;
          xn[c] = (jok && kok) ? xp[(long)kk * k] : T(0);
        }
        compute_scores();
#pragma unroll
        for (int c = 0; c < NC; c++) {
          const int kk = col(kbeg, c);
          zn[c] = (iok && kk < kend) ? zs[kk * TS + i] : ninf;
        }
      } else {
        fetch(kbeg);
      }
      for (int kc = kbeg; kc < kend; kc += 16 * CH) {
        T z[NC], a[NC], b[NC], lj[NC];
        int lab[NC];
#pragma unroll
        for (int c = 0; c < NC; c++) { z[c] = zn[c]; lab[c] = ln[c]; b[c] = xn[c]; }
        if (kc + 16 * CH < kend) fetch(kc + 16 * CH);
#pragma unroll
        for (int c = 0; c < NC; c++) {
          // lanes r16 = 0..15 of this quarter hold the classes of column kk: max and sum over the row
          const bool kok = col(kc, c) < kend;
          const T mx = row16_max(z[c]);
          const T e = dev_exp(z[c] - (mx == ninf ? T(0) : mx));
          const T sum = row16_sum(e);
          if (lab[c] < 0 || lab[c] > m) lab[c] = 0;   // as nll_logsoftmax_back_S: an out-of-range label is skipped, never dereferenced
          a[c] = (iok && kok) ? nll_dz(e, sum, lab[c], i, scale) : T(0);
          lj[c] = -((z[c] - mx) - dev_log(sum));
        }
        if (first) {
#pragma unroll
          for (int c = 0; c < NC; c++) {
            const int kk = col(kc, c);
            if (kk < kend) {
              if (lab[c] > 0 && i + 1 == lab[c]) {
                lacc = lacc + lj[c];
                if (loss != nullptr) loss[kk] = lj[c];
              }
              if (lab[c] == 0 && r16 == 0 && loss != nullptr) loss[kk] = T(0);
            }
          }
        }
#pragma unroll
        for (int h = 0; h < CH; h++)
          if (sums) rowsum = rowsum + ((a[4 * h] + a[4 * h + 1]) + (a[4 * h + 2] + a[4 * h + 3]));
#pragma unroll
        for (int c = 0; c < NC; c++) acc = Mfma16<T>::run(a[c], b[c], acc);
      }
    } else {
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
    }
  } else {
    // A(i, kk) = W(kk, i) and B(kk, j) = dz(kk, j): both contiguous along the inner dimension
    const T* wp = W + (long)(iok ? i : 0) * m;
    const T* gp = HEAD ? nullptr : (NLL ? y : dy) + (long)(jok ? j : 0) * m;
    const T* yp = relu ? y + (long)(jok ? j : 0) * m : nullptr;
    if (HEAD) compute_scores();   // every wave, also those whose slice of the (short) inner dimension is empty
#pragma unroll 2
    for (int kc = kbeg; kc < kend; kc += 16) {
      T a[4], b[4];
      mfma_load4<T, true>(a, wp, 1, kc + 4 * kq, kend, iok, vecw);
      if (HEAD) {
#pragma unroll
        for (int c = 0; c < 4; c++) b[c] = (jok && kc + 4 * kq + c < kend) ? zs[r16 * TS + kc + 4 * kq + c] : T(0);
      } else {
        mfma_load4<T, true>(b, gp, 1, kc + 4 * kq, kend, jok, vecz);
      }
      if (NLL) {
        // m <= 16: this one step holds every class of column j, four per lane in the lanes j, j+16, j+32, j+48
        T z[4], mx = ninf;
#pragma unroll
        for (int c = 0; c < 4; c++) { z[c] = (jok && kc + 4 * kq + c < kend) ? b[c] : ninf; mx = mx > z[c] ? mx : z[c]; }
#pragma unroll
        for (int off = 16; off < kWave; off <<= 1) { const T o = __shfl_xor(mx, off, kWave); mx = mx > o ? mx : o; }
        T e[4], sum = T(0);
#pragma unroll
        for (int c = 0; c < 4; c++) { e[c] = dev_exp(z[c] - (mx == ninf ? T(0) : mx)); sum = sum + e[c]; }
#pragma unroll
        for (int off = 16; off < kWave; off <<= 1) sum = sum + __shfl_xor(sum, off, kWave);
        int lab = jok ? labels[j] : 0;
        if (lab < 0 || lab > m) lab = 0;
#pragma unroll
        for (int c = 0; c < 4; c++) b[c] = (jok && kc + 4 * kq + c < kend) ? nll_dz(e[c], sum, lab, kc + 4 * kq + c, scale) : T(0);
      }
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
  if (NLL && first && mean != nullptr) {   // wave butterfly, then the waves in order: a fixed summation tree
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) lacc = lacc + __shfl_xor(lacc, off, kWave);
    if (l == 0) ls[w] = lacc;
  }
  __syncthreads();
  if (NLL && first && mean != nullptr && threadIdx.x == 0) {
    T tot = T(0);
#pragma unroll
    for (int q = 0; q < KS; q++) tot = tot + ls[q];
    *mean = tot * scale;
  }
  T* C = job_w ? dW : dx;
  {
    const int o = threadIdx.x;   // one lane per output
    if (o < TS * TS) {
      T sum = T(0);
#pragma unroll
      for (int q = 0; q < KS; q++) sum += part[q][o];
      const int oi = i0 + (o & (TS - 1)), oj = j0 + o / TS;
      if (oi < M && oj < N) C[oi + (long)oj * M] = sum;
    }
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
template <typename T, int MODE>
inline int launch_dense_back_impl(hipStream_t stream, int act, int m, int n, int k, const T* W, const T* x, const T* y, const T* dy, T* dW, T* db, T* dx,
                                  const int* labels, T scale, T* loss, T* mean, const T* bias = nullptr, T* zout = nullptr) {
  constexpr bool NLL = MODE >= 1;
  // both products have 2*m*n*k flop; kernel durations against reluback_biasgrad + two gemm launches (us, kernel trace): 64x100x784
  // 3.6/11.3, 256^3 5.2/12.6, 300^3 7.3/14.8, 512x128x512 9.6/14.1, 400^3 11.9/18.8, 512^3 20.8/26.2 -- one launch wins over the whole range of
  // the small-product kernels (2.7e8 flop); beyond it the separate launches reach the vendor library's large tiles
  if (2.0 * m * n * (double)k > 1.0e6 * tuning(kTuneDenseBackMflop) || (db != nullptr && dW == nullptr)) return 1;
  const int tw_m = (m + kDbTile - 1) / kDbTile, tw_n = (k + kDbTile - 1) / kDbTile;
  const int tx_m = (k + kDbTile - 1) / kDbTile, tx_n = (n + kDbTile - 1) / kDbTile;
  const int tiles_w = dW ? tw_m * tw_n : 0, tiles_x = dx ? tx_m * tx_n : 0;
  if (tiles_w + tiles_x == 0) return 0;
  // inner dimension per wave, in whole 16-deep steps
  auto slice = [](int K) { const int steps = (K + 15) / 16; return ((steps + kDbWaves - 1) / kDbWaves) * 16; };
  // 16-byte (fp64: 32-byte) loads along the inner dimension of dx = W'*dz need columns of W, dy and y that start on such a boundary
  const bool vecw = W != nullptr && mfma_vec_ok(W, m);
  // (head form: the flag covers the loads of x along its inner dimension instead)
  const bool vecz = MODE == 2 ? mfma_vec_ok(x, k) : NLL ? mfma_vec_ok(y, m) : (mfma_vec_ok(dy, m) && (act != 1 || mfma_vec_ok(y, m)));
  hipLaunchKernelGGL((dense_back_kernel<T, MODE>), dim3((unsigned)(tiles_w + tiles_x)), dim3(kDbWaves * kWave), 0, stream, act, m, n, k, W, x, y, dy, dW, db, dx,
                     tiles_w, tw_m, tx_m, slice(n), slice(m), vecw, vecz, labels, scale, loss, mean, bias, zout);
  return 0;
}

template <typename T>
inline int launch_dense_back(hipStream_t stream, int act, int m, int n, int k, const T* W, const T* x, const T* y, const T* dy, T* dW, T* db, T* dx) {
  if (act != 0 && act != 1) { record_error("dense_back: act must be 0 (none) or 1 (relu)"); return -1; }
  if (m <= 0 || n <= 0 || k <= 0) return 0;
  if (dy == nullptr || (act == 1 && y == nullptr) || (dW != nullptr && x == nullptr) || (dx != nullptr && W == nullptr)) {
    record_error("dense_back: missing operand");
    return -1;
  }
  return launch_dense_back_impl<T, 0>(stream, act, m, n, k, W, x, y, dy, dW, db, dx, nullptr, T(0), nullptr, nullptr);
}

// The classifier's output layer: scores z = W*x + b (m classes x n instances) and labels in, the loss per instance and the layer's
// gradients out (mean = scale * sum of the losses).  At most 16 classes; the losses are written only when dW is asked for (the tiles of dW are the ones that see all of dz).
template <typename T>
inline int launch_dense_nll_back(hipStream_t stream, int m, int n, int k, const T* W, const T* x, const T* z, const int* labels, T scale, T* dW, T* db,
                                 T* dx, T* loss, T* mean) {
  if (m <= 0 || n <= 0 || k <= 0) return 0;
  if (z == nullptr || labels == nullptr || (dW != nullptr && x == nullptr) || (dx != nullptr && W == nullptr)) {
    record_error("dense_nll_back: missing operand");
    return -1;
  }
  if (m > kDbTile || ((loss != nullptr || mean != nullptr) && dW == nullptr)) return 1;
  return launch_dense_back_impl<T, 1>(stream, 0, m, n, k, W, x, z, nullptr, dW, db, dx, labels, scale, loss, mean);
}

// The head form: forward product included.  W (m x k), bias (m), x (k x n) in; the scores themselves are written to z when asked for.
// At most 16 classes and DenseHead<T>::kCols instances (512 in fp32, 256 in fp64: their scores stay in LDS); dW is required.
template <typename T>
inline int launch_dense_head(hipStream_t stream, int m, int n, int k, const T* W, const T* bias, const T* x, const int* labels, T scale, T* dW, T* db,
                             T* dx, T* loss, T* mean, T* z) {
  if (m <= 0 || n <= 0 || k <= 0) return 0;
  if (W == nullptr || bias == nullptr || x == nullptr || labels == nullptr) {
    record_error("dense_head: missing operand");
    return -1;
  }
  if (m > kDbTile || n > DenseHead<T>::kCols || dW == nullptr) return 1;
  return launch_dense_back_impl<T, 2>(stream, 0, m, n, k, W, x, nullptr, nullptr, dW, db, dx, labels, scale, loss, mean, bias, z);
}

}  // namespace knet8
