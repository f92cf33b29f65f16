// Small-matrix GEMM C = alpha*op(A)*op(B) + beta*C (column-major), for products far too small to fill the
// machine -- the 64x100x784-class products of the MNIST MLP, where the vendor library needs 15-25 us per call.  Large products
// go to hipBLASLt (knet8_runtime.hip).  At this size a product's time is one launch (3.2 us for an empty kernel), one memory round
// trip and a few 32-deep tile steps: what matters is how many steps run one after the other and whether partial results have to
// leave the workgroup.  Three kernels, chosen in launch_gemm_small:
//   * gemm_wave_kernel<.., KS, 16>: 16x16 output tile per workgroup, one wave per k slice (KS = 1..16 slices), partial tiles summed
//     in LDS -- everything up to about 7e7 flop;
//   * gemm_wave_kernel<.., KS, 32>: the same with 32x32 tiles (4x4 outputs per lane) for the upper end of the range, when there are
//     at least 16 such tiles;
//   * gemm_small_kernel: 32x32 tile per 256-lane workgroup, k split over P workgroups per tile whose partial tiles are combined, in
//     fixed order, by the last one to finish (write-through + ticket, as in the reductions) -- few tiles with a very long k.
// All three add the bias and apply relu in their output stage when asked (gemm_bias_act_S): same bits as separate launches.
#pragma once
#include "knet8_device.h"
#include "knet8_runtime.h"

namespace knet8 {

constexpr int kGsTile = 32;
// The library is built with -ffp-contract=off for the elementwise contracts; a matrix product wants the fused form.
__device__ __forceinline__ float kfma(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
__device__ __forceinline__ double kfma(double a, double b, double c) { return __builtin_fma(a, b, c); }

// Output stage shared by the kernels below: v = alpha*acc [+ beta*C] [+ bias[i]] [relu].  Each step is one rounded operation, so
// a product with bias and relu folded in gives the bits of the product followed by the separate bias-add and relu launches.
template <typename T>
__device__ __forceinline__ void gemm_store(T* c, T acc, T alpha, T beta, const T* bias, int i, int act) {
  T v = alpha * acc;
  if (beta != T(0)) v = v + beta * *c;
  if (bias) v = v + bias[i];
  if (act == 1) v = v != v ? v : (v > T(0) ? v : T(0));
  *c = v;
}

template <typename T, bool TA, bool TB>
__global__ __launch_bounds__(256) void gemm_small_kernel(int m, int n, int k, T alpha, const T* __restrict__ A, int lda,
                                                         const T* __restrict__ B, int ldb, T beta, T* C, int ldc, const T* bias, int act,
                                                         int kchunk, unsigned P, T* partial, unsigned* counters) {
  __shared__ T As[kGsTile][kGsTile + 1];  // As[kk][i] = op(A)(i0+i, k0+kk)
  __shared__ T Bs[kGsTile][kGsTile + 1];  // Bs[kk][j] = op(B)(k0+kk, j0+j)
  __shared__ unsigned flag;
  const int tiles_m = (m + kGsTile - 1) / kGsTile;
  const unsigned tile = blockIdx.x / P, p = blockIdx.x % P;
  const int i0 = (int)(tile % tiles_m) * kGsTile, j0 = (int)(tile / tiles_m) * kGsTile;
  const int t = threadIdx.x, tx = t & 15, ty = t >> 4;
  const int lo = t & 31, hi = t >> 5;  // loader coordinates: `lo` runs along the contiguous axis of the operand
  const int kbeg = (int)p * kchunk;
  int kend = kbeg + kchunk;
  if (kend > k) kend = k;
  T acc[2][2] = {{T(0), T(0)}, {T(0), T(0)}};
  // global -> registers for one k step (zero outside the matrices); `lo` runs along the operand's contiguous axis
  T ga[4], gb[4];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int r = 0; r < 4; r++) {
      const int h = hi + 8 * r;
      if (!TA) { const int i = i0 + lo, kk = k0 + h; ga[r] = (i < m && kk < kend) ? A[i + (long)kk * lda] : T(0); }
      else     { const int kk = k0 + lo, i = i0 + h; ga[r] = (i < m && kk < kend) ? A[kk + (long)i * lda] : T(0); }
      if (!TB) { const int kk = k0 + lo, j = j0 + h; gb[r] = (j < n && kk < kend) ? B[kk + (long)j * ldb] : T(0); }
      else     { const int j = j0 + lo, kk = k0 + h; gb[r] = (j < n && kk < kend) ? B[j + (long)kk * ldb] : T(0); }
    }
  };
  if (kbeg < kend) fetch(kbeg);
  for (int k0 = kbeg; k0 < kend; k0 += kGsTile) {
#pragma unroll
    for (int r = 0; r < 4; r++) {
      const int h = hi + 8 * r;
      if (!TA) As[h][lo] = ga[r]; else As[lo][h] = ga[r];
      if (!TB) Bs[lo][h] = gb[r]; else Bs[h][lo] = gb[r];
    }
    __syncthreads();
    if (k0 + kGsTile < kend) fetch(k0 + kGsTile);  // next step's loads fly while this one is multiplied
#pragma unroll
    for (int kk = 0; kk < kGsTile; kk++) {
      const T a0 = As[kk][tx], a1 = As[kk][tx + 16], b0 = Bs[kk][ty], b1 = Bs[kk][ty + 16];
      acc[0][0] = kfma(a0, b0, acc[0][0]); acc[1][0] = kfma(a1, b0, acc[1][0]); acc[0][1] = kfma(a0, b1, acc[0][1]); acc[1][1] = kfma(a1, b1, acc[1][1]);
    }
    __syncthreads();
  }
  if (P > 1) {
    T* mine = partial + ((size_t)tile * P + p) * (kGsTile * kGsTile);
#pragma unroll
    for (int a = 0; a < 2; a++)
#pragma unroll
      for (int b = 0; b < 2; b++) st_coherent(mine + (ty + 16 * b) * kGsTile + tx + 16 * a, acc[a][b]);
    if (!last_block_ticket(counters + tile, P, &flag)) return;
    const T* all = partial + (size_t)tile * P * (kGsTile * kGsTile);
#pragma unroll
    for (int a = 0; a < 2; a++)
#pragma unroll
      for (int b = 0; b < 2; b++) {
        T s = T(0);
#pragma unroll 8
        for (unsigned q = 0; q < P; q++) s += all[(size_t)q * (kGsTile * kGsTile) + (ty + 16 * b) * kGsTile + tx + 16 * a];
        acc[a][b] = s;
      }
    if (t == 0) st_coherent(counters + tile, 0u);
  }
#pragma unroll
  for (int a = 0; a < 2; a++)
#pragma unroll
    for (int b = 0; b < 2; b++) {
      const int i = i0 + tx + 16 * a, j = j0 + ty + 16 * b;
      if (i < m && j < n) gemm_store(C + i + (long)j * ldc, acc[a][b], alpha, beta, bias, i, act);
    }
}

// ---- k split inside the workgroup ------------------------------------------------------------------------------
// For the very small products (a few output tiles, k in the tens to hundreds) the cross-workgroup ticket costs more than the
// arithmetic: three dependent memory round trips after the last product.  Here one wave owns the whole 32x32 tile for a slice
// of k (4x4 outputs per lane) and the KS waves of a workgroup take KS slices; their partial tiles meet in LDS.  Every wave runs
// the same number of k steps (loads beyond its slice or beyond k read zeros), so the workgroup barriers line up.
// TS is the edge of a wave's output tile: 32 (4x4 outputs per lane) or 16 (2x2 per lane).  The small tile is for products with
// so few 32x32 tiles and so long a k that even sixteen waves per tile leave most of the chip idle and each wave with a long serial
// walk: four times the workgroups, a quarter of the arithmetic per wave.
template <typename T, bool TA, bool TB, int KS, int TS = kGsTile>
__global__ __launch_bounds__(KS * kWave) void gemm_wave_kernel(int m, int n, int k, T alpha, const T* __restrict__ A, int lda,
                                                              const T* __restrict__ B, int ldb, T beta, T* C, int ldc, const T* bias, int act, int kslice) {
  constexpr int KT = kGsTile;            // k elements per step
  constexpr int Q = TS / 8;              // outputs per lane along each axis (lanes form an 8x8 grid)
  constexpr int R = TS * KT / kWave;     // operand elements a lane stages per step
  __shared__ T As[KS][KT][TS + 1];  // As[w][kk][i] = op(A)(i0+i, k0+kk) of wave w's current step
  __shared__ T Bs[KS][KT][TS + 1];
  const int tiles_m = (m + TS - 1) / TS;
  const int tile = blockIdx.x;
  const int i0 = (tile % tiles_m) * TS, j0 = (tile / tiles_m) * TS;
  const int w = threadIdx.x / kWave, l = threadIdx.x & (kWave - 1);
  const int tx = l & 7, ty = l >> 3;  // outputs (tx + 8a, ty + 8b), a, b = 0..Q-1
  // loader coordinates: `lo` runs along the operand's contiguous axis (TS long for the tile edge, KT long for k), `hi` across it
  const int lo_t = l & (TS - 1), hi_t = l / TS;           // contiguous along the tile edge: kk = hi_t + (64/TS) r
  const int lo_k = l & (KT - 1), hi_k = l / KT;           // contiguous along k: edge index = hi_k + (64/KT) r
  const int kbeg = w * kslice;
  int kend = kbeg + kslice;
  if (kend > k) kend = k;
  T acc[Q][Q];
#pragma unroll
  for (int a = 0; a < Q; a++)
#pragma unroll
    for (int b = 0; b < Q; b++) acc[a][b] = T(0);
  T ga[R], gb[R];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int r = 0; r < R; r++) {
      if (!TA) { const int i = i0 + lo_t, kk = k0 + hi_t + (kWave / TS) * r; ga[r] = (i < m && kk < kend) ? A[i + (long)kk * lda] : T(0); }
      else     { const int kk = k0 + lo_k, i = i0 + hi_k + (kWave / KT) * r; ga[r] = (i < m && kk < kend) ? A[kk + (long)i * lda] : T(0); }
      if (!TB) { const int kk = k0 + lo_k, j = j0 + hi_k + (kWave / KT) * r; gb[r] = (j < n && kk < kend) ? B[kk + (long)j * ldb] : T(0); }
      else     { const int j = j0 + lo_t, kk = k0 + hi_t + (kWave / TS) * r; gb[r] = (j < n && kk < kend) ? B[j + (long)kk * ldb] : T(0); }
    }
  };
  fetch(kbeg);
  for (int k0 = kbeg; k0 < kbeg + kslice; k0 += KT) {
#pragma unroll
    for (int r = 0; r < R; r++) {
      if (!TA) As[w][hi_t + (kWave / TS) * r][lo_t] = ga[r]; else As[w][lo_k][hi_k + (kWave / KT) * r] = ga[r];
      if (!TB) Bs[w][lo_k][hi_k + (kWave / KT) * r] = gb[r]; else Bs[w][hi_t + (kWave / TS) * r][lo_t] = gb[r];
    }
    __syncthreads();
    if (k0 + KT < kbeg + kslice) fetch(k0 + KT);
#pragma unroll 8
    for (int kk = 0; kk < KT; kk++) {
      T av[Q], bv[Q];
#pragma unroll
      for (int a = 0; a < Q; a++) av[a] = As[w][kk][tx + 8 * a];
#pragma unroll
      for (int b = 0; b < Q; b++) bv[b] = Bs[w][kk][ty + 8 * b];
#pragma unroll
      for (int a = 0; a < Q; a++)
#pragma unroll
        for (int b = 0; b < Q; b++) acc[a][b] = kfma(av[a], bv[b], acc[a][b]);
    }
    __syncthreads();
  }
  if (KS > 1) {
    // partial tiles into LDS (each wave reuses its own staging area: KT*(TS+1) >= TS*TS elements), summed in wave order
    T* mine = &As[w][0][0];
#pragma unroll
    for (int a = 0; a < Q; a++)
#pragma unroll
      for (int b = 0; b < Q; b++) mine[(ty + 8 * b) * TS + tx + 8 * a] = acc[a][b];
    __syncthreads();
    for (int o = threadIdx.x; o < TS * TS; o += KS * kWave) {
      T sum = T(0);
#pragma unroll
      for (int q = 0; q < KS; q++) sum += (&As[q][0][0])[o];
      const int i = i0 + (o & (TS - 1)), j = j0 + o / TS;
      if (i < m && j < n) gemm_store(C + i + (long)j * ldc, sum, alpha, beta, bias, i, act);
    }
  } else {
#pragma unroll
    for (int a = 0; a < Q; a++)
#pragma unroll
      for (int b = 0; b < Q; b++) {
        const int i = i0 + tx + 8 * a, j = j0 + ty + 8 * b;
        if (i < m && j < n) gemm_store(C + i + (long)j * ldc, acc[a][b], alpha, beta, bias, i, act);
      }
  }
}

// True if this product should use the small kernel.
// hipBLASLt has a floor of about 12 us per call on this chip; the kernels here stay below it up to about 1e8 flop in general and
// 2.7e8 flop when k <= 512 (512^3: 10.4 vs 12.0 us; 256x256x2048: 28 vs 12.6 us -- long k runs serially inside a wave).
inline bool gemm_is_small(int m, int n, int k) {
  const double flop = 2.0 * m * n * (double)k, limit = 1.0e6 * tuning(kTuneGemmSmallMflop);
  return (flop <= limit || (flop <= 2.7 * limit && k <= 512)) && (long)m * n <= 262144;
}

template <typename T>
inline void launch_gemm_small(hipStream_t stream, bool ta, bool tb, int m, int n, int k, T alpha, const T* A, int lda, const T* B, int ldb,
                              T beta, T* C, int ldc, const T* bias = nullptr, int act = 0) {
  const long tiles = (long)((m + kGsTile - 1) / kGsTile) * ((n + kGsTile - 1) / kGsTile);
  const long ksteps = (k + kGsTile - 1) / kGsTile;
  const long tiles16 = (long)((m + 15) / 16) * ((n + 15) / 16);
  if (tiles16 * ksteps <= 4096 && tuning(kTuneGemmWaveTiles) != 1) {
    // The smaller products (up to about 7e7 flop): 16x16 tiles, one wave per tile and k slice, as many slices per workgroup as there
    // are 32-deep steps (up to 16), partial tiles combined in LDS -- every load of the product is in flight at once and no combine
    // leaves the workgroup.  Measured (us per call, back-to-back launches; this path vs the 32x32-tile paths below):
    // 64x100x784 7.6/12.1, 10x100x64 3.8/5.3, 64x784x100 NT 4.1/6.1, 128^3 3.9/6.1, 256^3 4.2/6.4, 300^3 7.5/9.6, 256x300x512 TN 7.7/10.1,
    // 1000x10x1000 7.8/15.5, 64x4096x100 5.2/6.7; from about 1e8 flop (512x512x190: 7.8/6.9) the larger tiles win.
    int ks = 1;
    while (ks < 16 && ks < ksteps) ks *= 2;
    const int kslice = (int)((ksteps + ks - 1) / ks) * kGsTile;
    const dim3 grid16((unsigned)tiles16);
#define KNET8_GW16K(TA, TB, KSX) hipLaunchKernelGGL((gemm_wave_kernel<T, TA, TB, KSX, 16>), grid16, dim3(KSX * kWave), 0, stream, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc, bias, act, kslice)
#define KNET8_GW16(TA, TB) do { if (ks == 1) KNET8_GW16K(TA, TB, 1); else if (ks == 2) KNET8_GW16K(TA, TB, 2); else if (ks == 4) KNET8_GW16K(TA, TB, 4); \
                                else if (ks == 8) KNET8_GW16K(TA, TB, 8); else KNET8_GW16K(TA, TB, 16); } while (0)
    if (!ta && !tb) KNET8_GW16(false, false);
    else if (ta && !tb) KNET8_GW16(true, false);
    else if (!ta && tb) KNET8_GW16(false, true);
    else KNET8_GW16(true, true);
#undef KNET8_GW16
#undef KNET8_GW16K
    return;
  }
  if (ksteps >= 4 && tiles >= 16 && tiles <= tuning(kTuneGemmWaveTiles)) {
    // Enough tiles to occupy a fair share of the CUs and a k long enough that walking it serially would dominate: one wave per k
    // slice inside the workgroup, no cross-workgroup combine.  Measured (us per call, back-to-back launches, this kernel vs the
    // one below): 128^3 6.1/7.1, 256^3 6.3/9.9, 512x300x256 6.4/10.0, 512x256x300 NT 9.2/12.4, 256x300x512 TN 10.4/17.3.  With fewer
    // tiles (64x100x784: 15.4/11.8) one CU's LDS bandwidth limits a 16-wave workgroup and the cross-workgroup split wins; with
    // short k (256x300x96: 6.7/5.1) the 256-lane tiles win.
    constexpr int kMaxKs = sizeof(T) == 4 ? 16 : 8;  // 2 * 32*33 elements of LDS per wave
    int ks = 1;
    while (ks < kMaxKs && ks < ksteps) ks *= 2;
    const int kslice = (int)((ksteps + ks - 1) / ks) * kGsTile;
    const dim3 grid((unsigned)tiles);
#define KNET8_GW1(TA, TB, KS) hipLaunchKernelGGL((gemm_wave_kernel<T, TA, TB, KS>), grid, dim3(KS * kWave), 0, stream, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc, bias, act, kslice)
#define KNET8_GW(TA, TB) do { if (ks == 1) KNET8_GW1(TA, TB, 1); else if (ks == 2) KNET8_GW1(TA, TB, 2); else if (ks == 4) KNET8_GW1(TA, TB, 4); \
                              else if (ks == 8) KNET8_GW1(TA, TB, 8); else { if constexpr (kMaxKs >= 16) KNET8_GW1(TA, TB, kMaxKs); } } while (0)
    if (!ta && !tb) KNET8_GW(false, false);
    else if (ta && !tb) KNET8_GW(true, false);
    else if (!ta && tb) KNET8_GW(false, true);
    else KNET8_GW(true, true);
#undef KNET8_GW
#undef KNET8_GW1
    return;
  }
  long P = 1;
  const long ncu = tuning(kTuneNumCUs);
  if (tiles * 8 <= ncu) P = ncu / (2 * tiles);  // measured: splitting pays only when the tiles cover a small fraction of the CUs
  if (P > ksteps) P = ksteps;
  if (P < 1) P = 1;
  int kchunk = (int)(((ksteps + P - 1) / P) * kGsTile);
  if (kchunk < kGsTile) kchunk = kGsTile;
  P = (k + kchunk - 1) / kchunk;
  if (P < 1) P = 1;
  Workspace ws = {nullptr, nullptr};
  if (P > 1) ws = workspace_for(stream, sizeof(T) * (size_t)tiles * P * kGsTile * kGsTile, (size_t)tiles);
  const dim3 grid((unsigned)(tiles * P)), block(256);
  T* partial = static_cast<T*>(ws.partial);
#define KNET8_GS(TA, TB) hipLaunchKernelGGL((gemm_small_kernel<T, TA, TB>), grid, block, 0, stream, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc, bias, act, kchunk, (unsigned)P, partial, ws.counters)
  if (!ta && !tb) KNET8_GS(false, false);
  else if (ta && !tb) KNET8_GS(true, false);
  else if (!ta && tb) KNET8_GS(false, true);
  else KNET8_GS(true, true);
#undef KNET8_GS
}

}  // namespace knet8
