// Small-matrix GEMM C = alpha*op(A)*op(B) + beta*C (column-major), for products far too small to fill the
// machine -- the 64x100x784-class products of the MNIST MLP, where the vendor library needs 12-25 us of host and device time per
// call.  Large products go to hipBLASLt (knet8_runtime.hip).  At this size a product's time is one launch (3.2 us for an empty
// kernel), one memory round trip and a short k walk: what matters is how many steps run one after the other and whether partial
// results have to leave the workgroup.  Two kernels, chosen in launch_gemm_small:
//   * gemm_mfma_kernel: 16x16 output tile per workgroup on the matrix cores, one wave per k slice (1..16 slices), operands straight
//     from global memory into the instruction's registers, partial tiles summed in LDS -- every product with k <= 8192;
//   * gemm_small_kernel: 32x32 tile per 256-lane workgroup, k split over P workgroups per tile whose partial tiles are combined, in
//     fixed order, by the last one to finish (write-through + ticket, as in the reductions) -- few tiles with a very long k.
// Both add the bias and apply relu in their output stage when asked (gemm_bias_act_S): same bits as separate launches.
#pragma once
#include "knet8_device.h"
#include "knet8_runtime.h"

namespace knet8 {

constexpr int kGsTile = 32;
// The library is built with -ffp-contract=off for the elementwise contracts; a matrix product wants the fused form.
__device__ __forceinline__ float kfma(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
__device__ __forceinline__ double kfma(double a, double b, double c) { return __builtin_fma(a, b, c); }

// Output stage shared by the kernels below: v = alpha*acc [+ beta*C] [+ bias[i]] [relu].  Each step is one rounded operation, so
// a product with bias and relu folded in gives the bits of the product followed by the separate bias-add and relu launches (on data without
// NaN: this relu is z > 0 ? z : 0 on every route of gemm_bias_act_S, the vendor epilogue included, where relu_S keeps a NaN).
template <typename T>
__device__ __forceinline__ void gemm_store(T* c, T acc, T alpha, T beta, const T* bias, int i, int act) {
  T v = alpha * acc;
  if (beta != T(0)) v = v + beta * *c;
  if (bias) v = v + bias[i];
  if (act == 1) v = v > T(0) ? v : T(0);   // the device relu of the reference (src/libknet8/ops.jl:63) and of the vendor epilogue: NaN -> 0
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

// ---- 16x16 tiles on the matrix cores, k split inside the workgroup ------------------------------------------------
// v_mfma_{f32,f64}_16x16x4: one instruction multiplies a 16x4 by a 4x16 panel in full fp32/fp64 precision.  Lane l supplies
// A(i = l%16, kk = l/16) and B(kk = l/16, j = l%16) and receives four outputs, column j = l%16, rows 4*(l/16) + r in fp32 and
// 4*r + l/16 in fp64 (r = 0..3).  The operands go from global memory straight into the instruction's registers -- no LDS staging, no
// barrier inside the k walk.  Which k a lane feeds to which of the four instructions of a 16-deep step is free as long as A and B
// agree: lane (.., q = l/16) takes k = 4q .. 4q+3, so an operand that is contiguous along k is read with one 16-byte (fp64: 32-byte)
// load per lane and step -- with 4-byte loads the sixteen lines a wave touches per instruction keep the CU's address unit busy four
// times as long, and the sixteen waves of a workgroup share it.  The KS waves of a workgroup take KS slices of k (every wave of
// the product has all its loads in flight at once) and their partial tiles meet in LDS: no combine leaves the workgroup.
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef double f64x4_t __attribute__((ext_vector_type(4)));
template <typename T> struct Mfma16;
template <> struct Mfma16<float> {
  typedef f32x4_t Acc;
  __device__ static __forceinline__ Acc run(float a, float b, Acc c) { return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0); }
  __device__ static __forceinline__ int row(int r, int kq) { return 4 * kq + r; }
};
template <> struct Mfma16<double> {
  typedef f64x4_t Acc;
  __device__ static __forceinline__ Acc run(double a, double b, Acc c) { return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0); }
  __device__ static __forceinline__ int row(int r, int kq) { return 4 * r + kq; }
};

// Four consecutive k of one operand column (or row) for a lane: p points at k = 0 of it, `step` is the distance between consecutive k.
template <typename T, bool KCONT>
__device__ __forceinline__ void mfma_load4(T (&v)[4], const T* __restrict__ p, long step, int kk0, int kend, bool ok, bool vec) {
  typedef T V4 __attribute__((ext_vector_type(4)));
  if (KCONT && vec && ok && kk0 + 3 < kend) {
    const V4 q = *reinterpret_cast<const V4*>(p + kk0);
#pragma unroll
    for (int c = 0; c < 4; c++) v[c] = q[c];
  } else {
#pragma unroll
    for (int c = 0; c < 4; c++) v[c] = (ok && kk0 + c < kend) ? p[(kk0 + c) * step] : T(0);
  }
}
template <typename T>
inline bool mfma_vec_ok(const T* p, int ld) { return (reinterpret_cast<uintptr_t>(p) % (4 * sizeof(T))) == 0 && ld % 4 == 0; }

template <typename T, bool TA, bool TB, int KS>
__global__ __launch_bounds__(KS * kWave) void gemm_mfma_kernel(int m, int n, int k, T alpha, const T* __restrict__ A, int lda, const T* __restrict__ B,
                                                              int ldb, T beta, T* C, int ldc, const T* bias, int act, int kslice, bool veca, bool vecb) {
  constexpr int TS = 16;
  __shared__ T part[KS > 1 ? KS : 1][TS * TS];   // part[w][j*16 + i]
  const int tiles_m = (m + TS - 1) / TS;
  const int tile = blockIdx.x;
  const int i0 = (tile % tiles_m) * TS, j0 = (tile / tiles_m) * TS;
  const int w = threadIdx.x / kWave, l = threadIdx.x & (kWave - 1);
  const int r16 = l & 15, kq = l >> 4;
  const int kbeg = w * kslice;
  int kend = kbeg + kslice;
  if (kend > k) kend = k;
  const int i = i0 + r16, j = j0 + r16;
  const bool iok = i < m, jok = j < n;
  // column (or row) of each operand this lane walks; out-of-range lanes read element 0 of a valid column and are masked to zero
  const T* ap = TA ? A + (long)(iok ? i : 0) * lda : A + (iok ? i : 0);
  const T* bp = TB ? B + (jok ? j : 0) : B + (long)(jok ? j : 0) * ldb;
  const long astep = TA ? 1 : lda, bstep = TB ? ldb : 1;
  typename Mfma16<T>::Acc acc = {T(0), T(0), T(0), T(0)};
#pragma unroll 4
  for (int kc = kbeg; kc < kend; kc += 16) {
    T a[4], b[4];
    mfma_load4<T, TA>(a, ap, astep, kc + 4 * kq, kend, iok, veca);
    mfma_load4<T, !TB>(b, bp, bstep, kc + 4 * kq, kend, jok, vecb);
#pragma unroll
    for (int c = 0; c < 4; c++) acc = Mfma16<T>::run(a[c], b[c], acc);
  }
  if (KS > 1) {
#pragma unroll
    for (int r = 0; r < 4; r++) part[w][r16 * TS + Mfma16<T>::row(r, kq)] = acc[r];
    __syncthreads();
    for (int o = threadIdx.x; o < TS * TS; o += KS * kWave) {
      T sum = T(0);
#pragma unroll
      for (int q = 0; q < KS; q++) sum += part[q][o];
      const int oi = i0 + (o & (TS - 1)), oj = j0 + o / TS;
      if (oi < m && oj < n) gemm_store(C + oi + (long)oj * ldc, sum, alpha, beta, bias, oi, act);
    }
  } else {
#pragma unroll
    for (int r = 0; r < 4; r++) {
      const int oi = i0 + Mfma16<T>::row(r, kq);
      if (oi < m && jok) gemm_store(C + oi + (long)j * ldc, acc[r], alpha, beta, bias, oi, act);
    }
  }
}

// True if this product should use the library's own kernels.  Against the vendor library's kernels (durations by kernel trace, fp32,
// us; own / vendor): 1000x100x1000 8.5/9.0 (TN 8.4/10.2, dW form 1000x1000x100 NT 9.1/7.5), 1024x128x1024 8.1/8.2, 512x256x512 5.4/6.6,
// 2048x64x784 7.1/8.2, 768x768x128 6.3/6.2 -- level up to about 2.7e8 flop whatever the shape, and the vendor call costs its caller another
// 12 us of host time; beyond that its large LDS tiles win clearly (640^3 15.5/9.8, 2048x128x2048 28/15, 4096x100x4096 141/34).
inline bool gemm_is_small(int m, int n, int k) {
  const double flop = 2.0 * m * n * (double)k, limit = 1.0e6 * tuning(kTuneGemmSmallMflop);
  if (k > 8192) return flop <= limit && (long)m * n <= 262144;   // cross-workgroup split: its partial tiles live in the stream's scratch
  return flop <= limit;
}

template <typename T>
inline void launch_gemm_small(hipStream_t stream, bool ta, bool tb, int m, int n, int k, T alpha, const T* A, int lda, const T* B, int ldb,
                              T beta, T* C, int ldc, const T* bias = nullptr, int act = 0) {
  const long tiles = (long)((m + kGsTile - 1) / kGsTile) * ((n + kGsTile - 1) / kGsTile);
  const long ksteps = (k + kGsTile - 1) / kGsTile;
  const long tiles16 = (long)((m + 15) / 16) * ((n + 15) / 16);
  if (ksteps <= 256) {
    // One wave per 16x16 tile and k slice, as many slices per workgroup as there are 32-deep steps (up to 16).  Kernel durations
    // (us, rocprofv3 kernel trace, fp32; this kernel / the vendor library's kernel, which costs its caller another 12 us of host time):
    // 64x100x784 4.6/-, 10x100x64 3.4/-, 32^3 2.5/-, 128^3 3.0/-, 256^3 3.5/-, 300^3 4.5/-, 512x300x256 4.9/6.9, 256x300x512 TN 6.1/11.6,
    // 700x300x200 5.2/6.8, 400^3 6.3/7.3, 512^3 8.5/8.2 (NT 8.8/8.7, TN 10.7/7.0), 256x256x2048 8.6/11.4, 64x64x2000 7.5/11.1, 16x16x4000 12.0/-.
    // Beyond k = 8192 with few tiles a wave's serial walk gets long and the cross-workgroup split below takes over.
    int ks = 1;
    while (ks < 16 && ks < ksteps) ks *= 2;
    const int kslice = (int)((ksteps + ks - 1) / ks) * kGsTile;
    const dim3 grid16((unsigned)tiles16);
    const bool veca = ta && mfma_vec_ok(A, lda), vecb = !tb && mfma_vec_ok(B, ldb);
#define KNET8_GM16K(TA, TB, KSX) hipLaunchKernelGGL((gemm_mfma_kernel<T, TA, TB, KSX>), grid16, dim3(KSX * kWave), 0, stream, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc, bias, act, kslice, veca, vecb)
#define KNET8_GM16(TA, TB) do { if (ks == 1) KNET8_GM16K(TA, TB, 1); else if (ks == 2) KNET8_GM16K(TA, TB, 2); else if (ks == 4) KNET8_GM16K(TA, TB, 4); \
                                else if (ks == 8) KNET8_GM16K(TA, TB, 8); else KNET8_GM16K(TA, TB, 16); } while (0)
    if (!ta && !tb) KNET8_GM16(false, false);
    else if (ta && !tb) KNET8_GM16(true, false);
    else if (!ta && tb) KNET8_GM16(false, true);
    else KNET8_GM16(true, true);
#undef KNET8_GM16
#undef KNET8_GM16K
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
  if (P > 1) {
    ws = workspace_for(stream, sizeof(T) * (size_t)tiles * P * kGsTile * kGsTile, (size_t)tiles);
    if (!scratch_ready(ws, "gemm (small, k split): no scratch memory for a split launch")) return;
  }
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
