// Small-matrix GEMM C = alpha*op(A)*op(B) + beta*C (column-major), for products far too small to fill the
// machine -- the 64x100x784-class products of the MNIST MLP, where the vendor library needs 15-25 us per call and
// a whole captured training step is otherwise ~80 us.  Large products go to hipBLASLt (knet8_runtime.hip).
//
// 32x32 output tile per 256-lane workgroup (2x2 outputs per lane), k walked in steps of 32 through LDS; when the
// tiles alone would leave most CUs idle the k range is split over P workgroups per tile whose partial tiles are
// combined, in fixed order, by the last one to finish (same write-through + ticket scheme as the reductions).
#pragma once
#include "knet8_device.h"
#include "knet8_runtime.h"

namespace knet8 {

constexpr int kGsTile = 32;
// The library is built with -ffp-contract=off for the elementwise contracts; a matrix product wants the fused form.
__device__ __forceinline__ float kfma(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
__device__ __forceinline__ double kfma(double a, double b, double c) { return __builtin_fma(a, b, c); }

template <typename T, bool TA, bool TB>
__global__ __launch_bounds__(256) void gemm_small_kernel(int m, int n, int k, T alpha, const T* __restrict__ A, int lda,
                                                         const T* __restrict__ B, int ldb, T beta, T* C, int ldc, int kchunk,
                                                         unsigned P, T* partial, unsigned* counters) {
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
      if (i < m && j < n) {
        T* c = C + i + (long)j * ldc;
        const T v = alpha * acc[a][b];
        *c = beta == T(0) ? v : v + beta * *c;
      }
    }
}

// True if this product should use the small kernel.
inline bool gemm_is_small(int m, int n, int k) { return 2.0 * m * n * (double)k <= 1.0e8 && (long)m * n <= 262144; }

template <typename T>
inline void launch_gemm_small(hipStream_t stream, bool ta, bool tb, int m, int n, int k, T alpha, const T* A, int lda, const T* B, int ldb,
                              T beta, T* C, int ldc) {
  const long tiles = (long)((m + kGsTile - 1) / kGsTile) * ((n + kGsTile - 1) / kGsTile);
  const long ksteps = (k + kGsTile - 1) / kGsTile;
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
#define KNET8_GS(TA, TB) hipLaunchKernelGGL((gemm_small_kernel<T, TA, TB>), grid, block, 0, stream, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc, kchunk, (unsigned)P, partial, ws.counters)
  if (!ta && !tb) KNET8_GS(false, false);
  else if (ta && !tb) KNET8_GS(true, false);
  else if (!ta && tb) KNET8_GS(false, true);
  else KNET8_GS(true, true);
#undef KNET8_GS
}

}  // namespace knet8
