// Fused layer kernels for y = f(w*x .+ b) with b of shape (m,1) on an m x n column-major matrix.
//
// The reference runs this as separate launches: bias add (src/knetarrays/binary.jl:61-95 -> add_S_12),
// activation (src/ops20_gpu/activation.jl:17-29), dropout (src/ops20_gpu/dropout.jl:12-21) on the way forward;
// dropback, activation gradient (src/ops20_gpu/activation.jl:30-37) and the bias gradient sum(dz;dims=2)
// (src/knetarrays/reduction.jl:21-77) on the way back.  Each fused kernel here makes one pass instead:
//   forward   y = f(z + b[i])            [then dropout]   2 streams (3 with the uniform buffer) instead of 6 (9)
//   backward  dz = f'(dy, y), db = sum_j dz               3 streams instead of 7 (10 with dropback)
// Every element goes through the same rounded operations as the separate launches, so dz and y are bit-identical
// to the chain; db differs from the chain's sum only by summation order.
#pragma once
#include "knet8_elementwise.h"
#include "knet8_reduce.h"

namespace knet8 {

// ---- forward -----------------------------------------------------------------------------------------
// F(T zb [, T u]) maps the biased pre-activation (and, with DROP, the uniform draw found in y) to the output.
template <typename T, typename F, bool DROP, int NV>
__global__ __launch_bounds__(kEwBlock) void bias_act_kernel(long nitems, const T* z, const T* b, unsigned m, T* y, F f) {
  const long i = (long)blockIdx.x * kEwBlock + threadIdx.x;
  if (i >= nitems) return;
  const long e = i * NV;
  const unsigned r = (unsigned)e % m;  // sizes are 32-bit ints at the ABI; m % NV == 0 on the vector path, so the NV elements share a column
  if (NV > 1) {
    typedef typename Vec16<T>::type V;
    const V a = ld_stream(reinterpret_cast<const V*>(z + e));
    const V bv = *reinterpret_cast<const V*>(b + r);
    V u, o;
    if (DROP) u = ld_stream(reinterpret_cast<const V*>(y + e));
#pragma unroll
    for (int k = 0; k < NV; k++) {
      const T zb = a[k] + bv[k];
      o[k] = f(zb, DROP ? u[k] : T(0));
    }
    st_stream(reinterpret_cast<V*>(y + e), o);
  } else {
    const T zb = z[e] + b[r];
    y[e] = f(zb, DROP ? y[e] : T(0));
  }
}

// Any number of units (1001, 50257): z and y still move in 16-byte accesses over the flat array, the bias entries are fetched one by one with the row
// carried along; the last m*n % NV elements are done by workgroup 0.
template <typename T, typename F, bool DROP>
__global__ __launch_bounds__(kEwBlock) void bias_act_wrap_kernel(long nvec, long count, const T* z, const T* b, unsigned m, T* y, F f) {
  typedef typename Vec16<T>::type V;
  constexpr int NV = Vec16<T>::N;
  const long i = (long)blockIdx.x * kEwBlock + threadIdx.x;
  if (i < nvec) {
    const long e = i * NV;
    unsigned r = (unsigned)e % m;
    const V a = ld_stream(reinterpret_cast<const V*>(z + e));
    V u, o;
    if (DROP) u = ld_stream(reinterpret_cast<const V*>(y + e));
#pragma unroll
    for (int k = 0; k < NV; k++) {
      const T zb = a[k] + b[r];
      o[k] = f(zb, DROP ? u[k] : T(0));
      if (++r == m) r = 0;
    }
    st_stream(reinterpret_cast<V*>(y + e), o);
  }
  if (blockIdx.x == 0) {
    const long e = nvec * NV + threadIdx.x;
    if (e < count) {
      const T zb = z[e] + b[(unsigned)e % m];
      y[e] = f(zb, DROP ? y[e] : T(0));
    }
  }
}

template <typename T, bool DROP, typename F>
inline void launch_bias_act(hipStream_t stream, long m, long n, const T* z, const T* b, T* y, F f) {
  if (m <= 0 || n <= 0) return;
  if (m * n >= (1L << 31)) { record_error("bias + activation: 2^31 or more elements; the kernel's 32-bit row arithmetic does not reach that far"); return; }
  constexpr int N = Vec16<T>::N;
  const bool vec = (m % N == 0) && aligned16(z) && aligned16(b) && aligned16(y);
  if (!vec && aligned16(z) && aligned16(y) && m * n >= 4 * N) {
    const long nvec = m * n / N, grid = (nvec + kEwBlock - 1) / kEwBlock;
    hipLaunchKernelGGL((bias_act_wrap_kernel<T, F, DROP>), dim3((unsigned)grid), dim3(kEwBlock), 0, stream, nvec, m * n, z, b, (unsigned)m, y, f);
    return;
  }
  const long nitems = vec ? m * n / N : m * n;
  const long grid = (nitems + kEwBlock - 1) / kEwBlock;
  if (vec)
    hipLaunchKernelGGL((bias_act_kernel<T, F, DROP, N>), dim3((unsigned)grid), dim3(kEwBlock), 0, stream, nitems, z, b, (unsigned)m, y, f);
  else
    hipLaunchKernelGGL((bias_act_kernel<T, F, DROP, 1>), dim3((unsigned)grid), dim3(kEwBlock), 0, stream, nitems, z, b, (unsigned)m, y, f);
}

// ---- backward ----------------------------------------------------------------------------------------
// Row tile of 64*NV consecutive i's per workgroup, the BT/64 waves take columns j = j0+wave, j0+wave+NW, ...;
// P workgroups split the columns of a tile and the last one to finish adds their partial sums (same ticket
// scheme as the strided reduction).  F(dy, y) is the element gradient.  dz may be dy or y itself (each element is read
// before the same lane writes it).
// SC: rows that do not start on 16-byte boundaries (m odd) -- the lane's NV elements are the rows lane, lane+64, ... of the tile,
// each moved with its own 4- or 8-byte access (see strided_walk).
template <typename T, typename F, int NV, int BT, int U, bool SC>
__global__ __launch_bounds__(BT) void actback_biasgrad_kernel(const T* dy, const T* yv, long m, long n, long jchunk, unsigned P, T* dz, T* __restrict__ db,
                                                              T* partial, unsigned* counters, F f KNET8_TL_PARAM) {
  KNET8_TL_BEGIN
  constexpr int TILE = kWave * NV;
  constexpr int NW = BT / kWave;
  __shared__ T lds[NW][TILE];
  __shared__ unsigned flag;
  const long at = blockIdx.x / P;
  const unsigned p = blockIdx.x % P;
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const long a0 = at * TILE + (SC ? (long)lane : (long)lane * NV);
  unsigned livemask = 0;
#pragma unroll
  for (int e = 0; e < NV; e++)
    if (a0 + (SC ? e * kWave : e) < m) livemask |= 1u << e;   // vector path: m % NV == 0, all or nothing
  const long j0 = (long)p * jchunk;
  long j1 = j0 + jchunk;
  if (j1 > n) j1 = n;
  T acc[NV];
#pragma unroll
  for (int e = 0; e < NV; e++) acc[e] = T(0);
  if (livemask) {
    for (long j = j0 + wave; j < j1; j += NW * U) {
      T g[U][NV];
      if constexpr (!SC && NV > 1) {
        // Vector path: the loads of all U columns first, then the U results and stores.  Written column by column, the second column's loads sink
        // below the first column's store (dz may be dy or y itself, so the compiler must keep that order), and every load then waits for the store
        // before it as well: U dependent round trips instead of one.  A column past the end of the share reads the share's last column again.
        typedef typename Vec16<T>::type V;
        V d[U], o[U];
#pragma unroll
        for (int q = 0; q < U; q++) {
          const long jj = j + q * NW < j1 ? j + q * NW : j;
          const long off = jj * m + a0;
          d[q] = ld_stream(reinterpret_cast<const V*>(dy + off));
          o[q] = ld_stream(reinterpret_cast<const V*>(yv + off));
        }
#pragma unroll
        for (int q = 0; q < U; q++) {
          const long jj = j + q * NW;
          V r;
#pragma unroll
          for (int e = 0; e < NV; e++) { r[e] = f(d[q][e], o[q][e]); g[q][e] = jj < j1 ? r[e] : T(0); }
          // written through (sc1), not merely streamed: what a kernel leaves dirty in the L2s is written back after its last workgroup has ended,
          // before the next launch may start; written through, dz drains while the partial sums are still being combined
          // ((4096,2048) fp32 cold: 19.3 -> 18.4 us; nt sc1 19.9-20.0, sc0 sc1 18.6, plain 19.3)
          if (jj < j1) st_through(reinterpret_cast<V*>(dz + jj * m + a0), r);
        }
      } else {
#pragma unroll
      for (int q = 0; q < U; q++) {
        const long jj = j + q * NW;
        if (jj < j1) {
          const long off = jj * m + a0;
#pragma unroll
          for (int e = 0; e < NV; e++) {
            if (livemask & (1u << e)) {
              const T r = f(__builtin_nontemporal_load(dy + off + e * kWave), __builtin_nontemporal_load(yv + off + e * kWave));
              g[q][e] = r;
              __builtin_nontemporal_store(r, dz + off + e * kWave);
            } else {
              g[q][e] = T(0);
            }
          }
        } else {
#pragma unroll
          for (int e = 0; e < NV; e++) g[q][e] = T(0);
        }
      }
      }
#pragma unroll
      for (int q = 0; q < U; q++)
#pragma unroll
        for (int e = 0; e < NV; e++) acc[e] = acc[e] + g[q][e];
    }
  }
  KNET8_TL_MID
  if (P > 1) {
#pragma unroll
    for (int e = 0; e < NV; e++) lds[wave][SC ? e * kWave + lane : lane * NV + e] = acc[e];
    __syncthreads();
    if (threadIdx.x < TILE) {
      T r = T(0);
#pragma unroll
      for (int w = 0; w < NW; w++) r = r + lds[w][threadIdx.x];
      st_coherent(partial + (at * P + p) * TILE + threadIdx.x, r);
    }
    if (!last_block_ticket(counters + at * kTicketStride, P, &flag)) { KNET8_TL_END return; }
#pragma unroll
    for (int e = 0; e < NV; e++) acc[e] = T(0);
    strided_walk<T, RedSum<T>, NV, false, NW, kCombineU, SC>(partial + at * P * TILE + (SC ? lane : lane * NV), TILE, 0, P, wave, acc);
    if (threadIdx.x == 0) st_coherent(counters + at * kTicketStride, 0u);
  }
#pragma unroll
  for (int e = 0; e < NV; e++) lds[wave][SC ? e * kWave + lane : lane * NV + e] = acc[e];
  __syncthreads();
  const long a = at * TILE + threadIdx.x;
  if (threadIdx.x < TILE && a < m) {
    T r = T(0);
#pragma unroll
    for (int w = 0; w < NW; w++) r = r + lds[w][threadIdx.x];
    db[a] = r;
  }
  KNET8_TL_END
}

// The element gradient alone, over the flat array (few rows: see launch_actback_biasgrad).
template <typename T, typename F, int NV>
__global__ __launch_bounds__(256) void actback_flat_kernel(const T* dy, const T* yv, long count, T* dz, F f) {
  const long i = ((long)blockIdx.x * 256 + threadIdx.x) * NV;
  if (i >= count) return;
  if (NV > 1) {
    typedef typename Vec16<T>::type V;
    const V a = ld_stream(reinterpret_cast<const V*>(dy + i)), b = ld_stream(reinterpret_cast<const V*>(yv + i));
    V o;
#pragma unroll
    for (int e = 0; e < NV; e++) o[e] = f(a[e], b[e]);
    st_stream(reinterpret_cast<V*>(dz + i), o);
  } else {
    dz[i] = f(dy[i], yv[i]);
  }
}

template <typename T, typename F>
inline void launch_actback_biasgrad(hipStream_t stream, long m, long n, const T* dy, const T* y, T* dz, T* db, F f) {
  if (m <= 0) return;
  if (n > 0 && m * n >= (1L << 31)) { record_error("activation gradient + bias gradient: 2^31 or more elements are not supported"); return; }
  constexpr int N = Vec16<T>::N;
  const bool flat16 = (m * n) % N == 0 && aligned16(dy) && aligned16(y) && aligned16(dz);
  if ((m < kWave || (m % N != 0 && flat16)) && n > 0) {
    // A layer of few units (ten classes): a 256-row tile would idle nearly all its lanes ((2, 4M): 531 us, (10, 839K): 132 us for 100 MB).
    // Two launches instead: the element gradient over the flat array, then the row sums of dz by the reduction family -- one more read of dz,
    // 4/3 of the bytes, same bits for dz and the same kind of fixed-order sum for db.  Also for a number of units that is not a multiple of the
    // vector width (1001) when the flat array can still move in 16-byte accesses: the tiled kernel falls back on 4-byte ones there.
    const long count = m * n;
    const bool v = flat16;
    if (v) hipLaunchKernelGGL((actback_flat_kernel<T, F, N>), dim3((unsigned)ceil_div(count / N, 256)), dim3(256), 0, stream, dy, y, count, dz, f);
    else hipLaunchKernelGGL((actback_flat_kernel<T, F, 1>), dim3((unsigned)ceil_div(count, 256)), dim3(256), 0, stream, dy, y, count, dz, f);
    launch_reduce_strided<T, RedSum<T>>(stream, dz, m, n, 1, db);
    return;
  }
  const bool vec = (m % N == 0) && aligned16(dy) && aligned16(y) && aligned16(dz);
  const long tile = (long)kWave * N;
  const long atiles = ceil_div(m, tile);
  // (parts by memory round trips, as in the strided reduction; a part's waves take sixteen columns per trip here: (256, 8192) fp32 13.9 us with 256 parts of
  //  32 columns, whose 256 partial rows one four-wave workgroup then combines)
  unsigned P = n > 0 ? plan_parts_by_trips(atiles, n, 16, 64) : 1;
  long jchunk = ceil_div(n, P);
  P = (unsigned)ceil_div(n, jchunk > 0 ? jchunk : 1);
  if (P < 1) P = 1;
  Workspace ws = {nullptr, nullptr};
  if (P > 1) {
    ws = workspace_for(stream, sizeof(T) * (size_t)atiles * P * tile, (size_t)atiles * kTicketStride);
    if (!scratch_ready(ws, "activation gradient + bias gradient: no scratch memory for a split launch")) return;
  }
  const dim3 grid((unsigned)(atiles * P));
  T* partial = static_cast<T*>(ws.partial);
  const bool big = jchunk >= 64;
#define KNET8_ABG(BT, U, SC) \
  hipLaunchKernelGGL((actback_biasgrad_kernel<T, F, N, BT, U, SC>), grid, dim3(BT), 0, stream, dy, y, m, n, jchunk, P, dz, db, partial, ws.counters, f KNET8_TL_ARG)
  // (sixteen waves, one column at a time each: (4096,2048) fp32 cold 19.2-19.4 us against 20.1-20.4 with two columns per wave and step, 20.8 with four or
  //  eight; 512 lanes x 32 parts 19.5, 256 lanes x 64 parts 22.1)
  if (vec) { if (big) KNET8_ABG(1024, 1, false); else KNET8_ABG(256, 4, false); }
  else     { if (big) KNET8_ABG(1024, 2, true); else KNET8_ABG(256, 4, true); }
#undef KNET8_ABG
}

}  // namespace knet8
