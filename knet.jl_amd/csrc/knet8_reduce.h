// Reduction kernel family behind the `_20` (array -> scalar), `_21` (array -> vector) and `_22`
// (array -> array, one reduced dimension) entry points.
//
// The reference runs one 128-thread block per output element on a fixed <<<128,128>>> grid
// (src/libknet8/cuda20.jl:27-104, cuda21.jl:22-77, cuda22.jl:22-66); its `sy==1` branch reads with lanes
// `ny` elements apart.  Here every shape is mapped onto one of two views of the column-major input and
// each view has a kernel whose lanes always walk the contiguous axis:
//
//   run view      x(sy, ny, no)  ->  y(ny)      reduce axes 1 and 3   (`_21` with sy>1, `_20`, `_22` with s1==1)
//   strided view  x(s1, d, nb)   ->  y(s1, nb)  reduce axis 2         (`_21` with sy==1, `_22` with s1>1)
//
// Both split the reduced axis over P workgroups per output group when one group alone would leave the
// machine idle or take too long; the P partials are combined, in fixed order, by whichever workgroup
// draws the last ticket of its group, so one launch suffices and the result is deterministic (no float atomics).
//
// HBM roofline: sizeof(T)*(nx + ny) algorithmic bytes.
#pragma once
#include "knet8_device.h"
#include "knet8_runtime.h"

namespace knet8 {

constexpr int kRedBlock = 256;
constexpr int kRedWaves = kRedBlock / kWave;

// ---- operator table: (merge, item, init) triples of src/libknet8/ops.jl:144-156 ---------------------
template <typename T> struct RedSum     { __host__ __device__ static T init() { return T(0); } __device__ static T item(T x) { return x; } __device__ static T merge(T a, T x) { return a + x; } };
template <typename T> struct RedProd    { __host__ __device__ static T init() { return T(1); } __device__ static T item(T x) { return x; } __device__ static T merge(T a, T x) { return a * x; } };
template <typename T> struct RedMaximum { __host__ __device__ static T init() { return -INFINITY; } __device__ static T item(T x) { return x; } __device__ static T merge(T a, T x) { return a > x ? a : x; } };
template <typename T> struct RedMinimum { __host__ __device__ static T init() { return INFINITY; } __device__ static T item(T x) { return x; } __device__ static T merge(T a, T x) { return a < x ? a : x; } };
template <typename T> struct RedSumabs  { __host__ __device__ static T init() { return T(0); } __device__ static T item(T x) { return x < 0 ? -x : x; } __device__ static T merge(T a, T x) { return a + x; } };
template <typename T> struct RedSumabs2 { __host__ __device__ static T init() { return T(0); } __device__ static T item(T x) { return x * x; } __device__ static T merge(T a, T x) { return a + x; } };
template <typename T> struct RedMaxabs  { __host__ __device__ static T init() { return T(0); } __device__ static T item(T x) { return x < 0 ? -x : x; } __device__ static T merge(T a, T x) { return a > x ? a : x; } };
template <typename T> struct RedMinabs  { __host__ __device__ static T init() { return INFINITY; } __device__ static T item(T x) { return x < 0 ? -x : x; } __device__ static T merge(T a, T x) { return a < x ? a : x; } };
template <typename T> struct RedCountnz { __host__ __device__ static T init() { return T(0); } __device__ static T item(T x) { return x != 0 ? T(1) : T(0); } __device__ static T merge(T a, T x) { return a + x; } };

template <typename Op, typename T> struct MergeFn {
  __device__ __forceinline__ T operator()(T a, T b) const { return Op::merge(a, b); }
};

// ---- run view ------------------------------------------------------------------------------------
// Output j reduces K = no*sy elements: flattened index k -> x[(k/sy)*sy*ny + j*sy + k%sy].
// NV = elements per lane per load (Vec16<T>::N on the aligned path, 1 otherwise); on the vector path
// sy % NV == 0 so a vector never straddles two runs.  Workgroup (j,p) covers units [p*chunk, (p+1)*chunk)
// of the K/NV units of output j.
template <typename T, typename Op, int NV, bool SINGLE, int BT, int U>
__global__ __launch_bounds__(BT) void reduce_run_kernel(const T* __restrict__ x, long sy, long ny, long units, long chunk,
                                                               unsigned P, T* __restrict__ y, T* partial, unsigned* counters) {
  constexpr int NW = BT / kWave;
  __shared__ T lds[NW];
  __shared__ unsigned flag;
  const long j = blockIdx.x / P;
  const unsigned p = blockIdx.x % P;
  const long u0 = (long)p * chunk;
  long u1 = u0 + chunk;
  if (u1 > units) u1 = units;
  const long usy = sy / NV;              // units per run
  const long slab = sy * ny;             // elements between the same run of consecutive slabs
  const T* xj = x + j * sy;
  T acc[NV];
#pragma unroll
  for (int e = 0; e < NV; e++) acc[e] = Op::init();
  for (long u = u0 + threadIdx.x; u < u1; u += BT * U) {
    T v[U][NV];
#pragma unroll
    for (int q = 0; q < U; q++) {
      const long uu = u + q * BT;
      if (uu < u1) {
        long off;
        if (SINGLE) off = uu * NV;
        else { const unsigned o = (unsigned)uu / (unsigned)usy; off = o * slab + ((unsigned)uu - o * (unsigned)usy) * NV; }
        if (NV > 1) {
          typedef typename Vec16<T>::type V;
          V t = ld_stream(reinterpret_cast<const V*>(xj + off));
#pragma unroll
          for (int e = 0; e < NV; e++) v[q][e] = Op::item(t[e]);
        } else {
          v[q][0] = Op::item(__builtin_nontemporal_load(xj + off));
        }
      } else {
#pragma unroll
        for (int e = 0; e < NV; e++) v[q][e] = Op::init();
      }
    }
#pragma unroll
    for (int q = 0; q < U; q++)
#pragma unroll
      for (int e = 0; e < NV; e++) acc[e] = Op::merge(acc[e], v[q][e]);
  }
  T r = acc[0];
#pragma unroll
  for (int e = 1; e < NV; e++) r = Op::merge(r, acc[e]);
  r = block_reduce<T, NW>(r, lds, MergeFn<Op, T>(), Op::init());
  if (P == 1) {
    if (threadIdx.x == 0) y[j] = r;
    return;
  }
  if (threadIdx.x == 0) st_coherent(partial + j * P + p, r);
  if (!last_block_ticket(counters + j, P, &flag)) return;
  T s = Op::init();
  for (unsigned q = threadIdx.x; q < P; q += BT) s = Op::merge(s, ld_coherent(partial + j * P + q));
  s = block_reduce<T, NW>(s, lds, MergeFn<Op, T>(), Op::init());
  if (threadIdx.x == 0) {
    y[j] = s;
    st_coherent(counters + j, 0u);
  }
}

// ---- strided view --------------------------------------------------------------------------------
// y[a + b*s1] = reduce_k x[a + k*s1 + b*s1*d].  A wave covers 64*NV consecutive a's with one load per
// lane; the four waves of a workgroup take k = k0+wave, k0+wave+4, ...; P workgroups split the k range.
// The same walk (rows `stride` apart, this wave's share of [k0,k1)) combines the P partial tiles at the end
// (ITEM=false: partials are merged as they are, the item map was applied when they were made).
// SC ("scalar, coalesced"): for rows that do not start on 16-byte boundaries (s1 odd) the lane's NV elements are the columns
// lane, lane+64, ... of the tile instead of NV neighbours, each fetched with its own 4-byte load: a wave instruction still reads
// 256 contiguous bytes and a lane keeps as many bytes in flight as on the vector path.  `livemask` bit e: column e of this lane exists.
template <typename T, typename Op, int NV, bool ITEM, int NW, int U, bool SC = false>
__device__ __forceinline__ void strided_walk(const T* base, long stride, long k0, long k1, int wave, T (&acc)[NV], unsigned livemask = ~0u) {
  for (long k = k0 + wave; k < k1; k += NW * U) {
    T v[U][NV];
#pragma unroll
    for (int q = 0; q < U; q++) {
      const long kk = k + q * NW;
      if (kk < k1) {
        if (SC) {
#pragma unroll
          for (int e = 0; e < NV; e++) {
            if (livemask & (1u << e)) {
              const T t = __builtin_nontemporal_load(base + kk * stride + e * kWave);
              v[q][e] = ITEM ? Op::item(t) : t;
            } else {
              v[q][e] = Op::init();
            }
          }
        } else if (NV > 1) {
          typedef typename Vec16<T>::type V;
          V t = ld_stream(reinterpret_cast<const V*>(base + kk * stride));
#pragma unroll
          for (int e = 0; e < NV; e++) v[q][e] = ITEM ? Op::item(t[e]) : t[e];
        } else {
          const T t = __builtin_nontemporal_load(base + kk * stride);
          v[q][0] = ITEM ? Op::item(t) : t;
        }
      } else {
#pragma unroll
        for (int e = 0; e < NV; e++) v[q][e] = Op::init();
      }
    }
#pragma unroll
    for (int q = 0; q < U; q++)
#pragma unroll
      for (int e = 0; e < NV; e++) acc[e] = Op::merge(acc[e], v[q][e]);
  }
}

template <typename T, typename Op, int NV, int BT, int U, bool SC = false>
__global__ __launch_bounds__(BT) void reduce_strided_kernel(const T* __restrict__ x, long s1, long d, long atiles, long kchunk,
                                                                   unsigned P, T* __restrict__ y, T* partial, unsigned* counters) {
  constexpr int TILE = kWave * NV;
  constexpr int NW = BT / kWave;
  __shared__ T lds[NW][TILE];
  __shared__ unsigned flag;
  // Consecutive workgroups share a row tile and take consecutive k ranges.  The other order (consecutive workgroups =
  // neighbouring row tiles of one k range, i.e. whole contiguous matrix rows per dispatch wave) was measured 20 % slower.
  const long group = blockIdx.x / P;   // (b, atile)
  const unsigned p = blockIdx.x % P;
  const long b = group / atiles, at = group % atiles;
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  // element e of this lane is column a0 + e (vector path: NV neighbours) or a0 + e*64 (SC: interleaved); `slot` is where it sits in the tile
  const long a0 = at * TILE + (SC ? (long)lane : (long)lane * NV);
  unsigned livemask = 0;
#pragma unroll
  for (int e = 0; e < NV; e++)
    if (a0 + (SC ? e * kWave : e) < s1) livemask |= 1u << e;   // on the vector path s1 % NV == 0: all or nothing
  const long k0 = (long)p * kchunk;
  long k1 = k0 + kchunk;
  if (k1 > d) k1 = d;
  T acc[NV];
#pragma unroll
  for (int e = 0; e < NV; e++) acc[e] = Op::init();
  if (livemask) strided_walk<T, Op, NV, true, NW, U, SC>(x + b * s1 * d + a0, s1, k0, k1, wave, acc, livemask);
  if (P > 1) {
    // partial tile p of this group = this workgroup's reduction over its k range
#pragma unroll
    for (int e = 0; e < NV; e++) lds[wave][SC ? e * kWave + lane : lane * NV + e] = acc[e];
    __syncthreads();
    if (threadIdx.x < TILE) {
      T r = Op::init();
#pragma unroll
      for (int w = 0; w < NW; w++) r = Op::merge(r, lds[w][threadIdx.x]);
      st_coherent(partial + (group * P + p) * TILE + threadIdx.x, r);
    }
    if (!last_block_ticket(counters + group, P, &flag)) return;
#pragma unroll
    for (int e = 0; e < NV; e++) acc[e] = Op::init();
    strided_walk<T, Op, NV, false, NW, U, SC>(partial + group * P * TILE + (SC ? lane : lane * NV), TILE, 0, P, wave, acc);
    if (threadIdx.x == 0) st_coherent(counters + group, 0u);
  }
#pragma unroll
  for (int e = 0; e < NV; e++) lds[wave][SC ? e * kWave + lane : lane * NV + e] = acc[e];
  __syncthreads();
  const long a = at * TILE + threadIdx.x;
  if (threadIdx.x < TILE && a < s1) {
    T r = Op::init();
#pragma unroll
    for (int w = 0; w < NW; w++) r = Op::merge(r, lds[w][threadIdx.x]);
    y[b * s1 + a] = r;
  }
}

// Strided view with a short contiguous axis (s1 < 64): lanes along `a` alone would idle most of a wave,
// so the (s1 x d) slab of batch b is walked as one contiguous range, L = s1*floor(256/s1) lanes at a
// time; lane t always meets a == t % s1.  Workgroup (b,p) covers elements [p*chunk, (p+1)*chunk) of the
// slab (chunk is a multiple of L).
template <typename T, typename Op>
__global__ __launch_bounds__(kRedBlock) void reduce_strided_small_kernel(const T* __restrict__ x, int s1, long d, long chunk,
                                                                         unsigned P, T* __restrict__ y, T* partial,
                                                                         unsigned* counters) {
  __shared__ T lds[kRedBlock];
  __shared__ unsigned flag;
  const long b = blockIdx.x / P;
  const unsigned p = blockIdx.x % P;
  const int reps = kRedBlock / s1, L = reps * s1;
  const long total = (long)s1 * d;
  const long i0 = (long)p * chunk;
  long i1 = i0 + chunk;
  if (i1 > total) i1 = total;
  const T* xb = x + b * total;
  T acc = Op::init();
  if ((int)threadIdx.x < L) {
    constexpr int U = 4;
    for (long i = i0 + threadIdx.x; i < i1; i += (long)L * U) {
      T v[U];
#pragma unroll
      for (int q = 0; q < U; q++) {
        const long ii = i + (long)q * L;
        v[q] = ii < i1 ? Op::item(__builtin_nontemporal_load(xb + ii)) : Op::init();
      }
#pragma unroll
      for (int q = 0; q < U; q++) acc = Op::merge(acc, v[q]);
    }
  }
  lds[threadIdx.x] = acc;
  __syncthreads();
  T r = Op::init();
  const bool owner = (int)threadIdx.x < s1;
  if (owner)
    for (int q = 0; q < reps; q++) r = Op::merge(r, lds[threadIdx.x + q * s1]);
  if (P == 1) {
    if (owner) y[b * s1 + threadIdx.x] = r;
    return;
  }
  if (owner) st_coherent(partial + (b * P + p) * s1 + threadIdx.x, r);
  if (!last_block_ticket(counters + b, P, &flag)) return;
  if (owner) {
    T s = Op::init();
    for (unsigned q = 0; q < P; q++) s = Op::merge(s, ld_coherent(partial + (b * P + q) * s1 + threadIdx.x));
    y[b * s1 + threadIdx.x] = s;
  }
  if (threadIdx.x == 0) st_coherent(counters + b, 0u);
}

// ---- host-side planning ----------------------------------------------------------------------------
// Measured on MI355X (256 CUs): these HBM-bound reductions run fastest when a launch has about one
// large workgroup per CU and no second stage; every extra split costs 2-4 us of ticket traffic and every
// extra round of workgroups a partial tail.  So: no split while the outputs alone give at least half a
// workgroup per CU; otherwise split until there is about one workgroup per CU, as long as each part keeps
// enough loads per lane to cover the memory latency.
inline long ceil_div(long a, long b) { return (a + b - 1) / b; }

inline unsigned plan_parts(long groups, long units_per_group, long min_units_per_wg) {
  const long ncu = tuning(kTuneNumCUs);
  long P = 1;
  if (groups * 2 <= ncu) P = ceil_div(ncu, groups);
  const long cap = units_per_group / min_units_per_wg;
  if (P > cap) P = cap;
  if (P > 65535) P = 65535;
  if (P < 1) P = 1;
  return (unsigned)P;
}

template <typename T, typename Op>
inline void launch_reduce_run(hipStream_t stream, const T* x, long sy, long ny, long no, T* y, const ScratchSource* scratch = nullptr) {
  if (ny <= 0) return;
  constexpr int N = Vec16<T>::N;
  const bool vec = aligned16(x) && (sy % N == 0);
  const int nv = vec ? N : 1;
  const long units = sy / nv * no;
  unsigned P = plan_parts(ny, units, 2048);
  long chunk = ceil_div(units, P);
  P = (unsigned)ceil_div(units, chunk > 0 ? chunk : 1);
  if (P < 1) P = 1;
  Workspace ws = {nullptr, nullptr};
  if (P > 1) {
    ws = take_scratch(scratch, stream, sizeof(T) * (size_t)ny * P, (size_t)ny);
    if (!scratch_ready(ws, "reduction: no scratch memory for a split launch")) return;
  }
  T* partial = static_cast<T*>(ws.partial);
  // workgroup size by the work of one part: a wave for short runs, 512 lanes when there is plenty
  const int bt = chunk <= 2 * kWave ? 64 : chunk <= 4096 ? 256 : 512;
  const dim3 grid((unsigned)(ny * P));
#define KNET8_RUN(NV, SINGLE, BT, U) \
  hipLaunchKernelGGL((reduce_run_kernel<T, Op, NV, SINGLE, BT, U>), grid, dim3(BT), 0, stream, x, sy, ny, units, chunk, P, y, partial, ws.counters)
  // (the scalar path, for runs that do not start on 16-byte boundaries, keeps four times as many loads in flight per lane to move the same bytes)
#define KNET8_RUN_BT(NV, SINGLE) \
  do { if (bt == 64) KNET8_RUN(NV, SINGLE, 64, (NV == 1 ? 16 : 8)); else if (bt == 256) KNET8_RUN(NV, SINGLE, 256, (NV == 1 ? 16 : 4)); \
       else KNET8_RUN(NV, SINGLE, 512, (NV == 1 ? 16 : 4)); } while (0)
  if (vec) { if (no == 1) KNET8_RUN_BT(N, true); else KNET8_RUN_BT(N, false); }
  else     { if (no == 1) KNET8_RUN_BT(1, true); else KNET8_RUN_BT(1, false); }
#undef KNET8_RUN_BT
#undef KNET8_RUN
}

template <typename T, typename Op>
inline void launch_reduce_strided(hipStream_t stream, const T* x, long s1, long d, long nb, T* y, const ScratchSource* scratch = nullptr) {
  if (s1 <= 0 || nb <= 0) return;
  constexpr int N = Vec16<T>::N;
  if (s1 < kWave) {
    const int reps = kRedBlock / (int)s1, L = reps * (int)s1;
    const long total = s1 * d;
    unsigned P = plan_parts(nb, ceil_div(total, L), 16);
    long chunk = ceil_div(ceil_div(total, L), P) * L;
    P = (unsigned)ceil_div(total, chunk > 0 ? chunk : 1);
    if (P < 1) P = 1;
    Workspace ws = {nullptr, nullptr};
    if (P > 1) {
      ws = take_scratch(scratch, stream, sizeof(T) * (size_t)nb * P * s1, (size_t)nb);
      if (!scratch_ready(ws, "reduction: no scratch memory for a split launch")) return;
    }
    hipLaunchKernelGGL((reduce_strided_small_kernel<T, Op>), dim3((unsigned)(nb * P)), dim3(kRedBlock), 0, stream, x, (int)s1, d,
                       chunk, P, y, static_cast<T*>(ws.partial), ws.counters);
    return;
  }
  const bool vec = aligned16(x) && (s1 % N == 0);
  // rows that do not start on 16-byte boundaries: the same tile width from N interleaved 4- or 8-byte loads per lane
  const long tile = (long)kWave * N;
  const long atiles = ceil_div(s1, tile);
  const long groups = atiles * nb;
  unsigned P = plan_parts(groups, d, 64);
  long kchunk = ceil_div(d, P);
  P = (unsigned)ceil_div(d, kchunk > 0 ? kchunk : 1);
  if (P < 1) P = 1;
  Workspace ws = {nullptr, nullptr};
  if (P > 1) {
    ws = take_scratch(scratch, stream, sizeof(T) * (size_t)groups * P * tile, (size_t)groups);
    if (!scratch_ready(ws, "reduction: no scratch memory for a split launch")) return;
  }
  const dim3 grid((unsigned)(groups * P));
  T* partial = static_cast<T*>(ws.partial);
  const bool big = kchunk >= 128;  // sixteen waves share a tile when each still gets >= 8 rows
#define KNET8_STR(NV, BT, U, SC) \
  hipLaunchKernelGGL((reduce_strided_kernel<T, Op, NV, BT, U, SC>), grid, dim3(BT), 0, stream, x, s1, d, atiles, kchunk, P, y, partial, ws.counters)
  if (vec) { if (big) KNET8_STR(N, 1024, 2, false); else KNET8_STR(N, 256, 8, false); }
  else     { if (big) KNET8_STR(N, 1024, 2, true); else KNET8_STR(N, 256, 8, true); }
#undef KNET8_STR
}

// `_21` contract: x[i] goes into y[(i/sy)%ny]  (src/libknet8/cuda21.jl:23).
template <typename T, typename Op>
inline void reduce_21(hipStream_t stream, long nx, const T* x, long sy, long ny, T* y, const ScratchSource* scratch = nullptr) {
  if (ny <= 0 || sy <= 0 || nx < 0) return;
  if (nx % (sy * ny) != 0) { record_error("reduce _21: nx is not a multiple of sy*ny"); return; }
  const long no = nx / (sy * ny);
  if (ny == 1) launch_reduce_run<T, Op>(stream, x, nx, 1, 1, y, scratch);
  else if (sy == 1) launch_reduce_strided<T, Op>(stream, x, ny, no, 1, y, scratch);
  else launch_reduce_run<T, Op>(stream, x, sy, ny, no, y, scratch);
}

// `_22` contract: output bi reduces x[lower + k*s1], k = 0..xd1, lower = bi%s1 + (bi/s1)*s2
// (src/libknet8/cuda22.jl:31-36); the dispatcher always passes s2 = s1*(xd1+1).
template <typename T, typename Op>
inline void reduce_22(hipStream_t stream, long nx, long xd1, const T* x, long s1, long s2, long ny, T* y) {
  (void)nx;
  if (ny <= 0 || s1 <= 0 || xd1 < 0) return;
  const long d = xd1 + 1;
  if (s2 != s1 * d || ny % s1 != 0) { record_error("reduce _22: expected s2 == s1*(xd1+1) and ny a multiple of s1"); return; }
  if (s1 == 1) launch_reduce_run<T, Op>(stream, x, d, ny, 1, y);
  else launch_reduce_strided<T, Op>(stream, x, s1, d, ny / s1, y);
}

}  // namespace knet8
