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
// Short runs and short contiguous axes (a (10, N) matrix summed over its columns, a (2, N) matrix over its rows) go to a third kernel that reads
// stretches of neighbouring runs or of whole slabs (reduce_stretch_kernel).
//
// All split the reduced axis over P workgroups per output group when one group alone would leave the
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
// Merged: the operator that combines values to which item() has been applied already (partial results of a first pass).
template <typename T> struct RedSum     { typedef RedSum<T> Merged; __host__ __device__ static T init() { return T(0); } __device__ static T item(T x) { return x; } __device__ static T merge(T a, T x) { return a + x; } };
template <typename T> struct RedProd    { typedef RedProd<T> Merged; __host__ __device__ static T init() { return T(1); } __device__ static T item(T x) { return x; } __device__ static T merge(T a, T x) { return a * x; } };
template <typename T> struct RedMaximum { typedef RedMaximum<T> Merged; __host__ __device__ static T init() { return -INFINITY; } __device__ static T item(T x) { return x; } __device__ static T merge(T a, T x) { return a > x ? a : x; } };
template <typename T> struct RedMinimum { typedef RedMinimum<T> Merged; __host__ __device__ static T init() { return INFINITY; } __device__ static T item(T x) { return x; } __device__ static T merge(T a, T x) { return a < x ? a : x; } };
template <typename T> struct RedSumabs  { typedef RedSum<T> Merged; __host__ __device__ static T init() { return T(0); } __device__ static T item(T x) { return x < 0 ? -x : x; } __device__ static T merge(T a, T x) { return a + x; } };
template <typename T> struct RedSumabs2 { typedef RedSum<T> Merged; __host__ __device__ static T init() { return T(0); } __device__ static T item(T x) { return x * x; } __device__ static T merge(T a, T x) { return a + x; } };
template <typename T> struct RedMaxabs  { typedef RedMaximum<T> Merged; __host__ __device__ static T init() { return T(0); } __device__ static T item(T x) { return x < 0 ? -x : x; } __device__ static T merge(T a, T x) { return a > x ? a : x; } };
template <typename T> struct RedMinabs  { typedef RedMinimum<T> Merged; __host__ __device__ static T init() { return INFINITY; } __device__ static T item(T x) { return x < 0 ? -x : x; } __device__ static T merge(T a, T x) { return a < x ? a : x; } };
template <typename T> struct RedCountnz { typedef RedSum<T> Merged; __host__ __device__ static T init() { return T(0); } __device__ static T item(T x) { return x != 0 ? T(1) : T(0); } __device__ static T merge(T a, T x) { return a + x; } };

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
                                                               unsigned P, T* __restrict__ y, T* partial, unsigned* counters KNET8_TL_PARAM) {
  KNET8_TL_BEGIN
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
  KNET8_TL_MID
  if (P == 1) {
    if (threadIdx.x == 0) y[j] = r;
    KNET8_TL_END
    return;
  }
  if (threadIdx.x == 0) st_coherent(partial + j * P + p, r);
  if (!last_block_ticket(counters + j * kTicketStride, P, &flag)) { KNET8_TL_END return; }
  T s = Op::init();
  for (unsigned q = threadIdx.x; q < P; q += BT) s = Op::merge(s, ld_coherent(partial + j * P + q));
  s = block_reduce<T, NW>(s, lds, MergeFn<Op, T>(), Op::init());
  if (threadIdx.x == 0) {
    y[j] = s;
    st_coherent(counters + j * kTicketStride, 0u);
  }
  KNET8_TL_END
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

// Rows of partial results a wave of the combining workgroup has in flight at once: with many parts (a tile split 256 ways is 16 rows per wave) two
// rows at a time are eight memory round trips in a row.
constexpr int kCombineU = 8;

template <typename T, typename Op, int NV, int BT, int U, bool SC = false>
__global__ __launch_bounds__(BT) void reduce_strided_kernel(const T* __restrict__ x, long s1, long d, long atiles, long kchunk,
                                                                   unsigned P, T* __restrict__ y, T* partial, unsigned* counters KNET8_TL_PARAM) {
  KNET8_TL_BEGIN
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
  KNET8_TL_MID
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
    if (!last_block_ticket(counters + group * kTicketStride, P, &flag)) { KNET8_TL_END return; }
#pragma unroll
    for (int e = 0; e < NV; e++) acc[e] = Op::init();
    strided_walk<T, Op, NV, false, NW, kCombineU, SC>(partial + group * P * TILE + (SC ? lane : lane * NV), TILE, 0, P, wave, acc);
    if (threadIdx.x == 0) st_coherent(counters + group * kTicketStride, 0u);
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
  KNET8_TL_END
}

// ---- stretches of short runs ------------------------------------------------------------------------
// Run view whose runs are short (sy of at most a few hundred elements), and the strided view with a short contiguous axis.  One wave per output
// would read a few bytes per lane and leave most lanes idle (run view), or have lanes read `s1` elements apart; instead a workgroup takes a
// STRETCH of E contiguous elements -- the runs of g neighbouring outputs (R = 1), or, when all ny outputs of a slab fit several times, R whole
// slabs (g = ny) -- so that wave instructions read whole cache lines whatever sy is.  Lane t holds elements (t + 256 q) NV .. +NV-1 of the stretch,
// q < U, and sums them over the stretches of its part, `iter_stride` elements apart; which output an element belongs to depends on its place in
// the stretch only: (i / sy) % g.  At the end the accumulators go to LDS and a team of TL lanes reduces the R*sy entries of each output.
// P workgroups split the iterations of a group; the last to finish combines their g-vectors in fixed order.
// O: stretches in flight per lane (1 for a launch whose workgroups have a single stretch each: the registers go to a longer stretch, U, instead).
template <typename T, typename Op, int NV, int U, int O>
__global__ __launch_bounds__(kRedBlock) void reduce_stretch_kernel(const T* __restrict__ x, int sy, int g_full, long nout, int R, int TL, long group_stride,
                                                                  long iter_stride, long iters, long iters_per_part, long limit, unsigned P,
                                                                  T* __restrict__ y, T* partial, unsigned* counters KNET8_TL_PARAM) {
  KNET8_TL_BEGIN
  constexpr int CAP = kRedBlock * U * NV;
  __shared__ T lds[CAP + CAP / 32];
  __shared__ unsigned flag;
  const long group = blockIdx.x / P;
  const unsigned p = blockIdx.x % P;
  const long j0 = group * g_full;
  const int g = (int)(nout - j0 < g_full ? nout - j0 : g_full);   // outputs of this group (nout: outputs of the whole launch)
  const int E = R * g * sy;                                   // elements of one stretch
  const T* base = x + group * group_stride;
  const long t0 = (long)p * iters_per_part;
  long t1 = t0 + iters_per_part;
  if (t1 > iters) t1 = iters;
  T acc[U][NV];
#pragma unroll
  for (int q = 0; q < U; q++)
#pragma unroll
    for (int e = 0; e < NV; e++) acc[q][e] = Op::init();
  for (long t = t0; t < t1; t += O) {
    T v[O][U][NV];
#pragma unroll
    for (int o = 0; o < O; o++) {
      const long at = (t + o) * iter_stride;
#pragma unroll
      for (int q = 0; q < U; q++) {
        const int i = ((int)threadIdx.x + q * kRedBlock) * NV;
        if (t + o < t1 && i < E && at + i < limit) {
          if (NV > 1 && i + NV <= E && at + i + NV <= limit) {
            typedef typename Vec16<T>::type V;
            const V w = ld_stream(reinterpret_cast<const V*>(base + at + i));
#pragma unroll
            for (int e = 0; e < NV; e++) v[o][q][e] = Op::item(w[e]);
          } else if (NV > 1) {   // the last vector of a stretch that does not end on a vector boundary: element by element, nothing past the end is touched
#pragma unroll
            for (int e = 0; e < NV; e++) v[o][q][e] = (i + e < E && at + i + e < limit) ? Op::item(__builtin_nontemporal_load(base + at + i + e)) : Op::init();
          } else {
            v[o][q][0] = Op::item(__builtin_nontemporal_load(base + at + i));
          }
        } else {
#pragma unroll
          for (int e = 0; e < NV; e++) v[o][q][e] = Op::init();
        }
      }
    }
#pragma unroll
    for (int o = 0; o < O; o++)
#pragma unroll
      for (int q = 0; q < U; q++)
#pragma unroll
        for (int e = 0; e < NV; e++) acc[q][e] = Op::merge(acc[q][e], v[o][q][e]);
  }
  KNET8_TL_MID
  // one padding word per 32 entries: a team walks entries TL apart, neighbouring teams start sy apart
#pragma unroll
  for (int q = 0; q < U; q++)
#pragma unroll
    for (int e = 0; e < NV; e++) {
      const int i = ((int)threadIdx.x + q * kRedBlock) * NV + e;
      lds[i + (i >> 5)] = acc[q][e];
    }
  __syncthreads();
  const int nteams = kRedBlock / TL, team = (int)threadIdx.x / TL, tl = (int)threadIdx.x % TL;
  const int entries = R * sy;
  T* mine = P > 1 ? partial + (group * P + p) * g_full : y + j0;
  for (int jb = 0; jb < g; jb += nteams) {   // the same trip count for every lane of a wave: the shuffles below need all of them
    const int jl = jb + team;
    T r = Op::init();
    if (jl < g) {
      if (sy == 1) {   // (slabs of single elements, the strided view: entry c of output jl is element c*g + jl)
        for (int c = tl; c < entries; c += TL) {
          const int i = c * g + jl;
          r = Op::merge(r, lds[i + (i >> 5)]);
        }
      } else if (R == 1 && entries <= 2 * TL) {   // (one slab per stretch: no division per entry; runs of a few elements: at most two per lane)
        for (int c = tl; c < entries; c += TL) {
          const int i = jl * sy + c;
          r = Op::merge(r, lds[i + (i >> 5)]);
        }
      } else if (R == 1) {   // (longer runs: the first eight entries of a lane -- all of them up to runs of 512 -- are fetched together and merged in
                             //  order: written as one loop, every LDS read waits for the merge before it; 2^25 elements, cold: runs of 32 29.3 -> 26.7 us,
                             //  of 100 34.2 -> 30.8, of 256 29.9 -> 27.4)
        const int i0 = jl * sy + tl;
        T v[8];
#pragma unroll
        for (int k = 0; k < 8; k++) {
          const int i = i0 + k * TL;
          v[k] = tl + k * TL < entries ? lds[i + (i >> 5)] : Op::init();
        }
#pragma unroll
        for (int k = 0; k < 8; k++)
          if (tl + k * TL < entries) r = Op::merge(r, v[k]);
        for (int c = tl + 8 * TL; c < entries; c += TL) {
          const int i = jl * sy + c;
          r = Op::merge(r, lds[i + (i >> 5)]);
        }
      } else {
        for (int c = tl; c < entries; c += TL) {
          const int i = ((c / sy) * g + jl) * sy + c % sy;
          r = Op::merge(r, lds[i + (i >> 5)]);
        }
      }
    }
    for (int o = TL >> 1; o > 0; o >>= 1) r = Op::merge(r, __shfl_xor(r, o));
    if (jl < g && tl == 0) {
      if (P > 1) st_coherent(mine + jl, r);
      else mine[jl] = r;
    }
  }
  if (P == 1 || O == 1) { KNET8_TL_END return; }   // (O == 1: launches of one stretch per workgroup are never split; their registers stay what the walk needs)
  if (!last_block_ticket(counters + group * kTicketStride, P, &flag)) { KNET8_TL_END return; }
  // Combine: 256/gp lanes per output share the P partials (one lane alone would wait for P memory round trips in a row), 32 loads in flight each
  // (512 parts of 64 outputs are 128 partials per lane: four round trips instead of sixteen; (64, 512K) summed over the long axis 32.5 -> 29.4 us);
  // their sums meet in LDS in fixed order.
  int gp = 1;
  while (gp < g && gp < kRedBlock) gp <<= 1;
  const int tlc = kRedBlock / gp;
  for (int jb = 0; jb < g; jb += gp) {
    const int jl = jb + (int)threadIdx.x % gp;
    T r = Op::init();
    if (jl < g) {
      const T* pj = partial + group * P * g_full + jl;
      unsigned q = threadIdx.x / gp;
      constexpr int B = 32;
      for (; q + (B - 1) * tlc < P; q += B * tlc) {
        T v[B];
#pragma unroll
        for (int k = 0; k < B; k++) v[k] = ld_coherent(pj + (long)(q + k * tlc) * g_full);
#pragma unroll
        for (int k = 0; k < B; k++) r = Op::merge(r, v[k]);
      }
      for (; q + 7 * tlc < P; q += 8 * tlc) {
        T v[8];
#pragma unroll
        for (int k = 0; k < 8; k++) v[k] = ld_coherent(pj + (long)(q + k * tlc) * g_full);
#pragma unroll
        for (int k = 0; k < 8; k++) r = Op::merge(r, v[k]);
      }
      for (; q < P; q += tlc) r = Op::merge(r, ld_coherent(pj + (long)q * g_full));
    }
    __syncthreads();
    lds[threadIdx.x] = r;
    __syncthreads();
    if ((int)threadIdx.x < gp && jl < g) {
      T s = lds[threadIdx.x];
      for (int k = 1; k < tlc; k++) s = Op::merge(s, lds[threadIdx.x + k * gp]);
      y[j0 + jl] = s;
    }
  }
  if (threadIdx.x == 0) st_coherent(counters + group * kTicketStride, 0u);
  KNET8_TL_END
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
  if (groups * 2 <= ncu) P = ncu / groups;   // rounded down: one workgroup more than there are CUs would double the time of the CU that gets it
  const long cap = units_per_group / min_units_per_wg;
  if (P > cap) P = cap;
  if (P > 65535) P = 65535;
  if (P < 1) P = 1;
  return (unsigned)P;
}

// Parts of a split along an axis of d rows (or columns) per group, chosen by counting dependent memory round trips: a part's waves walk `per_trip` rows
// per trip (sixteen waves with two rows in flight, or four with eight), the ticket costs two trips, and the workgroup that combines reads 128 partial rows
// per trip when it has sixteen waves (parts of at least `big_from` rows) and 32 with four.  At most one workgroup per compute unit, parts of at least 16 rows.
inline unsigned plan_parts_by_trips(long groups, long d, long per_trip, long big_from) {
  const long ncu = tuning(kTuneNumCUs);
  long pmax = groups * 2 <= ncu ? ncu / groups : 1;
  if (pmax > d / 16) pmax = d / 16;
  if (pmax > 65535) pmax = 65535;
  auto trips = [&](long p) {
    const long rows = ceil_div(d, p);
    return ceil_div(rows, per_trip) + (p > 1 ? ceil_div(p, rows >= big_from ? 128 : 32) + 2 : 0);
  };
  long best = trips(1);
  unsigned P = 1;
  for (long p = 2; p <= pmax; p = (p * 2 <= pmax || p == pmax) ? p * 2 : pmax) {
    const long t = trips(p);
    if (t < best) { best = t; P = (unsigned)p; }
  }
  return P;
}

constexpr long kStretchMaxRun = 1024;   // longest run the stretch kernel takes

// Stretch kernel for x(sy, ny, no) -> y(ny) per batch (nb batches, `batch_stride` elements apart, outputs ny apart); sy*ny small enough for
// whole slabs (R >= 1 of them per stretch) or sy <= kStretchMaxRun.  Returns false if the shape is not one for it.
// `launched` (if given) is set to false when the shape was this kernel's but its split could not get scratch: nothing was written to y.
template <typename T, typename Op>
inline bool launch_reduce_stretch(hipStream_t stream, const T* x, long sy, long ny, long no, long nb, long batch_stride, T* y,
                                  const ScratchSource* scratch, bool* launched = nullptr) {
  if (launched) *launched = true;
  constexpr int N = Vec16<T>::N;
  constexpr int U1 = 4, UV = 2;      // accesses per lane and stretch, scalar and vector kernels
  constexpr int S1 = 16, SV = 4;     // the same for launches of one stretch per workgroup (one slab of short runs)
  const long slab = sy * ny;
  if (sy > kStretchMaxRun || slab <= 0 || no <= 0) return false;
  const bool whole = slab <= kRedBlock * U1 / 2;          // whole slabs, several per stretch (the scalar kernel's capacity decides: it must hold for both)
  if (!whole && nb != 1) return false;
  auto gcd = [](long a, long b) { while (b) { const long t = a % b; a = b; b = t; } return a; };
  // 16-byte loads: every stretch must start on a 16-byte boundary and no vector may reach past the end of the array
  bool vec = aligned16(x) && (nb == 1 || batch_stride % N == 0);
  int g, R;
  bool single = false;
  long groups, group_stride, iter_stride, iters, limit;
  if (whole) {
    vec = vec && (no * slab) % N == 0;
    const int cap = kRedBlock * (vec ? UV * N : U1);
    g = (int)ny;
    R = (int)(cap / slab);
    if (vec) { const long step = N / gcd(N, slab); R = (int)(R / step * step); }   // R*slab is a multiple of N
    if (R > no) R = (int)no;                                                       // a single stretch, at offset 0
    if (R < 1) return false;
    groups = nb; group_stride = batch_stride; iter_stride = R * slab; iters = ceil_div(no, R); limit = no * slab;
  } else {
    single = no == 1;
    vec = vec && (single || slab % N == 0);   // one slab: only the groups have to start on 16-byte boundaries (a last vector that would reach past the group is read element by element)
    const int cap = single ? kRedBlock * (vec ? SV * N : S1) : kRedBlock * (vec ? UV * N : U1);
    long G = cap / sy;
    if (vec) { const long step = N / gcd(N, sy); G = G / step * step; }   // groups start on 16-byte boundaries
    if (G < 1) return false;
    if (G > ny) G = ny;
    g = (int)G; R = 1;
    groups = ceil_div(ny, G); group_stride = G * sy; iter_stride = slab; iters = no; limit = 0x7fffffffffffffffL;
  }
  if (groups > 0x7fffffffL / 2) return false;
  const long entries = (long)R * sy;
  int TL = 1;
  while (TL < kWave && TL * 8 < entries) TL <<= 1;
  // parts: about two workgroups per compute unit, a minimum of stretches each (below), and the combining pass reads g*P partials.  Every workgroup is resident
  // from the start and all finish their stretches at about the same time; what follows (partial results written through, ticket, the last one's
  // combining pass) are memory round trips behind everybody else's last loads, and they get longer with the number of workgroups.  Stamps on
  // (8, 4M) and (32, 1M) summed over the long axis, cold: two per CU have their sums after 15-21 us and are done after 27-29 us, four per CU after 12-26 us
  // and 32-36 us; back to back (2..32 rows) x 2^25 elements: 33.5 / 31.6 / 44.0 / 32.6 us with one per CU, 30.1 / 28.0 / 34.9 / 30.1 with two, 33.1 / 33.0 / 36.6 / 37.4 with four.
  const long ncu = tuning(kTuneNumCUs);
  long P = 1;
  if (groups < 2 * ncu) P = 2 * ncu / groups;
  // (at least eight stretches per part; two in arrays of less than 8 MB, where the parts' walks are the longest thing in the launch: (10, 25000) 8.9 -> 7.5 us,
  //  (32, 1953) 8.0 -> 6.3, (2, 125000) 9.7 -> 7.9; from 16 MB on eight are faster, 12.4 against 14.6-15.6)
  const long per_part = sizeof(T) * (size_t)iters * (size_t)iter_stride * (size_t)groups < (size_t(8) << 20) ? 2 : 8;
  if (P > iters / per_part) P = iters / per_part;
  if (P * g > 65536) P = 65536 / g;
  if (P < 1 || !scratch_fits(scratch, sizeof(T) * (size_t)groups * P * g, (size_t)groups * kTicketStride)) P = 1;   // a provider of fixed size: no split beyond it
  long ipp = ceil_div(iters, P);
  P = ceil_div(iters, ipp);
  Workspace ws = {nullptr, nullptr};
  if (P > 1) {
    ws = take_scratch(scratch, stream, sizeof(T) * (size_t)groups * P * g, (size_t)groups * kTicketStride);
    if (!scratch_ready(ws, "reduction: no scratch memory for a split launch")) { if (launched) *launched = false; return true; }
  }
  const dim3 grid((unsigned)(groups * P));
#define KNET8_STRETCH(NV, U, O) \
  hipLaunchKernelGGL((reduce_stretch_kernel<T, Op, NV, U, O>), grid, dim3(kRedBlock), 0, stream, x, (int)sy, g, whole ? nb * ny : ny, R, TL, group_stride, \
                     iter_stride, iters, ipp, limit, (unsigned)P, y, static_cast<T*>(ws.partial), ws.counters KNET8_TL_ARG)
  if (single) { if (vec) KNET8_STRETCH(N, SV, 1); else KNET8_STRETCH(1, S1, 1); }
  else        { if (vec) KNET8_STRETCH(N, UV, 4); else KNET8_STRETCH(1, U1, 4); }
#undef KNET8_STRETCH
  return true;
}

// Both launchers return false when a launch that had to be split could not get its scratch memory: the error is recorded, nothing was
// launched and y is untouched.
template <typename T, typename Op>
inline bool launch_reduce_strided(hipStream_t stream, const T* x, long s1, long d, long nb, T* y, const ScratchSource* scratch = nullptr, size_t front = 0);

// The slab sums of the two-pass route below live in scratch memory (sy*ny elements): beyond this size the route is not taken, so that one
// odd call cannot pin hundreds of megabytes for as long as its stream lives.
constexpr size_t kTwoPassMaxBytes = size_t(32) << 20;

template <typename T, typename Op>
inline bool launch_reduce_run(hipStream_t stream, const T* x, long sy, long ny, long no, T* y, const ScratchSource* scratch = nullptr) {
  if (ny <= 0) return true;
  // Short runs.  One slab (a (2, 16M) matrix summed over its columns): one run per workgroup would read a few bytes per lane (3.5 ms); stretches of
  // neighbouring runs instead.  Many slabs (the bias gradient of a 7x7 feature map, x(49, 2048, N)): the slabs are first added onto each other as
  // rows of sy*ny contiguous elements by the strided-view kernel, into scratch, then the sy*ny sums are reduced as one slab; the sy*ny extra
  // elements written and read are nothing next to the no slabs.  (Measured, 134 MB fp32: (4,1000,8388) 158 -> 26.5 us, (49,2048,334) 43.7 -> 28.5 us, (16,16,131072) 35.9 -> 29.0 us.)
  // Neither pays below a size that grows with the run length: the two passes cost 8.5-9.5 us before the first byte (two launches, the first one split) and 0.13 us per MB
  // after it, the run kernel below 3.5 us and 2.3 / 1.5 / 0.6 / 0.45 / 0.34 us per MB at runs of 2 / 4 / 8 / 12 / 16 and more elements -- and the bias gradient of a
  // convolution layer is a few MB.  Measured crossovers (fp32, 512 outputs): runs of 2: 2.5 MB, 4: 4 MB, 8: 11 MB, 12: 15 MB, 16 to 63: 22-48 MB.  Below 1.25 MB per
  // element of the run (at most 24 MB) the array goes to the run kernel: x(16,512,128) 9.0 -> 3.8 us, x(49,512,64) 9.0 -> 6.3, x(4,512,61) 7.0 -> 3.7, x(8,512,122) 9.4 -> 4.0.
  const size_t total_bytes = sizeof(T) * (size_t)sy * (size_t)ny * (size_t)no;
  const size_t two_pass_from = sy < 20 ? (size_t)sy * 1310720 : (size_t(24) << 20);
  const bool small_total = no > 1 && sy < kWave && total_bytes < two_pass_from;
  const size_t front = (sizeof(T) * (size_t)(sy * ny) + 255) / 256 * 256;
  if (!small_total && ny > 1 && sy < kWave && no >= 8 && sy * ny >= kWave && front <= kTwoPassMaxBytes && scratch_fits(scratch, 2 * front, 0)) {
    Workspace tw = take_scratch(scratch, stream, front, 0);
    if (tw.partial == nullptr) { record_error("reduction: no scratch memory for the slab sums"); return false; }
    T* tmp = static_cast<T*>(tw.partial);
    // the second pass reads what the first wrote: it must not run on scratch the first pass never filled
    if (!launch_reduce_strided<T, Op>(stream, x, sy * ny, no, 1, tmp, scratch, front)) return false;
    return launch_reduce_run<T, typename Op::Merged>(stream, tmp, sy, ny, 1, y, scratch);
  }
  // (one slab: up to 256-element runs, measured against the run kernel below -- 129: 39 against 195 us, 256: 29.6 / 30.8, 384: 34 / 21.6 --, and up to
  //  1024 when the runs do not start on 16-byte boundaries, where the run kernel is down to 4-byte loads: 513: 39 against 56 us)
  constexpr int NR = Vec16<T>::N;
  const bool short_one_slab = no == 1 && (sy <= 256 || (sy <= kStretchMaxRun && (sy % NR != 0 || !aligned16(x))));
  bool launched = true;
  if (!small_total && ny > 1 && (sy <= 8 || short_one_slab) && launch_reduce_stretch<T, Op>(stream, x, sy, ny, no, 1, 0, y, scratch, &launched)) return launched;
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
    ws = take_scratch(scratch, stream, sizeof(T) * (size_t)ny * P, (size_t)ny * kTicketStride);
    if (!scratch_ready(ws, "reduction: no scratch memory for a split launch")) return false;
  }
  T* partial = static_cast<T*>(ws.partial);
  // workgroup size by the work of one part: a wave for short runs, 512 lanes when there is plenty
  const int bt = chunk <= 2 * kWave ? 64 : chunk <= 4096 ? 256 : 512;
  const dim3 grid((unsigned)(ny * P));
#define KNET8_RUN(NV, SINGLE, BT, U) \
  hipLaunchKernelGGL((reduce_run_kernel<T, Op, NV, SINGLE, BT, U>), grid, dim3(BT), 0, stream, x, sy, ny, units, chunk, P, y, partial, ws.counters KNET8_TL_ARG)
  // (the scalar path, for runs that do not start on 16-byte boundaries, keeps four times as many loads in flight per lane to move the same bytes)
#define KNET8_RUN_BT(NV, SINGLE) \
  do { if (bt == 64) KNET8_RUN(NV, SINGLE, 64, (NV == 1 ? 16 : 8)); else if (bt == 256) KNET8_RUN(NV, SINGLE, 256, (NV == 1 ? 16 : 4)); \
       else KNET8_RUN(NV, SINGLE, 512, (NV == 1 ? 16 : 4)); } while (0)
  if (vec) { if (no == 1) KNET8_RUN_BT(N, true); else KNET8_RUN_BT(N, false); }
  else     { if (no == 1) KNET8_RUN_BT(1, true); else KNET8_RUN_BT(1, false); }
#undef KNET8_RUN_BT
#undef KNET8_RUN
  return true;
}

// `front`: bytes at the start of the scratch memory that belong to the caller (the partial results go behind them).
template <typename T, typename Op>
inline bool launch_reduce_strided(hipStream_t stream, const T* x, long s1, long d, long nb, T* y, const ScratchSource* scratch, size_t front) {
  if (s1 <= 0 || nb <= 0) return true;
  constexpr int N = Vec16<T>::N;
  // a short contiguous axis: lanes along `a` alone would idle most of a wave; whole (s1 x R) slabs per stretch instead
  bool launched = true;
  // By the bytes of a row: up to 128 always; up to 192 (256) in arrays of at least 48 (96) MB -- in smaller ones, and for longer rows, the strided kernel below with its
  // parts planned by round trips is faster.  Measured, stretches / strided kernel, fp32: 32 columns x 4 MB 9.1 / 8.2 us, x 16 MB 12.3 / 13.6, x 134 MB 27.9 / 52.7;
  // 48 x 4 MB 9.1 / 7.5, x 64 MB 22.1 / 23.2, x 134 MB 31.8 / 39.1; 64 x 16 MB 13.2 / 11.4, x 64 MB 21.1 / 20.1, x 134 MB 29.2 / 32.3; 72 x 134 MB 34.1 / 30.5;
  // fp64: 16 x 16 MB 12.1 / 13.7; 24 x 16 MB 12.4 / 12.0, x 64 MB 21.6 / 23.1; 32 x 64 MB 21.3 / 20.1, x 134 MB 28.8 / 32.3; 48 x 134 MB 33.2 / 26.8.
  const size_t row_bytes = (size_t)s1 * sizeof(T), array_bytes = row_bytes * (size_t)d * (size_t)nb;
  const bool short_axis = row_bytes <= 128 || (row_bytes <= 192 && array_bytes >= (size_t(48) << 20)) || (row_bytes <= 256 && array_bytes >= (size_t(96) << 20));
  if (short_axis && launch_reduce_stretch<T, Op>(stream, x, 1, s1, d, nb, s1 * d, y, scratch, &launched)) return launched;
  const bool vec = aligned16(x) && (s1 % N == 0);
  // rows that do not start on 16-byte boundaries: the same tile width from N interleaved 4- or 8-byte loads per lane
  const long tile = (long)kWave * N;
  const long atiles = ceil_div(s1, tile);
  const long groups = atiles * nb;
  // Parts per tile, counted in memory round trips (plan_parts_by_trips): few parts of long walks and many parts with a long combining pass both lose:
  // (256, 8192) 8.6 us with 128 parts, 7.0 with 64, 11.8 with 256; (1000, 128) 5.3 us with 2 parts, 4.6 with 4, 4.8 with 1; (4096, 512) 5.9 -> 5.4.
  // Large arrays end up where the bound of one workgroup per compute unit puts them, as before.
  unsigned P = plan_parts_by_trips(groups, d, 32, 128);
  long kchunk = ceil_div(d, P);
  P = (unsigned)ceil_div(d, kchunk > 0 ? kchunk : 1);
  if (P < 1) P = 1;
  Workspace ws = {nullptr, nullptr};
  if (P > 1) {
    ws = take_scratch(scratch, stream, front + sizeof(T) * (size_t)groups * P * tile, (size_t)groups * kTicketStride);
    if (!scratch_ready(ws, "reduction: no scratch memory for a split launch")) return false;
  }
  const dim3 grid((unsigned)(groups * P));
  T* partial = reinterpret_cast<T*>(static_cast<char*>(ws.partial) + (ws.partial ? front : 0));
  const bool big = kchunk >= 128;  // sixteen waves share a tile when each still gets >= 8 rows
#define KNET8_STR(NV, BT, U, SC) \
  hipLaunchKernelGGL((reduce_strided_kernel<T, Op, NV, BT, U, SC>), grid, dim3(BT), 0, stream, x, s1, d, atiles, kchunk, P, y, partial, ws.counters KNET8_TL_ARG)
  // A row of at most 512 bytes occupies at most half of a wave's 16-byte lanes: four rows in flight per wave instead of two make up for the idle ones
  // (2^25 fp32 elements, cold: 76 columns 40.3 -> 30.1 us, 100 34.0 -> 26.7, 128 29.3 -> 25.9; from 200 columns on two rows are as fast or faster, eight never better than four).
  const bool narrow = (size_t)s1 * sizeof(T) <= 512;
  if (vec) { if (big && narrow) KNET8_STR(N, 1024, 4, false); else if (big) KNET8_STR(N, 1024, 2, false); else KNET8_STR(N, 256, 8, false); }
  else     { if (big) KNET8_STR(N, 1024, 2, true); else KNET8_STR(N, 256, 8, true); }
#undef KNET8_STR
  return true;
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
