// Column softmax family: softmax / logsoftmax forward and backward and the fused nll+logsoftmax backward
// down each contiguous column of an m x n column-major matrix (the reference's dims=1 case).
//
// The reference sends these to cuDNN (src/ops20_gpu/softmax.jl:44-56, LOG/ACCURATE algorithms,
// MODE_INSTANCE on a (1,1,m,n) view); the arithmetic restated here is its CPU path
// (src/ops20/softmax.jl:42-63), to which the reference's own tests pin cuDNN (test/loss.jl:87-92).
//
// One "team" of lanes owns a column and keeps it in registers, so every operand is read from HBM exactly
// once and the result written once: the column is loaded with 16-byte vectors, reduced (max, then sum)
// with wave64 butterflies (+ LDS across waves), transformed and stored.  Team size follows the column
// length: one wave (m <= 1024), a 256-thread workgroup or a 1024-thread workgroup (up to 65536 rows in fp32, half
// of that when two inputs are held or in fp64; the table is in launch_softmax); longer columns fall back to a
// two-pass streaming kernel.
//
// HBM roofline: forward 2*sizeof(T)*m*n; backward 3*sizeof(T)*m*n; fused nll backward 2*sizeof(T)*m*n.
#pragma once
#include "knet8_device.h"
#include "knet8_runtime.h"

namespace knet8 {

// Workgroup size used when one wave owns a column (several columns per workgroup).
#ifndef KNET8_WAVE_TEAM_BLOCK
#define KNET8_WAVE_TEAM_BLOCK 256
#endif
constexpr int kWaveTeamBlock = KNET8_WAVE_TEAM_BLOCK;

// exp for the softmax family.  fp32 uses the hardware 2^x unit (v_exp_f32, 1 ulp) on a pre-scaled argument: the
// only extra error is the rounding of x*log2(e), about |x| * 6e-8 relative -- two orders of magnitude inside the
// 1e-5 contract of these kernels -- and it costs 2 instructions instead of the ~20 of the correctly rounded expf.
// With a 32000-row column resident per workgroup the exp work is not hidden behind memory traffic (only two columns
// fit in a CU's registers, so load, compute and store phases run in lock-step), so this is measurable wall time.
// The elementwise activation kernels, whose contract is 2 ulp, keep the precise expf.
template <typename T> __device__ __forceinline__ T dev_exp(T x);
template <> __device__ __forceinline__ float dev_exp<float>(float x) { return __builtin_amdgcn_exp2f(x * 1.4426950408889634f); }
template <> __device__ __forceinline__ double dev_exp<double>(double x) { return exp(x); }
template <typename T> __device__ __forceinline__ T dev_log(T x);
template <> __device__ __forceinline__ float dev_log<float>(float x) { return logf(x); }
template <> __device__ __forceinline__ double dev_log<double>(double x) { return log(x); }

// ---- algorithms -------------------------------------------------------------------------------------
// a, b: the (up to) two inputs.  kInputs==1: a = x.  kInputs==2: a = y, b = dy.
// kHoldA: a must stay in registers between the reduction and the output pass (false: it is only needed in
// the output pass and is streamed there).  term(): summand of the column sum.  out(): the result.  kKeepTerm: the summand
// replaces a in its register and the result is out_kept(term, fin) -- one exp per element instead of two, same bits.

// y = (x - max) - log(sum(exp(x - max)))                      src/ops20/softmax.jl:42-47
template <typename T> struct AlgoLogSoftmax {
  static constexpr int kInputs = 1; static constexpr bool kNeedMax = true, kHoldA = true, kNll = false, kKeepTerm = false;
  __device__ static T term(T a, T, T mx) { return dev_exp(a - mx); }
  __device__ static T finish(T s) { return dev_log(s); }
  __device__ static T out(T a, T, T mx, T fin) { return (a - mx) - fin; }
};
// y = exp(x - max) / sum(exp(x - max))                          src/ops20/softmax.jl:53-59
template <typename T> struct AlgoSoftmax {
  static constexpr int kInputs = 1; static constexpr bool kNeedMax = true, kHoldA = true, kNll = false, kKeepTerm = true;
  __device__ static T term(T a, T, T mx) { return dev_exp(a - mx); }
  __device__ static T finish(T s) { return s; }
  __device__ static T out(T a, T, T mx, T fin) { return dev_exp(a - mx) / fin; }
  __device__ static T out_kept(T t, T fin) { return t / fin; }
};
// dx = dy - exp(y)*sum(dy)                                      src/ops20/softmax.jl:49-51
template <typename T> struct AlgoLogSoftmaxBack {
  static constexpr int kInputs = 2; static constexpr bool kNeedMax = false, kHoldA = false, kNll = false, kKeepTerm = false;
  __device__ static T term(T, T b, T) { return b; }
  __device__ static T finish(T s) { return s; }
  __device__ static T out(T a, T b, T, T fin) { const T e = dev_exp(a); const T p = e * fin; return b - p; }
};
// dx = y*dy - y*sum(y*dy)                                       src/ops20/softmax.jl:61-63
template <typename T> struct AlgoSoftmaxBack {
  static constexpr int kInputs = 2; static constexpr bool kNeedMax = false, kHoldA = true, kNll = false, kKeepTerm = false;
  __device__ static T term(T a, T b, T) { return a * b; }
  __device__ static T finish(T s) { return s; }
  __device__ static T out(T a, T b, T, T fin) { const T p = a * b; const T q = a * fin; return p - q; }
};
// Fused nll backward on raw scores: with lsm = logsoftmax(x) and dlp = -scale at the labelled row of each
// counted column (0 elsewhere), dx = dlp - exp(lsm)*sum(dlp) -- the chain nll -> getindex -> logsoftmax of
// src/ops20/loss.jl:37-41 and src/ops20/softmax.jl:49-51 -- and loss[col] = -lsm[label].  Label 0 skips
// the column (dx = 0, loss = 0), as findindices does (src/ops20/loss.jl:125).
template <typename T> struct AlgoNll {
  static constexpr int kInputs = 1; static constexpr bool kNeedMax = true, kHoldA = true, kNll = true, kKeepTerm = false;
  __device__ static T term(T a, T, T mx) { return dev_exp(a - mx); }
  __device__ static T finish(T s) { return dev_log(s); }
  __device__ static T out(T a, T, T mx, T fin) { return (a - mx) - fin; }  // lsm; the kernel finishes the job
};

struct MaxFn { template <typename T> __device__ __forceinline__ T operator()(T a, T b) const { return a > b ? a : b; } };
struct AddFn { template <typename T> __device__ __forceinline__ T operator()(T a, T b) const { return a + b; } };

template <typename T, int TEAM, typename Merge>
__device__ __forceinline__ T team_reduce(T v, T* lds, Merge merge, T identity) {
  if (TEAM == kWave) return wave_reduce(v, merge);
  return block_reduce<T, TEAM / kWave>(v, lds, merge, identity);
}

// ---- register-resident column kernel -----------------------------------------------------------------
// TEAM lanes per column (64: four columns per 256-thread workgroup; 256 or 1024: the whole workgroup),
// E elements of each held input per lane, VEC: 16-byte accesses.
//
// Columns need not start on a 16-byte boundary (m odd: vocabularies of 50257 or 10001 classes): with VEC each column is
// cut into `head` elements up to its first aligned address, `nb` whole vectors and `tail` elements.  Lane tl of the team owns
// vectors tl, tl+TEAM, ...; the at most N-1 head and N-1 tail elements live in one extra register each of lanes 0..N-2.  All
// operands of a call must be congruent modulo 16 bytes (they then are in every column, the column length being common).
template <typename T, int NV>
__device__ __forceinline__ void cut_column(const T* p, int m, int& head, int& nb, int& tail) {
  if (NV == 1) { head = 0; nb = m; tail = 0; return; }
  const int mis = (int)((reinterpret_cast<uintptr_t>(p) / sizeof(T)) % NV);
  head = (NV - mis) % NV;
  if (head > m) head = m;
  nb = (m - head) / NV;
  tail = m - head - nb * NV;
}

// LV > 0 (single-input algorithms): the last LV of a lane's ITEMS vectors live in LDS (slot j of lane t at held[j*BT + t]: 16 bytes per lane,
// neighbours adjacent) instead of registers, filled by loads that go from memory to LDS directly.  A 32000-row fp64 column is 256 KB: held in
// registers alone it takes the whole register file of a compute unit -- one workgroup per CU, two rounds of workgroups for 512 columns; with 512
// lanes holding 23 vectors in registers and 9 in LDS each (72 KB per workgroup), two columns are resident per CU.
template <typename T, typename Algo, int TEAM, int E, bool VEC, int LV>
__device__ __forceinline__ void softmax_col_body(int m, long n, const T* a, const T* b, T* out KNET8_TL_PARAM) {
  KNET8_TL_BEGIN
  // Short columns (one wave each, few registers): load every input up front even if it is only needed for the
  // output pass, so the dependent chain is one memory round trip instead of two.
  constexpr bool kHold = Algo::kHoldA || (TEAM == kWave && E <= 16);
  constexpr bool kTwo = Algo::kInputs == 2;
  constexpr int BT = TEAM == kWave ? kWaveTeamBlock : TEAM;
  constexpr int TEAMS = BT / TEAM;
  constexpr int NV = VEC ? Vec16<T>::N : 1;
  constexpr int ITEMS = E / NV;
  constexpr int RI = ITEMS - LV;   // vectors per lane in registers
  static_assert(LV == 0 || (VEC && TEAMS == 1 && RI > 0 && kHold && !kTwo), "LDS slots: whole-workgroup teams of 16-byte vectors, one input");
  typedef typename Vec16<T>::type V;
  __shared__ T lds[BT / kWave];
  __shared__ V held[LV > 0 ? LV * BT : 1];
  V* const mine = held + threadIdx.x;
  const int tl = threadIdx.x % TEAM;
  const long col = (long)blockIdx.x * TEAMS + threadIdx.x / TEAM;
  const bool colok = col < n;  // only wave teams can be out of range
  const long base = colok ? col * (long)m : 0;
  const T* ac = a + base;
  const T* bc = kTwo ? b + base : nullptr;
  T* oc = out + base;
  int head, nb, tail;
  cut_column<T, NV>(ac, m, head, nb, tail);
  int cnt = (nb - tl + TEAM - 1) / TEAM;  // this lane's share of the nb vectors: the first `cnt` of its ITEMS slots
  cnt = !colok || cnt < 0 ? 0 : cnt;
  const bool hv = NV > 1 && colok && tl < head, tv = NV > 1 && colok && tl < tail;  // this lane holds a head / a tail element
  const int tpos = head + nb * NV + tl;                                         // where its tail element sits

  // a slot beyond the lane's share stays unwritten and is never read
#pragma unroll
  for (int j = 0; j < LV; j++)
    if (RI + j < cnt)
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(ac + head + (long)(tl + (RI + j) * TEAM) * NV),
                                       (__attribute__((address_space(3))) void*)(held + j * BT + (threadIdx.x & ~(kWave - 1))), 16, 0, 2);
  V ra[kHold ? RI : 1], rb[kTwo ? RI : 1];
  T ah = T(0), at = T(0), bh = T(0), bt = T(0);
#ifndef KNET8_LOAD_PACE
#define KNET8_LOAD_PACE 1
#endif
  constexpr bool kPacedLoads = KNET8_LOAD_PACE != 0 && !kHold && TEAM == 1024 && RI >= 4 && sizeof(T) == 4;   // (an fp64 column of this length has its compute unit to itself)
#pragma unroll
  for (int i = 0; i < RI; i++) {
    const long r = head + (long)(tl + i * TEAM) * NV;
    if (i < cnt) {
      if (VEC) {
        if (kHold) ra[i] = ld_stream(reinterpret_cast<const V*>(ac + r));
        if (kTwo) rb[i] = ld_stream(reinterpret_cast<const V*>(bc + r));
      } else {
        if (kHold) ra[i][0] = __builtin_nontemporal_load(ac + r);
        if (kTwo) rb[i][0] = __builtin_nontemporal_load(bc + r);
      }
    }
    // Long columns whose second operand is streamed later (logsoftmaxback): the held operand is requested two vectors at a time.  With all eight
    // requested at once the two workgroups of a compute unit are served one after the other -- the first has its column after 5 us, the second
    // after 13-22 -- and finish that far apart; in pairs their requests interleave and both have their sums by 10-11 us.  (32000 rows fp32, cold:
    // 33.9 -> 33.6 us on top of the batched output pass, which took it from 35.2 to 33.9.)
    if (kPacedLoads && (i + 1) % 2 == 0 && i + 1 < RI) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  }
  if (NV > 1) {
    if (hv) { ah = ac[tl]; if (kTwo) bh = bc[tl]; }
    if (tv) { at = ac[tpos]; if (kTwo) bt = bc[tpos]; }
  }
  T mx = T(0);
  if (Algo::kNeedMax) {
    mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < RI; i++)
      if (i < cnt) {
#pragma unroll
        for (int e = 0; e < NV; e++) mx = mx > ra[i][e] ? mx : ra[i][e];
      }
    if (LV > 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the direct loads are invisible to the compiler's own bookkeeping
#pragma unroll
    for (int j = 0; j < LV; j++)
      if (RI + j < cnt) {
        const V v = mine[j * BT];
#pragma unroll
        for (int e = 0; e < NV; e++) mx = mx > v[e] ? mx : v[e];
      }
    if (hv) mx = mx > ah ? mx : ah;
    if (tv) mx = mx > at ? mx : at;
    mx = team_reduce<T, TEAM>(mx, lds, MaxFn(), T(-INFINITY));
  }
  T s = T(0);
#pragma unroll
  for (int i = 0; i < RI; i++)
    if (i < cnt) {
#pragma unroll
      for (int e = 0; e < NV; e++) {
        const T t = Algo::term(kHold ? ra[i][e] : T(0), kTwo ? rb[i][e] : T(0), mx);
        if constexpr (Algo::kKeepTerm && kHold) ra[i][e] = t;
        s = s + t;
      }
    }
  if (LV > 0 && !Algo::kNeedMax) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
  for (int j = 0; j < LV; j++)
    if (RI + j < cnt) {
      V v = mine[j * BT];
#pragma unroll
      for (int e = 0; e < NV; e++) {
        const T t = Algo::term(v[e], T(0), mx);
        if constexpr (Algo::kKeepTerm && kHold) v[e] = t;
        s = s + t;
      }
      if constexpr (Algo::kKeepTerm && kHold) mine[j * BT] = v;
    }
  if (hv) { const T t = Algo::term(ah, bh, mx); if constexpr (Algo::kKeepTerm) ah = t; s = s + t; }
  if (tv) { const T t = Algo::term(at, bt, mx); if constexpr (Algo::kKeepTerm) at = t; s = s + t; }
  s = team_reduce<T, TEAM>(s, lds, AddFn(), T(0));
  const T fin = Algo::finish(s);
  KNET8_TL_MID
  // An operand that is only needed here (logsoftmaxback's y) is fetched kStreamBatch vectors at a time, all requested before the first of them is
  // used.  Written as load / use / store per vector, every load waits for the store before it as well (loads and stores share one counter, and a
  // wait on a mixed counter is a wait for all of it): eight dependent memory round trips per lane, during which a workgroup cannot take the
  // bandwidth that workgroups which are already done have freed.  A batch is one branch and one wait: its loads are unconditional (a lane whose
  // share ends inside the batch reads its last vector again instead) and only the stores are guarded.
#ifndef KNET8_STREAM_BATCH
#define KNET8_STREAM_BATCH 4
#endif
  constexpr int kStreamBatch = (!kHold && LV == 0 && ITEMS >= KNET8_STREAM_BATCH) ? KNET8_STREAM_BATCH : 1;   // (columns of two vectors per lane measured slower batched: 4000 rows 18.5 -> 20.9 us)
  if constexpr (kStreamBatch > 1) {
#pragma unroll
    for (int i0 = 0; i0 < ITEMS; i0 += kStreamBatch) {
      if (i0 < cnt) {
        V sa[kStreamBatch];
#pragma unroll
        for (int j = 0; j < kStreamBatch; j++) {
          const int ii = i0 + j < cnt ? i0 + j : cnt - 1;
          const long r = head + (long)(tl + ii * TEAM) * NV;
          if (VEC) sa[j] = ld_stream(reinterpret_cast<const V*>(ac + r));
          else sa[j][0] = __builtin_nontemporal_load(ac + r);
        }
#pragma unroll
        for (int j = 0; j < kStreamBatch; j++) {
          const int i = i0 + j;
          if (i < ITEMS) {
            const long r = head + (long)(tl + i * TEAM) * NV;
            V vo;
#pragma unroll
            for (int e = 0; e < NV; e++) vo[e] = Algo::out(sa[j][e], kTwo ? rb[kTwo && i < RI ? i : 0][e] : T(0), mx, fin);
            if (i < cnt) {
              if (VEC) st_stream(reinterpret_cast<V*>(oc + r), vo);
              else __builtin_nontemporal_store(vo[0], oc + r);
            }
          }
        }
      }
    }
  } else {
#pragma unroll
    for (int i = 0; i < ITEMS; i++) {
      if (i >= cnt) continue;
      const long r = head + (long)(tl + i * TEAM) * NV;
      V va = {}, vb = {};
      if (i < RI) {
        if (kHold) va = ra[kHold && i < RI ? i : 0];
        if (kTwo) vb = rb[kTwo && i < RI ? i : 0];
      } else {
        va = mine[(i - RI) * BT];
      }
      if (!kHold) {
        if (VEC) va = ld_stream(reinterpret_cast<const V*>(ac + r));
        else va[0] = __builtin_nontemporal_load(ac + r);
      }
      V vo;
#pragma unroll
      for (int e = 0; e < NV; e++) {
        if constexpr (Algo::kKeepTerm && kHold) vo[e] = Algo::out_kept(va[e], fin);
        else vo[e] = Algo::out(va[e], kTwo ? vb[e] : T(0), mx, fin);
      }
      if (VEC) st_stream(reinterpret_cast<V*>(oc + r), vo);
      else __builtin_nontemporal_store(vo[0], oc + r);
    }
  }
  if (NV > 1) {
    // a streamed (not held) first input was read above as ah/at all the same: the extras are always held
    if (hv) { if constexpr (Algo::kKeepTerm) oc[tl] = Algo::out_kept(ah, fin); else oc[tl] = Algo::out(ah, bh, mx, fin); }
    if (tv) { if constexpr (Algo::kKeepTerm) oc[tpos] = Algo::out_kept(at, fin); else oc[tpos] = Algo::out(at, bt, mx, fin); }
  }
  KNET8_TL_END
}

template <typename T, typename Algo, int TEAM, int E, bool VEC>
__global__ __launch_bounds__(TEAM == kWave ? kWaveTeamBlock : TEAM) void softmax_col_kernel(int m, long n, const T* a, const T* b, T* out KNET8_TL_PARAM) {
  softmax_col_body<T, Algo, TEAM, E, VEC, 0>(m, n, a, b, out KNET8_TL_PASS);
}
// four waves per SIMD (two 512-lane workgroups per compute unit): at most 128 registers per lane
template <typename T, typename Algo, int TEAM, int E, int LV>
__global__ __launch_bounds__(TEAM) __attribute__((amdgpu_waves_per_eu(4, 4))) void softmax_col_lds_kernel(int m, long n, const T* a, const T* b, T* out) {
  softmax_col_body<T, Algo, TEAM, E, true, LV>(m, n, a, b, out KNET8_TL_NONE);
}

// ---- fused nll + logsoftmax backward, register-resident, single reduction ---------------------------------
// The generic kernel above needs two workgroup-wide reductions (max, then sum of exp) and two exp per element.
// Here each lane first reduces its own elements (local max m_t, e_i = exp(a_i - m_t) kept in the registers that
// held a_i, s_t = sum e_i); the (max, sum) pairs are merged in ONE reduction with
// (m1,s1)+(m2,s2) = (M, s1*exp(m1-M) + s2*exp(m2-M)), M = max(m1,m2); then softmax_i = e_i * exp(m_t-M)/S is a
// single multiply per element.  One exp per element, one barrier phase less: the long serial tail of the
// 32000-row columns shrinks, which matters because only two such columns fit in the registers of a CU at a time.
// Rounding differs from the step-by-step formula by a few 1e-7 relative, inside the 1e-5 contract.
template <typename T> struct MaxSum { T m, s; };
template <typename T> __device__ __forceinline__ MaxSum<T> ms_merge(MaxSum<T> a, MaxSum<T> b) {
  const T M = a.m > b.m ? a.m : b.m;
  const T sa = a.m == M ? a.s : a.s * dev_exp(a.m - M);
  const T sb = b.m == M ? b.s : b.s * dev_exp(b.m - M);
  MaxSum<T> r = {M, sa + sb};
  return r;
}
// Over a wave: the max first, one rescaling of the lane's sum to it, then the sums -- one exp per lane instead of two per butterfly step.
template <typename T> __device__ __forceinline__ MaxSum<T> ms_wave_reduce(MaxSum<T> v) {
  const T M = wave_reduce(v.m, [](T a, T b) { return a > b ? a : b; });
  const T s = v.m == M ? v.s : v.s * dev_exp(v.m - M);   // a lane holding only -inf padding has s = 0: 0 * exp(-inf) = 0
  MaxSum<T> r = {M, wave_reduce(s, [](T a, T b) { return a + b; })};
  return r;
}

// The labelled logit is re-read by lane 0 of the team (one scalar load, issued with the others) instead of being
// fished out of the register that happens to hold it.  Columns are cut into head / vectors / tail as in softmax_col_kernel.
// LV > 0: the last LV vectors of each lane live in LDS, as in softmax_col_body.
template <typename T, int TEAM, int E, bool VEC, int LV>
__device__ __forceinline__ void nll_col_body(int m, long n, const T* a, T* out, const int* labels, T scale, T* loss KNET8_TL_PARAM) {
  KNET8_TL_BEGIN
  constexpr int BT = TEAM == kWave ? kWaveTeamBlock : TEAM;
  constexpr int TEAMS = BT / TEAM;
  constexpr int NW = TEAM / kWave;
  constexpr int NV = VEC ? Vec16<T>::N : 1;
  constexpr int ITEMS = E / NV;
  constexpr int RI = ITEMS - LV;   // vectors per lane in registers
  static_assert(LV == 0 || (VEC && TEAMS == 1 && RI > 0), "LDS slots: whole-workgroup teams of 16-byte vectors only");
  typedef typename Vec16<T>::type V;
  __shared__ T lds_m[BT / kWave], lds_s[BT / kWave];
  __shared__ V held[LV > 0 ? LV * BT : 1];
  V* const mine = held + threadIdx.x;
  const int tl = threadIdx.x % TEAM;
  const long col = (long)blockIdx.x * TEAMS + threadIdx.x / TEAM;
  const bool colok = col < n;
  const T* ac = a + (colok ? col * (long)m : 0);
  T* oc = out + (colok ? col * (long)m : 0);
  int head, nb, tail;
  cut_column<T, NV>(ac, m, head, nb, tail);
  int cnt = (nb - tl + TEAM - 1) / TEAM;
  cnt = !colok || cnt < 0 ? 0 : cnt;
  const bool hv = NV > 1 && colok && tl < head, tv = NV > 1 && colok && tl < tail;
  const int tpos = head + nb * NV + tl;
  const T ninf = T(-INFINITY);

  int lab = colok ? labels[col] : 0;
  if (lab < 0 || lab > m) lab = 0;  // callers check labels on the host; an out-of-range one is skipped, never dereferenced
  const T alab = (tl == 0 && lab > 0) ? ac[lab - 1] : T(0);
  V rv[RI];
  // the LDS slots are filled by loads that go from memory to LDS directly (lane t's 16 bytes land at the wave's base + 16 t), no register in between;
  // a slot beyond the lane's share stays unwritten and is never read
#pragma unroll
  for (int j = 0; j < LV; j++)
    if (RI + j < cnt)
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(ac + head + (long)(tl + (RI + j) * TEAM) * NV),
                                       (__attribute__((address_space(3))) void*)(held + j * BT + (threadIdx.x & ~(kWave - 1))), 16, 0, 2);
#pragma unroll
  for (int i = 0; i < RI; i++) {
    if (i < cnt) {
      if (VEC) rv[i] = ld_stream(reinterpret_cast<const V*>(ac + head + (long)(tl + i * TEAM) * NV));
      else rv[i][0] = __builtin_nontemporal_load(ac + (tl + i * TEAM));
    } else {
#pragma unroll
      for (int e = 0; e < NV; e++) rv[i][e] = ninf;
    }
  }
  T xh = hv ? ac[tl] : ninf, xt = tv ? ac[tpos] : ninf;  // -inf padding contributes exp(-inf) = 0

  T mt = ninf;
#pragma unroll
  for (int i = 0; i < RI; i++)
#pragma unroll
    for (int e = 0; e < NV; e++) mt = mt > rv[i][e] ? mt : rv[i][e];
  if (LV > 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the direct loads are invisible to the compiler's own bookkeeping
#pragma unroll
  for (int j = 0; j < LV; j++)
    if (RI + j < cnt) {
      const V v = mine[j * BT];
#pragma unroll
      for (int e = 0; e < NV; e++) mt = mt > v[e] ? mt : v[e];
    }
  if (NV > 1) { mt = mt > xh ? mt : xh; mt = mt > xt ? mt : xt; }
  T st = T(0);
  const T mref = mt == ninf ? T(0) : mt;  // a lane without elements holds only -inf padding: exp(-inf - 0) = 0
#pragma unroll
  for (int i = 0; i < RI; i++)
#pragma unroll
    for (int e = 0; e < NV; e++) {
      const T ex = dev_exp(rv[i][e] - mref);
      rv[i][e] = ex;
      st = st + ex;
    }
#pragma unroll
  for (int j = 0; j < LV; j++)
    if (RI + j < cnt) {
      V v = mine[j * BT];
#pragma unroll
      for (int e = 0; e < NV; e++) {
        const T ex = dev_exp(v[e] - mref);
        v[e] = ex;
        st = st + ex;
      }
      mine[j * BT] = v;
    }
  if (NV > 1) {
    xh = dev_exp(xh - mref);
    xt = dev_exp(xt - mref);
    st = st + xh + xt;
  }
  MaxSum<T> ms = {mt, st};
  ms = ms_wave_reduce(ms);
  if (NW > 1) {
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    if (lane == 0) { lds_m[wave] = ms.m; lds_s[wave] = ms.s; }
    __syncthreads();
    MaxSum<T> t = {lane < NW ? lds_m[lane] : ninf, lane < NW ? lds_s[lane] : T(0)};
    ms = ms_wave_reduce(t);
  }
  const T logS = dev_log(ms.s);
  // softmax_i = e_i * exp(m_t - M) / S; fold the upstream scale in: one multiply per element
  const T f = (mt == ninf ? T(0) : dev_exp(mt - ms.m) / ms.s) * scale;
  if (colok && tl == 0) loss[col] = lab > 0 ? -((alab - ms.m) - logS) : T(0);
  KNET8_TL_MID
#pragma unroll
  for (int i = 0; i < ITEMS; i++) {
    if (i >= cnt) continue;
    const int r = head + (tl + i * TEAM) * NV;
    V ve;
    if (i < RI) ve = rv[i < RI ? i : 0];
    else ve = mine[(i - RI) * BT];
    V vo;
#pragma unroll
    for (int e = 0; e < NV; e++) {
      const T p = ve[e] * f;
      const T dlp = (r + e + 1 == lab) ? -scale : T(0);
      vo[e] = lab == 0 ? T(0) : dlp + p;
    }
    if (VEC) st_stream(reinterpret_cast<V*>(oc + r), vo);
    else __builtin_nontemporal_store(vo[0], oc + r);
  }
  if (NV > 1) {
    if (hv) oc[tl] = lab == 0 ? T(0) : ((tl + 1 == lab) ? -scale : T(0)) + xh * f;
    if (tv) oc[tpos] = lab == 0 ? T(0) : ((tpos + 1 == lab) ? -scale : T(0)) + xt * f;
  }
  KNET8_TL_END
}

template <typename T, int TEAM, int E, bool VEC>
__global__ __launch_bounds__(TEAM == kWave ? kWaveTeamBlock : TEAM) void nll_col_kernel(int m, long n, const T* a, T* out, const int* labels,
                                                                            T scale, T* loss KNET8_TL_PARAM) {
  nll_col_body<T, TEAM, E, VEC, 0>(m, n, a, out, labels, scale, loss KNET8_TL_PASS);
}
// four waves per SIMD (two 512-lane workgroups per compute unit): at most 128 registers per lane
template <typename T, int TEAM, int E, int LV>
__global__ __launch_bounds__(TEAM) __attribute__((amdgpu_waves_per_eu(4, 4))) void nll_col_lds_kernel(int m, long n, const T* a, T* out,
                                                                                                      const int* labels, T scale, T* loss) {
  nll_col_body<T, TEAM, E, true, LV>(m, n, a, out, labels, scale, loss KNET8_TL_NONE);
}

// ---- many short columns -----------------------------------------------------------------------------------
// Columns of at most 128 rows (ten classes, the 21 of a segmentation map): a wave per column would move 40 bytes per instruction.  A workgroup
// takes a STRETCH of G whole columns instead -- G*m contiguous elements, read and written with full-width accesses whatever m is -- through LDS;
// a team of TL lanes (a power of two, about m/8) owns a column there: it reads its at most 8 elements per lane from LDS, reduces with shuffles,
// and puts the results back in place.  The same Algo table as the register-resident kernels; the fused nll variant uses the plain two-reduction
// form (max, then sum of exp), one exp per element.
constexpr int kShortRows = 128;
// The fused nll kernel goes this way up to 192 rows: beyond 128 rows one wave per column leaves half its lanes idle in a kernel with two reductions
// (2^23 elements, cold, wave per column -> stretches: fp32 130 rows 26.5 -> 19.0 us, 160 21.5 -> 17.1, 192 19.1 -> 16.5, 256 15.9 -> 15.2, 300 16.9 -> 17.7;
// fp64 130 rows 58 -> 45, 192 40 -> 36, 256 32 -> 34).  The other kernels are as fast or faster with a wave per column from 160 rows on.
constexpr int kShortRowsNll = 192;
// LDS layout: one padding word after every 32 entries, so that the teams of a wave, whose columns start m entries apart, do not meet in one bank
// when m is a power of two.  (Four padding words, which would keep a 16-byte vector whole and aligned for the stretch's way in and out, measured
// slower: 17 us against 12.4 us at m = 32: the column pass is the one that counts.)
__device__ __forceinline__ int short_pad(int i) { return i + (i >> 5); }

// Vectors per lane of a stretch.  One input: four (16 KB per workgroup).  Two inputs: one (fp32) or two (fp64) -- 4 / 8 KB per operand: with 16 KB
// each a compute unit holds four workgroups instead of eight, and all of them are in the same phase (all reading, then all in their column pass, then
// all writing), so the column pass is not hidden behind other workgroups' memory traffic.  Measured over m = 8 ... 100, 2^23 elements per operand, cold:
// logsoftmaxback fp32 19.8-24.0 us with 16 KB, 18.1-19.5 with 8 KB, 17.8-19.3 with 4 KB; fp64 36.6-39.2 / 33.6-35.8 / 33.2-38.7.  The one-input kernels lose
// with shorter stretches (fp32 logsoftmax m = 32: 12.4 / 14.3 / 15.9 us).
template <typename T, typename Algo> constexpr int short_stretch_vectors() { return Algo::kInputs == 2 ? (sizeof(T) == 4 ? 1 : 2) : 4; }

// R: elements of a column per lane (TL*R >= m).  Slots past the column's end are computed and thrown away, so the host picks, among R = 2 ... 8
// (and 10, 12, 16 for the one-input fp32 kernels), the pair that wastes fewest: ten classes run as one lane x 10, 21 as 2 lanes x 12.
template <typename T, typename Algo, bool VEC, int R>
__global__ __launch_bounds__(256) void softmax_short_kernel(int m, long n, int G, int TL, const T* a, const T* b, T* out, const int* labels, T scale,
                                                            T* loss) {
  constexpr bool kTwo = Algo::kInputs == 2;
  constexpr int NV = VEC ? Vec16<T>::N : 1;
  constexpr int Q = short_stretch_vectors<T, Algo>();
  constexpr int CAP = 256 * Q * Vec16<T>::N;     // elements of a stretch
  typedef typename Vec16<T>::type V;
  __shared__ T la[CAP + CAP / 32];
  __shared__ T lb[kTwo ? CAP + CAP / 32 : 1];
  const long col0 = (long)blockIdx.x * G;
  const int g = (int)(n - col0 < G ? n - col0 : G);
  const int E = g * m;
  const T* ab = a + col0 * m;
  const T* bb = kTwo ? b + col0 * m : nullptr;
  T* ob = out + col0 * m;
  constexpr int PER = VEC ? Q : Q * Vec16<T>::N;   // accesses per lane: the scalar path makes up for its narrow ones
#pragma unroll
  for (int q = 0; q < PER; q++) {
    const int i = ((int)threadIdx.x + q * 256) * NV;
    if (VEC && i + NV <= E) {
      const V va = ld_stream(reinterpret_cast<const V*>(ab + i));
#pragma unroll
      for (int e = 0; e < NV; e++) la[short_pad(i + e)] = va[e];
      if (kTwo) {
        const V vb = ld_stream(reinterpret_cast<const V*>(bb + i));
#pragma unroll
        for (int e = 0; e < NV; e++) lb[short_pad(i + e)] = vb[e];
      }
    } else {
#pragma unroll
      for (int e = 0; e < NV; e++)
        if (i + e < E) {
          la[short_pad(i + e)] = __builtin_nontemporal_load(ab + i + e);
          if (kTwo) lb[short_pad(i + e)] = __builtin_nontemporal_load(bb + i + e);
        }
    }
  }
  __syncthreads();
  const int nteams = 256 / TL, team = (int)threadIdx.x / TL, tl = (int)threadIdx.x % TL;
  for (int cb = 0; cb < g; cb += nteams) {   // the same trip count for every lane of a wave: the shuffles need all of them
    const int c = cb + team;
    const bool live = c < g;
    // (every slot is processed under a lane predicate: guarding the slots past the column's end with a branch of their own kept the LDS reads
    //  from being issued back to back and measured 40 % slower at m = 32)
    T av[R], bv[kTwo ? R : 1], tv[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
      const int k = tl + r * TL;
      const int i = short_pad(c * m + k);
      const bool ok = live && k < m;
      av[r] = ok ? la[i] : T(0);
      if (kTwo) bv[r] = ok ? lb[i] : T(0);
    }
    T mx = T(0);
    if (Algo::kNeedMax) {
      mx = -INFINITY;
#pragma unroll
      for (int r = 0; r < R; r++)
        if (live && tl + r * TL < m) mx = mx > av[r] ? mx : av[r];
      for (int o = TL >> 1; o > 0; o >>= 1) { const T t = __shfl_xor(mx, o); mx = mx > t ? mx : t; }
    }
    T s = T(0);
#pragma unroll
    for (int r = 0; r < R; r++) {
      const bool ok = live && tl + r * TL < m;
      tv[r] = ok ? Algo::term(av[r], kTwo ? bv[r] : T(0), mx) : T(0);
      s = s + tv[r];
    }
    for (int o = TL >> 1; o > 0; o >>= 1) s = s + __shfl_xor(s, o);
    const T fin = Algo::finish(s);
    if constexpr (Algo::kNll) {
      int lab = live ? labels[col0 + c] : 0;
      if (lab < 0 || lab > m) lab = 0;   // callers check labels on the host; an out-of-range one is skipped, never dereferenced
      const T f = scale / s;
      if (live && tl == 0) loss[col0 + c] = lab > 0 ? -((la[short_pad(c * m + lab - 1)] - mx) - fin) : T(0);
      // every lane of the team has read its elements and the labelled one before anything is overwritten: a team lies within one wave
#pragma unroll
      for (int r = 0; r < R; r++) {
        const int k = tl + r * TL;
        if (live && k < m) la[short_pad(c * m + k)] = lab == 0 ? T(0) : ((k + 1 == lab) ? -scale : T(0)) + tv[r] * f;
      }
    } else {
#pragma unroll
      for (int r = 0; r < R; r++) {
        const int k = tl + r * TL;
        if (live && k < m) {
          if constexpr (Algo::kKeepTerm) la[short_pad(c * m + k)] = Algo::out_kept(tv[r], fin);
          else la[short_pad(c * m + k)] = Algo::out(av[r], kTwo ? bv[r] : T(0), mx, fin);
        }
      }
    }
  }
  __syncthreads();
#pragma unroll
  for (int q = 0; q < PER; q++) {
    const int i = ((int)threadIdx.x + q * 256) * NV;
    if (VEC && i + NV <= E) {
      V vo;
#pragma unroll
      for (int e = 0; e < NV; e++) vo[e] = la[short_pad(i + e)];
      st_stream(reinterpret_cast<V*>(ob + i), vo);
    } else {
#pragma unroll
      for (int e = 0; e < NV; e++)
        if (i + e < E) __builtin_nontemporal_store(la[short_pad(i + e)], ob + i + e);
    }
  }
}

// ---- streaming fallback for columns too long to hold in registers ----------------------------------------
// One 1024-thread workgroup per column, two passes with 16-byte accesses and U of them in flight per lane.
// Pass 1 reduces: for the max-based algorithms max and sum(exp(x - max)) are carried together as a pair that is
// rescaled whenever the running max grows (one exp per element plus one per batch of U accesses), so x is read once
// for both; the other algorithms just sum their terms.  Pass 2 reads the inputs again (cache hits for the part of the
// column still resident in L2 / the memory-side cache) and writes the result.  HBM roofline: between the resident
// kernels' bytes and one extra read of every input.
template <typename T>
__device__ __forceinline__ void maxsum_merge(T& m, T& s, T m2, T s2) {
  const T mm = m > m2 ? m : m2;
  const T s1 = (m == mm) ? s : s * dev_exp(m - mm);    // equal maxima (both -inf included): no rescale, no inf - inf
  const T s3 = (m2 == mm) ? s2 : s2 * dev_exp(m2 - mm);
  m = mm;
  s = s1 + s3;
}

template <typename T, typename Algo, bool VEC>
__global__ __launch_bounds__(1024) void softmax_col_stream_kernel(long m, long n, const T* a, const T* b, T* out, const int* labels,
                                                                  T scale, T* loss) {
  constexpr int NV = VEC ? Vec16<T>::N : 1;
  constexpr int U = 4;
  constexpr bool kTwo = Algo::kInputs == 2;
  constexpr long STEP = 1024L * NV;
  typedef typename Vec16<T>::type V;
  __shared__ T lds[2][1024 / kWave];
  const long col = blockIdx.x;
  const T* ac = a + col * m;
  const T* bc = kTwo ? b + col * m : nullptr;
  T* oc = out + col * m;
  const T ninf = T(-INFINITY);
  T mx = Algo::kNeedMax ? ninf : T(0), s = T(0);
  for (long r0 = (long)threadIdx.x * NV; r0 < m; r0 += STEP * U) {
    T va[U][NV], vb[U][NV];
#pragma unroll
    for (int q = 0; q < U; q++) {
      const long r = r0 + q * STEP;
      if (r < m) {
        if (VEC) {
          const V t = *reinterpret_cast<const V*>(ac + r);
#pragma unroll
          for (int e = 0; e < NV; e++) va[q][e] = t[e];
          if (kTwo) {
            const V t2 = *reinterpret_cast<const V*>(bc + r);
#pragma unroll
            for (int e = 0; e < NV; e++) vb[q][e] = t2[e];
          }
        } else {
          va[q][0] = ac[r];
          if (kTwo) vb[q][0] = bc[r];
        }
      } else {
#pragma unroll
        for (int e = 0; e < NV; e++) { va[q][e] = Algo::kNeedMax ? ninf : T(0); vb[q][e] = T(0); }
      }
    }
    if (Algo::kNeedMax) {
      T bm = mx;
#pragma unroll
      for (int q = 0; q < U; q++)
#pragma unroll
        for (int e = 0; e < NV; e++) bm = va[q][e] > bm ? va[q][e] : bm;
      if (bm > mx) { s = s * dev_exp(mx - bm); mx = bm; }
#pragma unroll
      for (int q = 0; q < U; q++)
#pragma unroll
        for (int e = 0; e < NV; e++) s = s + (va[q][e] == ninf ? T(0) : dev_exp(va[q][e] - mx));
    } else {
#pragma unroll
      for (int q = 0; q < U; q++)
#pragma unroll
        for (int e = 0; e < NV; e++) s = s + Algo::term(va[q][e], kTwo ? vb[q][e] : T(0), T(0));
    }
  }
  if (Algo::kNeedMax) {
    {
      MaxSum<T> ms = {mx, s};
      ms = ms_wave_reduce(ms);
      mx = ms.m;
      s = ms.s;
    }
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    if (lane == 0) { lds[0][wave] = mx; lds[1][wave] = s; }
    __syncthreads();
    mx = lds[0][0];
    s = lds[1][0];
    for (int w = 1; w < 1024 / kWave; w++) maxsum_merge(mx, s, lds[0][w], lds[1][w]);
  } else {
    s = block_reduce<T, 1024 / kWave>(s, lds[0], AddFn(), T(0));
  }
  const T fin = Algo::finish(s);
  int lab = Algo::kNll ? labels[col] : 0;
  if (lab < 0 || lab > m) lab = 0;
  const T st = -scale;
  for (long r0 = (long)threadIdx.x * NV; r0 < m; r0 += STEP * U) {
    T va[U][NV], vb[U][NV];
#pragma unroll
    for (int q = 0; q < U; q++) {
      const long r = r0 + q * STEP;
      if (r < m) {
        if (VEC) {
          const V t = ld_stream(reinterpret_cast<const V*>(ac + r));
#pragma unroll
          for (int e = 0; e < NV; e++) va[q][e] = t[e];
          if (kTwo) {
            const V t2 = ld_stream(reinterpret_cast<const V*>(bc + r));
#pragma unroll
            for (int e = 0; e < NV; e++) vb[q][e] = t2[e];
          }
        } else {
          va[q][0] = ac[r];
          if (kTwo) vb[q][0] = bc[r];
        }
      }
    }
#pragma unroll
    for (int q = 0; q < U; q++) {
      const long r = r0 + q * STEP;
      if (r < m) {
        V vo;
#pragma unroll
        for (int e = 0; e < NV; e++) {
          T v = Algo::out(va[q][e], kTwo ? vb[q][e] : T(0), mx, fin);
          if (Algo::kNll) {
            const bool hit = (r + e + 1 == lab);
            if (hit) loss[col] = -v;
            const T dlp = hit ? st : T(0);
            const T p = dev_exp(v) * st;
            v = lab == 0 ? T(0) : dlp - p;
          }
          vo[e] = v;
        }
        if (VEC) st_stream(reinterpret_cast<V*>(oc + r), vo);
        else __builtin_nontemporal_store(vo[0], oc + r);
      }
    }
  }
  if (Algo::kNll && lab == 0 && threadIdx.x == 0) loss[col] = T(0);
}

// ---- softmax along a non-leading axis: x viewed as (inner, d, outer), softmax over d -----------------------
// Lanes run along `inner` (contiguous), so every access is coalesced; each lane walks its own d elements three
// times (max, sum, output).  The reference handles these `dims` with a chain of broadcast and reduction kernels
// (src/ops20/softmax.jl:42-63 through src/ops20_gpu/softmax.jl:22); one kernel replaces the chain.
template <typename T, typename Algo>
__global__ __launch_bounds__(256) void softmax_strided_kernel(long inner, long d, long outer, const T* a, const T* b, T* out) {
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= inner * outer) return;
  const long i = idx % inner, o = idx / inner;
  const long base = o * d * inner + i;
  T mx = T(0);
  if (Algo::kNeedMax) {
    mx = -INFINITY;
    for (long k = 0; k < d; k++) { const T v = a[base + k * inner]; mx = mx > v ? mx : v; }
  }
  T s = T(0);
  for (long k = 0; k < d; k++) s = s + Algo::term(a[base + k * inner], Algo::kInputs == 2 ? b[base + k * inner] : T(0), mx);
  const T fin = Algo::finish(s);
  for (long k = 0; k < d; k++)
    out[base + k * inner] = Algo::out(a[base + k * inner], Algo::kInputs == 2 ? b[base + k * inner] : T(0), mx, fin);
}

// The same for large arrays, in two launches.  A workgroup owns a panel: TI = 64*NV neighbouring `inner` positions (a wave reads
// 64*NV*sizeof(T) contiguous bytes per row) times a chunk of d, its four waves taking every fourth row.
//   reduce: every lane folds its rows into a running (max, sum of exp) pair per position (or a plain sum for the gradients),
//           the waves are merged in LDS and the panel's pairs go to scratch: partial[outer][chunk][max|sum][inner];
//   apply:  a workgroup merges the pairs of all chunks of its positions, then walks its panel again and writes the result.
// Each input is read twice (the second time mostly from the memory-side cache), the output written once; the permutation
// route (permute, column kernel, permute back) moves every array three times as often.
constexpr int kPanelWaves = 4, kPanelU = 4, kPanelMaxChunks = 64;

template <typename T, int NV>
__device__ __forceinline__ void panel_load(const T* p, T (&v)[NV]) {
  if (NV > 1) {
    typedef typename Vec16<T>::type V;
    const V t = *reinterpret_cast<const V*>(p);   // kept cacheable: the apply pass reads the same lines again
#pragma unroll
    for (int e = 0; e < NV; e++) v[e] = t[e];
  } else {
    v[0] = *p;
  }
}

template <typename T, typename Algo, int NV>
__global__ __launch_bounds__(kPanelWaves * kWave) void softmax_panel_reduce_kernel(long inner, long d, long itiles, long nchunks, long dchunk, long ipad,
                                                                                   const T* __restrict__ a, const T* __restrict__ b, T* __restrict__ partial) {
  constexpr int TI = kWave * NV, NW = kPanelWaves, U = kPanelU;
  constexpr bool kTwo = Algo::kInputs == 2;
  __shared__ T lds_m[NW][TI], lds_s[NW][TI];
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  long blk = blockIdx.x;
  const long it = blk % itiles; blk /= itiles;
  const long c = blk % nchunks;
  const long o = blk / nchunks;
  const long a0 = it * TI + (long)lane * NV;
  const bool live = a0 < inner;             // vector path: inner % NV == 0, a vector is inside or outside as a whole
  const long base = o * d * inner + a0;
  const long k0 = c * dchunk;
  long k1 = k0 + dchunk;
  if (k1 > d) k1 = d;
  const T ninf = T(-INFINITY);
  T m[NV], sum[NV];
#pragma unroll
  for (int e = 0; e < NV; e++) { m[e] = Algo::kNeedMax ? ninf : T(0); sum[e] = T(0); }
  if (live) {
    for (long k = k0 + wave; k < k1; k += NW * U) {
      T va[U][NV], vb[U][NV];
#pragma unroll
      for (int q = 0; q < U; q++) {
        const long kk = k + q * NW;
        if (kk < k1) {
          panel_load<T, NV>(a + base + kk * inner, va[q]);
          if (kTwo) panel_load<T, NV>(b + base + kk * inner, vb[q]);
        } else {
#pragma unroll
          for (int e = 0; e < NV; e++) { va[q][e] = Algo::kNeedMax ? ninf : T(0); vb[q][e] = T(0); }
        }
      }
#pragma unroll
      for (int e = 0; e < NV; e++) {
        if (Algo::kNeedMax) {
          T bm = m[e];
#pragma unroll
          for (int q = 0; q < U; q++) bm = va[q][e] > bm ? va[q][e] : bm;
          if (bm > m[e]) { sum[e] = sum[e] * dev_exp(m[e] - bm); m[e] = bm; }
#pragma unroll
          for (int q = 0; q < U; q++) sum[e] = sum[e] + (va[q][e] == ninf ? T(0) : dev_exp(va[q][e] - m[e]));
        } else {
#pragma unroll
          for (int q = 0; q < U; q++) sum[e] = sum[e] + Algo::term(va[q][e], kTwo ? vb[q][e] : T(0), T(0));
        }
      }
    }
  }
#pragma unroll
  for (int e = 0; e < NV; e++) { lds_m[wave][lane * NV + e] = m[e]; lds_s[wave][lane * NV + e] = sum[e]; }
  __syncthreads();
  if (threadIdx.x < TI) {
    T mm = lds_m[0][threadIdx.x], ss = lds_s[0][threadIdx.x];
#pragma unroll
    for (int w = 1; w < NW; w++) {
      if (Algo::kNeedMax) maxsum_merge(mm, ss, lds_m[w][threadIdx.x], lds_s[w][threadIdx.x]);
      else ss = ss + lds_s[w][threadIdx.x];
    }
    T* row = partial + ((o * nchunks + c) * 2) * ipad + it * TI + threadIdx.x;
    row[0] = mm;
    row[ipad] = ss;
  }
}

template <typename T, typename Algo, int NV>
__global__ __launch_bounds__(kPanelWaves * kWave) void softmax_panel_apply_kernel(long inner, long d, long itiles, long nchunks, long dchunk, long ipad,
                                                                                  const T* __restrict__ a, const T* __restrict__ b, const T* __restrict__ partial,
                                                                                  T* __restrict__ out) {
  constexpr int TI = kWave * NV, NW = kPanelWaves, U = kPanelU;
  constexpr bool kTwo = Algo::kInputs == 2;
  typedef typename Vec16<T>::type V;
  __shared__ T lds_m[TI], lds_f[TI];
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  long blk = blockIdx.x;
  const long it = blk % itiles; blk /= itiles;
  const long c = blk % nchunks;
  const long o = blk / nchunks;
  if (threadIdx.x < TI) {
    const T* row = partial + (o * nchunks * 2) * ipad + it * TI + threadIdx.x;
    T mm = row[0], ss = row[ipad];
    for (long cc = 1; cc < nchunks; cc++) {
      const T m2 = row[cc * 2 * ipad], s2 = row[(cc * 2 + 1) * ipad];
      if (Algo::kNeedMax) maxsum_merge(mm, ss, m2, s2);
      else ss = ss + s2;
    }
    lds_m[threadIdx.x] = mm;
    lds_f[threadIdx.x] = Algo::finish(ss);
  }
  __syncthreads();
  const long a0 = it * TI + (long)lane * NV;
  if (a0 >= inner) return;
  T mx[NV], fin[NV];
#pragma unroll
  for (int e = 0; e < NV; e++) { mx[e] = lds_m[lane * NV + e]; fin[e] = lds_f[lane * NV + e]; }
  const long base = o * d * inner + a0;
  const long k0 = c * dchunk;
  long k1 = k0 + dchunk;
  if (k1 > d) k1 = d;
  for (long k = k0 + wave; k < k1; k += NW * U) {
    T va[U][NV], vb[U][NV];
#pragma unroll
    for (int q = 0; q < U; q++) {
      const long kk = k + q * NW;
      if (kk < k1) {
        panel_load<T, NV>(a + base + kk * inner, va[q]);
        if (kTwo) panel_load<T, NV>(b + base + kk * inner, vb[q]);
      }
    }
#pragma unroll
    for (int q = 0; q < U; q++) {
      const long kk = k + q * NW;
      if (kk < k1) {
        if (NV > 1) {
          V vo;
#pragma unroll
          for (int e = 0; e < NV; e++) vo[e] = Algo::out(va[q][e], kTwo ? vb[q][e] : T(0), mx[e], fin[e]);
          st_stream(reinterpret_cast<V*>(out + base + kk * inner), vo);
        } else {
          __builtin_nontemporal_store(Algo::out(va[q][0], kTwo ? vb[q][0] : T(0), mx[0], fin[0]), out + base + kk * inner);
        }
      }
    }
  }
}

constexpr long kStridedSmall = 1 << 14;   // elements; below this one lane-per-slice launch beats two panel launches

template <typename T, typename Algo>
inline void launch_softmax_strided(hipStream_t stream, long inner, long d, long outer, const T* a, const T* b, T* out) {
  if (inner <= 0 || d <= 0 || outer <= 0) return;
  const long total = inner * outer;
  if (total * d <= kStridedSmall) {
    hipLaunchKernelGGL((softmax_strided_kernel<T, Algo>), dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, inner, d, outer, a, b, out);
    return;
  }
  constexpr int N = Vec16<T>::N;
  const bool vec = inner % N == 0 && aligned16(a) && aligned16(out) && (Algo::kInputs < 2 || aligned16(b));
  const long ti = (long)kWave * (vec ? N : 1);
  const long itiles = (inner + ti - 1) / ti, ipad = itiles * ti;
  long nchunks = (4L * tuning(kTuneNumCUs) + itiles * outer - 1) / (itiles * outer);   // about four workgroups per CU
  const long maxchunks = d / (kPanelWaves * kPanelU) > 0 ? d / (kPanelWaves * kPanelU) : 1;
  if (nchunks > maxchunks) nchunks = maxchunks;
  if (nchunks > kPanelMaxChunks) nchunks = kPanelMaxChunks;   // every workgroup of the apply pass merges all chunks of its positions
  if (nchunks < 1) nchunks = 1;
  const long dchunk = (d + nchunks - 1) / nchunks;
  nchunks = (d + dchunk - 1) / dchunk;
  const long blocks = itiles * nchunks * outer;
  if (blocks > 0x7fffffffL) { record_error("softmax over a strided dimension: too many panels"); return; }
  Workspace ws = workspace_for(stream, sizeof(T) * (size_t)(outer * nchunks * 2 * ipad), 0);
  if (ws.partial == nullptr) { record_error("softmax over a strided dimension: no scratch memory"); return; }
  T* partial = static_cast<T*>(ws.partial);
#define KNET8_PANEL(NV) do { \
    hipLaunchKernelGGL((softmax_panel_reduce_kernel<T, Algo, NV>), dim3((unsigned)blocks), dim3(kPanelWaves * kWave), 0, stream, inner, d, itiles, nchunks, dchunk, ipad, a, b, partial); \
    hipLaunchKernelGGL((softmax_panel_apply_kernel<T, Algo, NV>), dim3((unsigned)blocks), dim3(kPanelWaves * kWave), 0, stream, inner, d, itiles, nchunks, dchunk, ipad, a, b, partial, out); \
  } while (0)
  if (vec) KNET8_PANEL(N); else KNET8_PANEL(1);
#undef KNET8_PANEL
}

template <typename T, typename Algo, int TEAM, int E>
inline void launch_softmax_cfg(hipStream_t stream, bool vec, int m, long n, const T* a, const T* b, T* out, const int* labels,
                               T scale, T* loss) {
  constexpr int BT = TEAM == kWave ? kWaveTeamBlock : TEAM;
  constexpr int TEAMS = BT / TEAM;
  const dim3 block(BT);
  // (Handling two columns per team with the loads of both issued up front was measured on (32000,512): nothing for the fused nll
  // kernel, 23.0 us either way, and 8 % slower forward kernels -- both phases are limited by HBM itself, not by the bubbles
  // between them.)
  const dim3 grid((unsigned)((n + TEAMS - 1) / TEAMS));
  if constexpr (Algo::kNll) {
    if (vec) hipLaunchKernelGGL((nll_col_kernel<T, TEAM, E, true>), grid, block, 0, stream, m, n, a, out, labels, scale, loss KNET8_TL_ARG);
    else hipLaunchKernelGGL((nll_col_kernel<T, TEAM, E, false>), grid, block, 0, stream, m, n, a, out, labels, scale, loss KNET8_TL_ARG);
  } else {
    if (vec) hipLaunchKernelGGL((softmax_col_kernel<T, Algo, TEAM, E, true>), grid, block, 0, stream, m, n, a, b, out KNET8_TL_ARG);
    else hipLaunchKernelGGL((softmax_col_kernel<T, Algo, TEAM, E, false>), grid, block, 0, stream, m, n, a, b, out KNET8_TL_ARG);
  }
}

template <typename T, typename Algo>
inline void launch_softmax(hipStream_t stream, long m, long n, const T* a, const T* b, T* out, const int* labels, T scale, T* loss) {
  if (m <= 0 || n <= 0) return;
  constexpr int N = Vec16<T>::N;
  // Per-lane capacity: the 1024-lane workgroup is limited to 128 registers per lane, i.e. 64 fp32 / 32 fp64 held elements (half with two held
  // inputs) -- more than that spills.  Longer columns stream.
  constexpr int kHeld = (Algo::kInputs == 2 && Algo::kHoldA) ? 2 : 1;
  constexpr int kBig1024 = 256 / (int)(sizeof(T) * kHeld);
  // The fused nll kernel in fp32 holds up to 128 elements per lane in a 256-lane team (four waves, one per SIMD, two teams per compute
  // unit): on 32000-row columns 21.8-22.1 us against 22.0-22.3 us for the 1024-lane team (a barrier among four waves instead of sixteen).
  constexpr bool kWideNll = Algo::kNll && sizeof(T) == 4;
  // resident kernels: vectors whenever the operands are congruent modulo 16 bytes (each column is cut at its own aligned address);
  // streaming kernel: whole columns of vectors only
  const uintptr_t ma = reinterpret_cast<uintptr_t>(a) % 16, mo = reinterpret_cast<uintptr_t>(out) % 16;
  const uintptr_t mb = Algo::kInputs == 2 ? reinterpret_cast<uintptr_t>(b) % 16 : ma;
  const bool vec = ma == mo && ma == mb && ma % sizeof(T) == 0;
  const bool vec_stream = (m % N == 0) && ma == 0 && mo == 0 && mb == 0;
  const long resident_cap = tuning(kTuneSoftmaxResidentRows);  // 0: no limit below the register capacity (tests lower it to reach the streaming kernel with short columns)
#define KNET8_SM(TEAM, E) launch_softmax_cfg<T, Algo, TEAM, E>(stream, vec, (int)m, n, a, b, out, labels, scale, loss)
  if (m <= (Algo::kNll ? kShortRowsNll : kShortRows) && n >= 64 && !(resident_cap > 0 && m > resident_cap)) {
    // stretches of whole columns (see softmax_short_kernel): G columns per workgroup, starting on 16-byte boundaries on the vector path
    constexpr int cap = 256 * short_stretch_vectors<T, Algo>() * N;
    const bool v16 = ma == 0 && mo == 0 && mb == 0;
    long G = cap / m;
    if (v16) {
      long step = N;
      for (long t = 1; t <= N; t++)
        if ((t * m) % N == 0) { step = t; break; }
      G = G / step * step;
    }
    // (a matrix too small for sixteen workgroups stays with one wave per column: one launch is 2.8 us there against 3.5 us through LDS)
    if (G >= 1 && n * m >= 16L * 256 * 4 * N) {
      // lanes per column and elements per lane: cheapest passes over the workgroup's G columns, a pass costing its R slots plus about six slots' worth
      // of reductions and bookkeeping (measured: ten classes are faster as 2 lanes x 8 in four passes than as 4 x 3 in seven, and faster still as
      // one lane x 10 in one).  The stretch is cut to a whole number of passes when that costs less per column than a last pass with idle teams.
      // More than eight slots per lane pay only in the one-input fp32 kernels (fp32 logsoftmax, 2^23 elements, cold: m = 10 16.9 -> 14.6 us, 21 17.8 ->
      // 15.0, 40 18.4 -> 14.8, 100 17.9 -> 15.7; fp64, whose slots take two registers each, and the two-input kernels with their short stretches gain
      // nothing or lose); sixteen slots lose where eight cover the column exactly (m = 16, 32, 64, 128: 11.9-12.9 us with eight, 14.4-15.3 with sixteen).
      constexpr bool kManySlots = sizeof(T) == 4 && Algo::kInputs == 1;
      int bestR = 8, bestTL = kWave;
      long bestG = G;
      double best = -1;
      for (int R : {16, 12, 10, 8, 7, 6, 5, 4, 3, 2}) {
        if (R > 8 && (!kManySlots || (R == 16 && (m & (m - 1)) == 0))) continue;
        int TL = 1;
        while (TL < kWave && (long)TL * R < m) TL <<= 1;
        if ((long)TL * R < m) continue;
        const long nteams = 256 / TL;
        for (long Gc : {G, G / nteams * nteams}) {     // nteams is a power of two of at least 4: Gc stays a multiple of `step`
          if (Gc < 1) continue;
          const double cost = (double)(((Gc + nteams - 1) / nteams) * (R + 6)) / (double)Gc;
          if (best < 0 || cost < best) { best = cost; bestR = R; bestTL = TL; bestG = Gc; }
        }
      }
      G = bestG;
      const dim3 grid((unsigned)((n + G - 1) / G));
#define KNET8_SHORT(VEC, R) hipLaunchKernelGGL((softmax_short_kernel<T, Algo, VEC, R>), grid, dim3(256), 0, stream, (int)m, n, (int)G, bestTL, a, b, out, labels, scale, loss)
      if (v16) {
        bool launched = false;
        if constexpr (kManySlots) {
          launched = true;
          switch (bestR) { case 10: KNET8_SHORT(true, 10); break; case 12: KNET8_SHORT(true, 12); break; case 16: KNET8_SHORT(true, 16); break;
                           default: launched = false; }
        }
        if (!launched)
          switch (bestR) { case 2: KNET8_SHORT(true, 2); break; case 3: KNET8_SHORT(true, 3); break; case 4: KNET8_SHORT(true, 4); break;
                           case 5: KNET8_SHORT(true, 5); break; case 6: KNET8_SHORT(true, 6); break; case 7: KNET8_SHORT(true, 7); break;
                           default: KNET8_SHORT(true, 8); }
      } else {
        int TL = 1;   // operands that are not all on 16-byte boundaries: the one general variant
        while (TL < kWave && TL * 8 < m) TL <<= 1;
        bestTL = TL;
        KNET8_SHORT(false, 8);
      }
#undef KNET8_SHORT
      return;
    }
  }
  if ((resident_cap > 0 && m > resident_cap) || m > 1024L * kBig1024) {
    if (vec_stream) hipLaunchKernelGGL((softmax_col_stream_kernel<T, Algo, true>), dim3((unsigned)n), dim3(1024), 0, stream, m, n, a, b, out, labels, scale, loss);
    else hipLaunchKernelGGL((softmax_col_stream_kernel<T, Algo, false>), dim3((unsigned)n), dim3(1024), 0, stream, m, n, a, b, out, labels, scale, loss);
    return;
  }
  // Columns of 128 to 256 KB: two 512-lane workgroups per compute unit with part of the column in LDS (see softmax_col_body).
  // Measured on (32000,512) fp64, cold: logsoftmax 59.7 -> 44.5 us, softmax 59.8 -> 47.5, fused nll 52.2 -> 42.5; logsoftmaxback, whose output pass
  // reads a second operand, gains nothing (70.8 -> 71.6; 70.8 -> 73.4 with that pass fetching two vectors ahead, all that 128 registers leave room for) and keeps
  // its registers-only kernel.
  // The same 512-lane kernels serve fp32 columns of 32 769 to 65 536 rows (vocabularies of 50257 entries): forward kernels 44.5 -> 41.6 and 46.4 -> 40.7 us
  // on (50257,512); the fused fp32 nll kernel is as fast from registers alone (42.4 against 45.8) and keeps them.
  if constexpr (Algo::kInputs == 1 && (!Algo::kNll || sizeof(T) == 8)) {
    constexpr int kLdsE = 32 * N;   // 32 vectors per lane, 512 lanes: columns of up to 256 KB (32768 fp64 or 65536 fp32 rows)
    if (vec && m > 1024 * (kBig1024 / 2) && m <= 512 * kLdsE && tuning(kTuneSoftmaxNoLdsSlots) == 0) {
      if constexpr (Algo::kNll) hipLaunchKernelGGL((nll_col_lds_kernel<T, 512, kLdsE, 9>), dim3((unsigned)n), dim3(512), 0, stream, (int)m, n, a, out, labels, scale, loss);
      else hipLaunchKernelGGL((softmax_col_lds_kernel<T, Algo, 512, kLdsE, 9>), dim3((unsigned)n), dim3(512), 0, stream, (int)m, n, a, b, out);
      return;
    }
  }
  // Team and elements per lane by column length, from a sweep over m = 2000 ... 24000 in both widths (cold, 67-100 MB per launch; fractions of
  // 8 TB/s): many lanes with few elements each beat few lanes with many -- one wave holding a 4000-row column (64 elements per lane) gave
  // 0.63-0.64 where a 256-lane team gives 0.69-0.70; logsoftmaxback, which streams its second operand in the output pass, does best with 1024
  // lanes from 2 K rows on (12000 rows fp32: 0.61 with 256 lanes x 64, 0.74 with 1024 x 16).  fp64 single-input kernels keep 256-lane teams up to
  // 16 K rows (their exp needs the registers a 1024-lane workgroup cannot give: 0.68 against 0.61 at 6000 rows).
  constexpr bool kStreamsA = Algo::kInputs == 2 && !Algo::kHoldA;
  constexpr bool kWideSingle = sizeof(T) == 8 && Algo::kInputs == 1;
  if (m <= 64 * 4) KNET8_SM(64, 4);
  // (fp64 logsoftmaxback on columns of 769 to 1024 rows: 256 lanes with two vectors each, the second operand streamed, beat one wave holding both
  //  operands -- 1000 rows x 4096 columns, cold: 19.0 -> 18.1 us; every other kernel and width is 3 to 50 % slower that way, and so is this one below 768 rows)
  else if (m <= 64 * 16) { if (kStreamsA && sizeof(T) == 8 && m > 768) KNET8_SM(256, 4); else KNET8_SM(64, 16); }
  else if (m <= 256 * 16) { if (kStreamsA && m > 2048) KNET8_SM(1024, 8); else KNET8_SM(256, 16); }
  // (the 256-lane fp64 teams only with more than 512 columns: with fewer, a column per 1024 lanes keeps more of the chip busy -- (16384, 64) logsoftmax 12.6 -> 11.2 us,
  //  softmax 14.3 -> 12.0, fused nll 12.3 -> 10.5; (12000, 256) 14.8 -> 13.8 / 14.4 -> 13.5 / 14.4 -> 12.7; at 512 columns the two are level, at 1024 columns of 8192 rows
  //  the small teams lead 24.1 to 29.7)
  else if (m <= 1024 * 8) { if (kWideSingle && n > 512) { if constexpr (kWideSingle) KNET8_SM(256, 32); } else KNET8_SM(1024, 8); }
  else if (m <= 1024 * 16) { if (kWideSingle && n > 512) { if constexpr (kWideSingle) KNET8_SM(256, 64); } else KNET8_SM(1024, 16); }
  // (the 256-lane fused nll kernel only where it was found: more than 24 K rows and 257 to 512 columns, i.e. a launch between one and two workgroups per compute
  //  unit.  Everywhere else around it the 1024-lane team is faster: (32000, 32) 9.4 -> 7.2 us, (32000, 128) 10.1 -> 8.0, (32000, 256) 13.9 -> 12.5, (32000, 640) 31.7 -> 29.0,
  //  (32000, 1024) 48.5 -> 46.5, (17000, 576) 20.8 -> 17.3; against it (32000, 384) 17.9 / 20.2, (28000, 448) 17.7 / 19.0, (32000, 512) 22.3-23.5 / 22.4-22.8)
  else if (kWideNll && m <= 256 * 128 && m > 24 * 1024 && n > 256 && n <= 512) { if constexpr (kWideNll) KNET8_SM(256, 128); }
  else if (m <= 1024 * (kBig1024 / 2)) KNET8_SM(1024, kBig1024 / 2);
  else KNET8_SM(1024, kBig1024);
#undef KNET8_SM
}

}  // namespace knet8
