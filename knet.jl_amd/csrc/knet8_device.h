// Device-side building blocks shared by every libknet8 kernel family (gfx950 / CDNA4 only).
//
// Conventions
//   * wavefront = 64 lanes; workgroups are multiples of 64 threads.
//   * streaming operands are moved as 16-byte vectors (global_load_dwordx4 /
//     global_store_dwordx4) with the non-temporal hint: every array on the gradient path is
//     touched exactly once per launch, so nothing is worth keeping in L2.
//   * all arithmetic is compiled with -ffp-contract=off: one rounding per operation, the same
//     sequence of operations as the CPU Array path of the reference.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace knet8 {

constexpr int kWave = 64;

template <typename T> struct Vec16;
template <> struct Vec16<float> {
  typedef float type __attribute__((ext_vector_type(4)));
  static constexpr int N = 4;
};
template <> struct Vec16<double> {
  typedef double type __attribute__((ext_vector_type(2)));
  static constexpr int N = 2;
};
template <> struct Vec16<int> {
  typedef int type __attribute__((ext_vector_type(4)));
  static constexpr int N = 4;
};

// Streaming (read-once / write-once) accesses.
template <typename V> __device__ __forceinline__ V ld_stream(const V* p) { return __builtin_nontemporal_load(p); }
template <typename V> __device__ __forceinline__ void st_stream(V* p, V v) { __builtin_nontemporal_store(v, p); }

// A 16-byte store written through to the device-coherent level (sc1) instead of staying dirty in this XCD's L2.  The compiler has no form of
// it for vectors; the inline instruction is an ordinary vector store (the "memory" clobber keeps later loads of the same address behind it).
template <typename V> __device__ __forceinline__ void st_through(V* p, V v) {
  static_assert(sizeof(V) == 16, "st_through: 16-byte vectors");
  asm volatile("global_store_dwordx4 %0, %1, off sc1" ::"v"(p), "v"(v) : "memory");
}

template <typename T> __host__ __device__ __forceinline__ bool aligned16(const T* p) {
  return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
}

// ---- wave64 reductions -------------------------------------------------------------------------
// Cross-lane moves by DPP (data-parallel primitives: a modifier of an ordinary ALU move, full rate, no LDS traffic).  __shfl_xor
// goes through ds_bpermute, a dependent LDS round trip per step: measured on a latency-bound kernel, sixteen such steps cost 0.5 us.
//   row_ror:n   (0x120 + n) rotate within each row of 16 lanes
//   row_bcast15 (0x142)     lane 15 of each row to every lane of the next row (rows chosen by the row mask)
//   row_bcast31 (0x143)     lane 31 to every lane of rows 2 and 3
template <int CTRL, int ROW_MASK, typename T> __device__ __forceinline__ T dpp_move(T v) {
  static_assert(sizeof(T) == 4 || sizeof(T) == 8, "dpp_move: 4- or 8-byte values");
  if constexpr (sizeof(T) == 4) {
    const int b = __builtin_bit_cast(int, v);
    return __builtin_bit_cast(T, __builtin_amdgcn_update_dpp(b, b, CTRL, ROW_MASK, 0xf, false));
  } else {
    const long long b = __builtin_bit_cast(long long, v);
    const int lo = (int)b, hi = (int)(b >> 32);
    const int nlo = __builtin_amdgcn_update_dpp(lo, lo, CTRL, ROW_MASK, 0xf, false);
    const int nhi = __builtin_amdgcn_update_dpp(hi, hi, CTRL, ROW_MASK, 0xf, false);
    return __builtin_bit_cast(T, ((long long)nhi << 32) | (unsigned int)nlo);
  }
}
template <typename T> __device__ __forceinline__ T wave_read_lane63(T v) {
  if constexpr (sizeof(T) == 4) {
    return __builtin_bit_cast(T, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
  } else {
    const long long b = __builtin_bit_cast(long long, v);
    const int lo = __builtin_amdgcn_readlane((int)b, 63), hi = __builtin_amdgcn_readlane((int)(b >> 32), 63);
    return __builtin_bit_cast(T, ((long long)hi << 32) | (unsigned int)lo);
  }
}
// All-reduce over the 16 lanes of each row by rotations (every lane of a row ends with the row's result).
template <typename T, typename Merge> __device__ __forceinline__ T row16_reduce(T v, Merge merge) {
  v = merge(v, dpp_move<0x128, 0xf>(v));
  v = merge(v, dpp_move<0x124, 0xf>(v));
  v = merge(v, dpp_move<0x122, 0xf>(v));
  v = merge(v, dpp_move<0x121, 0xf>(v));
  return v;
}
// All-reduce over the 64 lanes: rows first, then row 0 into row 1 and row 2 into row 3, then rows 0+1 into row 3, whose last lane is
// read back to everyone.  A fixed order, every lane the same bits: results are deterministic run to run.  Must be called by all 64
// lanes of the wave (no divergence around it).
template <typename T, typename Merge> __device__ __forceinline__ T wave_reduce(T v, Merge merge) {
  v = row16_reduce(v, merge);
  const int row = (threadIdx.x & (kWave - 1)) >> 4;
  T t = dpp_move<0x142, 0xa>(v);
  v = (row & 1) ? merge(v, t) : v;
  t = dpp_move<0x143, 0xc>(v);
  v = (row >= 2) ? merge(v, t) : v;
  return wave_read_lane63(v);
}

// Reduce over a workgroup of NWAVES*64 threads.  `lds` must hold NWAVES elements.  Every thread
// returns the full result.  Contains two barriers: may be called repeatedly with the same `lds`.
template <typename T, int NWAVES, typename Merge>
__device__ __forceinline__ T block_reduce(T v, T* lds, Merge merge, T identity) {
  v = wave_reduce(v, merge);
  if (NWAVES == 1) return v;
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  __syncthreads();  // previous use of lds is over
  if (lane == 0) lds[wave] = v;
  __syncthreads();
  T r = (lane < NWAVES) ? lds[lane] : identity;
  // NWAVES <= 16: a 16-lane butterfly is enough, but the full one keeps every lane identical
  r = wave_reduce(r, merge);
  return r;
}

// Device-scope "last workgroup of a group finishes the job" ticket.  Workgroups that contribute to the
// same output group store their partials with st_coherent() and call this; the one that draws the last
// ticket (returns true) may then read all partials and must reset the counter so the next launch on the
// same stream finds it zero.
//
// The L2s of the eight XCDs are not coherent with each other, so the textbook form of this pattern (plain
// stores, then an agent-scope release fence per workgroup) makes every workgroup write its whole L2 back
// (buffer_wbl2); measured, a few thousand such fences cost 100+ us, several times the reduction itself.
// Instead the partials are written through to the device-coherent level as they are stored (agent-scope
// relaxed atomic stores: global_store ... sc1), each lane waits for its own stores to be acknowledged
// (s_waitcnt vmcnt(0)), the barrier collects the lanes, and only then does lane 0 take the ticket with an
// agent-scope atomic.  Whoever sees the last ticket therefore finds every partial at the coherent level;
// it drops stale lines with one acquire fence (buffer_inv sc1) before the workgroup reads them.
template <typename T> __device__ __forceinline__ void st_coherent(T* p, T v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ bool last_block_ticket(unsigned* counter, unsigned nparts, unsigned* lds_flag) {
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  if (threadIdx.x == 0) {
    const unsigned t = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const bool last = (t == nparts - 1);
    if (last) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    *lds_flag = last ? 1u : 0u;
  }
  __syncthreads();
  return *lds_flag != 0;
}

template <typename T> __device__ __forceinline__ T ld_coherent(const T* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// ---- per-workgroup time stamps (measurement build only) ------------------------------------------------------------
// With -DKNET8_TIMELINE (a second library compiled from these same headers for measurements, never the one that ships) the kernels behind
// the roofline tables take one more argument, a stamp buffer, and record for every `every`-th workgroup (all of them up to kTlSlots) the
// 100 MHz wall clock at its start, at its phase boundary (operands arrived, own share reduced) and after its last store has been acknowledged,
// with the XCD it ran on.  Without the macro the six macros below expand to nothing: the product's kernels carry no trace of them.
#ifdef KNET8_TIMELINE
struct TlStamp { unsigned long long t0, t1, t2; unsigned xcc, wg; };
constexpr unsigned kTlSlots = 16384;
struct TlClock {
  TlStamp* buf;
  unsigned long long t0, t1;
  __device__ __forceinline__ explicit TlClock(TlStamp* b) : buf(b) { t0 = t1 = wall_clock64(); }
  __device__ __forceinline__ void mid() { t1 = wall_clock64(); }
  __device__ __forceinline__ void end() {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    const unsigned every = (gridDim.x + kTlSlots - 1) / kTlSlots;
    if (buf != nullptr && threadIdx.x == 0 && blockIdx.x % every == 0) {
      TlStamp q;
      q.t0 = t0; q.t1 = t1; q.t2 = wall_clock64();
      q.xcc = __builtin_amdgcn_s_getreg((3 << 11) | 20) & 7;   // XCC_ID, bits 3:0
      q.wg = blockIdx.x;
      buf[blockIdx.x / every] = q;
    }
  }
};
#define KNET8_TL_PARAM , knet8::TlStamp* tl_buf
#define KNET8_TL_PASS , tl_buf
#define KNET8_TL_NONE , nullptr
#define KNET8_TL_ARG , knet8::timeline_buffer()
#define KNET8_TL_BEGIN knet8::TlClock tl_clock(tl_buf);
#define KNET8_TL_MID tl_clock.mid();
#define KNET8_TL_END tl_clock.end();
#else
#define KNET8_TL_PARAM
#define KNET8_TL_PASS
#define KNET8_TL_NONE
#define KNET8_TL_ARG
#define KNET8_TL_BEGIN
#define KNET8_TL_MID
#define KNET8_TL_END
#endif

}  // namespace knet8

// ---- libm calls used by the operator tables (ocml, full precision: the library is built without fast-math)
namespace knet8 {
__device__ __forceinline__ float kexp(float x) { return expf(x); }
__device__ __forceinline__ double kexp(double x) { return exp(x); }
__device__ __forceinline__ float klog(float x) { return logf(x); }
__device__ __forceinline__ double klog(double x) { return log(x); }
__device__ __forceinline__ float ktanh(float x) { return tanhf(x); }
__device__ __forceinline__ double ktanh(double x) { return tanh(x); }
__device__ __forceinline__ float kerf(float x) { return erff(x); }
__device__ __forceinline__ double kerf(double x) { return erf(x); }
__device__ __forceinline__ float ksqrt(float x) { return sqrtf(x); }
__device__ __forceinline__ double ksqrt(double x) { return sqrt(x); }

// The rest of the unary table of src/libknet8/ops.jl:6-80: one wrapper per libm routine, so that the op bodies are written once for both types.
__device__ __forceinline__ float kacos(float x) { return acosf(x); }
__device__ __forceinline__ double kacos(double x) { return acos(x); }
__device__ __forceinline__ float kacosh(float x) { return acoshf(x); }
__device__ __forceinline__ double kacosh(double x) { return acosh(x); }
__device__ __forceinline__ float kasin(float x) { return asinf(x); }
__device__ __forceinline__ double kasin(double x) { return asin(x); }
__device__ __forceinline__ float kasinh(float x) { return asinhf(x); }
__device__ __forceinline__ double kasinh(double x) { return asinh(x); }
__device__ __forceinline__ float katan(float x) { return atanf(x); }
__device__ __forceinline__ double katan(double x) { return atan(x); }
__device__ __forceinline__ float katanh(float x) { return atanhf(x); }
__device__ __forceinline__ double katanh(double x) { return atanh(x); }
__device__ __forceinline__ float kcbrt(float x) { return cbrtf(x); }
__device__ __forceinline__ double kcbrt(double x) { return cbrt(x); }
__device__ __forceinline__ float kceil(float x) { return ceilf(x); }
__device__ __forceinline__ double kceil(double x) { return ceil(x); }
__device__ __forceinline__ float kcos(float x) { return cosf(x); }
__device__ __forceinline__ double kcos(double x) { return cos(x); }
__device__ __forceinline__ float kcosh(float x) { return coshf(x); }
__device__ __forceinline__ double kcosh(double x) { return cosh(x); }
__device__ __forceinline__ float kcospi(float x) { return cospif(x); }
__device__ __forceinline__ double kcospi(double x) { return cospi(x); }
__device__ __forceinline__ float kerfc(float x) { return erfcf(x); }
__device__ __forceinline__ double kerfc(double x) { return erfc(x); }
__device__ __forceinline__ float kerfcinv(float x) { return erfcinvf(x); }
__device__ __forceinline__ double kerfcinv(double x) { return erfcinv(x); }
__device__ __forceinline__ float kerfcx(float x) { return erfcxf(x); }
__device__ __forceinline__ double kerfcx(double x) { return erfcx(x); }
__device__ __forceinline__ float kerfinv(float x) { return erfinvf(x); }
__device__ __forceinline__ double kerfinv(double x) { return erfinv(x); }
__device__ __forceinline__ float kexp10(float x) { return exp10f(x); }
__device__ __forceinline__ double kexp10(double x) { return exp10(x); }
__device__ __forceinline__ float kexp2(float x) { return exp2f(x); }
__device__ __forceinline__ double kexp2(double x) { return exp2(x); }
__device__ __forceinline__ float kexpm1(float x) { return expm1f(x); }
__device__ __forceinline__ double kexpm1(double x) { return expm1(x); }
__device__ __forceinline__ float kfloor(float x) { return floorf(x); }
__device__ __forceinline__ double kfloor(double x) { return floor(x); }
__device__ __forceinline__ float kj0(float x) { return j0f(x); }
__device__ __forceinline__ double kj0(double x) { return j0(x); }
__device__ __forceinline__ float kj1(float x) { return j1f(x); }
__device__ __forceinline__ double kj1(double x) { return j1(x); }
__device__ __forceinline__ float klgamma(float x) { return lgammaf(x); }
__device__ __forceinline__ double klgamma(double x) { return lgamma(x); }
__device__ __forceinline__ float ktgamma(float x) { return tgammaf(x); }
__device__ __forceinline__ double ktgamma(double x) { return tgamma(x); }
__device__ __forceinline__ float klog10(float x) { return log10f(x); }
__device__ __forceinline__ double klog10(double x) { return log10(x); }
__device__ __forceinline__ float klog1p(float x) { return log1pf(x); }
__device__ __forceinline__ double klog1p(double x) { return log1p(x); }
__device__ __forceinline__ float klog2(float x) { return log2f(x); }
__device__ __forceinline__ double klog2(double x) { return log2(x); }
__device__ __forceinline__ float krint(float x) { return rintf(x); }
__device__ __forceinline__ double krint(double x) { return rint(x); }
__device__ __forceinline__ float ksin(float x) { return sinf(x); }
__device__ __forceinline__ double ksin(double x) { return sin(x); }
__device__ __forceinline__ float ksinh(float x) { return sinhf(x); }
__device__ __forceinline__ double ksinh(double x) { return sinh(x); }
__device__ __forceinline__ float ksinpi(float x) { return sinpif(x); }
__device__ __forceinline__ double ksinpi(double x) { return sinpi(x); }
__device__ __forceinline__ float ktan(float x) { return tanf(x); }
__device__ __forceinline__ double ktan(double x) { return tan(x); }
__device__ __forceinline__ float ktrunc(float x) { return truncf(x); }
__device__ __forceinline__ double ktrunc(double x) { return trunc(x); }
__device__ __forceinline__ float ky0(float x) { return y0f(x); }
__device__ __forceinline__ double ky0(double x) { return y0(x); }
__device__ __forceinline__ float ky1(float x) { return y1f(x); }
__device__ __forceinline__ double ky1(double x) { return y1(x); }
__device__ __forceinline__ float kpow(float x, float y) { return powf(x, y); }
__device__ __forceinline__ double kpow(double x, double y) { return pow(x, y); }
}  // namespace knet8
