// Device random numbers: what `rand!(a::KnetArray)` / `randn!` take from cuRAND in the reference (src/knetarrays/random.jl:5-6),
// the source of the uniform buffer that dropout! consumes (src/ops20_gpu/dropout.jl:14).
//
// Generator: Philox4x32-10 (Salmon, Moraes, Dror, Shaw: "Parallel random numbers: as easy as 1, 2, 3", SC'11), counter based:
// block c of a stream is philox(key = seed, counter = c), four 32-bit words, with no state carried between lanes or launches.
// A call that writes n elements consumes ceil(n / per_block) consecutive counters starting at `offset`:
//   fp32 uniform: 4 per block, u = (w >> 8) * 2^-24                       in [0, 1)
//   fp64 uniform: 2 per block, u = ((w0 >> 5) * 2^26 + (w1 >> 6)) * 2^-53  in [0, 1)
//   normal: Box-Muller on (u1, u2) with u1 moved to (0, 1]: fp32 two pairs per block -> 4 values, fp64 one pair -> 2 values
// so element i depends on (seed, offset, i) only: the same call reproduces the same numbers on any grid, stream or device.
// One lane produces one block and stores it as one 16-byte vector: a write-only stream, sizeof(T) bytes per element.  The ten
// rounds (20 32x32->64-bit multiplies per block) hide behind the stores: uniforms are written at the rate of fill_S; normals
// are bound by log/sqrt/sincos instead (about 40 % of that rate in fp32, 30 % in fp64).
#pragma once
#include "knet8_device.h"
#include "knet8_runtime.h"

namespace knet8 {

struct Philox4 { unsigned w[4]; };

__host__ __device__ __forceinline__ Philox4 philox4x32_10(unsigned long long counter, unsigned long long key, unsigned long long counter_hi = 0) {
  constexpr unsigned kM0 = 0xD2511F53u, kM1 = 0xCD9E8D57u;   // round multipliers
  constexpr unsigned kW0 = 0x9E3779B9u, kW1 = 0xBB67AE85u;   // key schedule increments (golden ratio, sqrt(3)-1)
  unsigned c0 = (unsigned)counter, c1 = (unsigned)(counter >> 32), c2 = (unsigned)counter_hi, c3 = (unsigned)(counter_hi >> 32);
  unsigned k0 = (unsigned)key, k1 = (unsigned)(key >> 32);
#pragma unroll
  for (int r = 0; r < 10; r++) {
    const unsigned long long p0 = (unsigned long long)kM0 * c0, p1 = (unsigned long long)kM1 * c2;
    const unsigned n0 = (unsigned)(p1 >> 32) ^ c1 ^ k0, n1 = (unsigned)p1;
    const unsigned n2 = (unsigned)(p0 >> 32) ^ c3 ^ k1, n3 = (unsigned)p0;
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    k0 += kW0; k1 += kW1;
  }
  Philox4 out = {{c0, c1, c2, c3}};
  return out;
}

template <typename T> struct RandConv;
template <> struct RandConv<float> {
  static constexpr int kPerBlock = 4;
  __device__ static void uniform(const Philox4& b, float (&o)[4]) {
#pragma unroll
    for (int j = 0; j < 4; j++) o[j] = (float)(b.w[j] >> 8) * 5.9604644775390625e-08f;  // 2^-24
  }
  __device__ static void normal(const Philox4& b, float (&o)[4]) {
#pragma unroll
    for (int j = 0; j < 2; j++) {
      const float u1 = (float)((b.w[2 * j] >> 8) + 1u) * 5.9604644775390625e-08f;   // (0, 1]
      const float u2 = (float)(b.w[2 * j + 1] >> 8) * 5.9604644775390625e-08f;      // [0, 1)
      const float r = sqrtf(-2.0f * logf(u1));
      float s, c;
      sincospif(2.0f * u2, &s, &c);
      o[2 * j] = r * c;
      o[2 * j + 1] = r * s;
    }
  }
};
template <> struct RandConv<double> {
  static constexpr int kPerBlock = 2;
  __device__ static double u53(unsigned hi, unsigned lo) {
    return ((double)(hi >> 5) * 67108864.0 + (double)(lo >> 6)) * 1.1102230246251565e-16;  // 2^26, 2^-53
  }
  __device__ static void uniform(const Philox4& b, double (&o)[2]) {
    o[0] = u53(b.w[0], b.w[1]);
    o[1] = u53(b.w[2], b.w[3]);
  }
  __device__ static void normal(const Philox4& b, double (&o)[2]) {
    const double u1 = 1.0 - u53(b.w[0], b.w[1]);  // (0, 1]
    const double u2 = u53(b.w[2], b.w[3]);
    const double r = sqrt(-2.0 * log(u1));
    double s, c;
    sincospi(2.0 * u2, &s, &c);
    o[0] = r * c;
    o[1] = r * s;
  }
};

template <typename T, bool NORMAL>
__global__ __launch_bounds__(256) void rand_kernel(long n, unsigned long long seed, unsigned long long offset, T* __restrict__ y, bool vec) {
  constexpr int N = RandConv<T>::kPerBlock;
  typedef typename Vec16<T>::type V;
  const long blk = (long)blockIdx.x * 256 + threadIdx.x;
  const long i0 = blk * N;
  if (i0 >= n) return;
  const Philox4 b = philox4x32_10(offset + (unsigned long long)blk, seed);
  T o[N];
  if (NORMAL) RandConv<T>::normal(b, o); else RandConv<T>::uniform(b, o);
  if (vec && i0 + N <= n) {
    V v;
#pragma unroll
    for (int j = 0; j < N; j++) v[j] = o[j];
    st_stream(reinterpret_cast<V*>(y + i0), v);
  } else {
#pragma unroll
    for (int j = 0; j < N; j++)
      if (i0 + j < n) y[i0 + j] = o[j];
  }
}

// Generator position kept in device memory: state[0] = seed, state[1] = next unused counter.  A launch that reads its position
// from there and a one-lane launch that moves it forward can be captured into a hipGraph: every replay draws fresh numbers,
// which kernel arguments frozen at capture time cannot give.
template <typename T, bool NORMAL>
__global__ __launch_bounds__(256) void rand_state_kernel(long n, const unsigned long long* __restrict__ state, T* __restrict__ y, bool vec) {
  constexpr int N = RandConv<T>::kPerBlock;
  typedef typename Vec16<T>::type V;
  const long blk = (long)blockIdx.x * 256 + threadIdx.x;
  const long i0 = blk * N;
  if (i0 >= n) return;
  const Philox4 b = philox4x32_10(state[1] + (unsigned long long)blk, state[0]);
  T o[N];
  if (NORMAL) RandConv<T>::normal(b, o); else RandConv<T>::uniform(b, o);
  if (vec && i0 + N <= n) {
    V v;
#pragma unroll
    for (int j = 0; j < N; j++) v[j] = o[j];
    st_stream(reinterpret_cast<V*>(y + i0), v);
  } else {
#pragma unroll
    for (int j = 0; j < N; j++)
      if (i0 + j < n) y[i0 + j] = o[j];
  }
}
static __global__ void rand_state_advance_kernel(unsigned long long* state, unsigned long long blocks) {
  if (threadIdx.x == 0 && blockIdx.x == 0) state[1] += blocks;
}

// Counters a call of n elements consumes.
template <typename T> inline unsigned long long rand_blocks(long n) {
  constexpr int N = RandConv<T>::kPerBlock;
  return n <= 0 ? 0ull : (unsigned long long)((n + N - 1) / N);
}

template <typename T, bool NORMAL>
inline void launch_rand(hipStream_t stream, long n, unsigned long long seed, unsigned long long offset, T* y) {
  if (n <= 0) return;
  const unsigned long long blocks = rand_blocks<T>(n);
  const unsigned long long grid = (blocks + 255) / 256;
  if (grid > 0x7fffffffull) { record_error("rand: too many elements"); return; }
  hipLaunchKernelGGL((rand_kernel<T, NORMAL>), dim3((unsigned)grid), dim3(256), 0, stream, n, seed, offset, y, aligned16(y));
}

template <typename T, bool NORMAL>
inline void launch_rand_state(hipStream_t stream, long n, unsigned long long* state, T* y) {
  if (n <= 0) return;
  if (state == nullptr) { record_error("rand_state: null state"); return; }
  const unsigned long long blocks = rand_blocks<T>(n);
  const unsigned long long grid = (blocks + 255) / 256;
  if (grid > 0x7fffffffull) { record_error("rand: too many elements"); return; }
  hipLaunchKernelGGL((rand_state_kernel<T, NORMAL>), dim3((unsigned)grid), dim3(256), 0, stream, n, state, y, aligned16(y));
  hipLaunchKernelGGL(rand_state_advance_kernel, dim3(1), dim3(64), 0, stream, state, blocks);
}

}  // namespace knet8
