// In-kernel timelines of the launch shapes behind the roofline tables, on cold (rotating) buffers: every workgroup stamps the 100 MHz
// wall clock when it starts, when its loads have arrived (phase boundary) and when its last store has been acknowledged, together with
// the XCD it ran on.  What the stamps separate is the time a launch spends inside its workgroups (first start to last end) from the fixed
// cost around it, and how evenly the workgroups of a static launch are served.  The stamped kernels restate the library's launch shapes
// (same headers, same helper routines, same tile sizes); the stamps cost a few hundred nanoseconds per workgroup.
//
// Measurement tool, run by `python3 bench.py --timeline` (needs hipcc); it is not part of libknet8.so.
#include "../../knet.jl_amd/csrc/knet8_softmax.h"
#include "../../knet.jl_amd/csrc/knet8_reduce.h"
#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <vector>
using namespace knet8;
namespace knet8 {   // the host services the headers expect; nothing here allocates through the library
void record_error(const char* w) { printf("ERR %s\n", w); }
void check_launch(const char*) {}
Workspace workspace_for(hipStream_t, size_t, size_t) { return Workspace{nullptr, nullptr}; }
void* scalar_slot(hipStream_t) { return nullptr; }
void fetch_scalar(hipStream_t, const void*, void*, size_t) {}
int tuning(int k) { return k == kTuneNumCUs ? 256 : 0; }
}
#define CK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("ERR %s line %d\n", hipGetErrorString(e_), __LINE__); exit(1); } } while (0)
typedef float v4 __attribute__((ext_vector_type(4)));
struct Stamp { unsigned long long t0, t1, t2; unsigned xcc, pad; };

__device__ __forceinline__ void put_stamp(Stamp* st, long slot, unsigned long long t0, unsigned long long t1, unsigned long long t2) {
  Stamp q; q.t0 = t0; q.t1 = t1; q.t2 = t2; q.xcc = __builtin_amdgcn_s_getreg((3 << 11) | 20) & 7; q.pad = 0;   // XCC_ID, bits 3:0
  st[slot] = q;
}
__device__ __forceinline__ void wait_all() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// (a) one-shot elementwise 2R+1W: 256-lane workgroups, one 16-byte vector per lane and operand (the library's ew_vec_kernel shape)
__global__ __launch_bounds__(256) void oneshot_tl(const v4* a, const v4* b, v4* o, Stamp* st) {
  const unsigned long long t0 = wall_clock64();
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  const v4 x = ld_stream(a + i), y = ld_stream(b + i);
  v4 r;
  for (int e = 0; e < 4; e++) r[e] = x[e] > 0.f ? y[e] : 0.f;
  st_stream(o + i, r);
  wait_all();
  if (threadIdx.x == 0 && (blockIdx.x & 63) == 0) put_stamp(st, blockIdx.x >> 6, t0, t0, wall_clock64());
}

// (b) logsoftmaxback, one 32000-row column per 1024-lane workgroup: dy held in registers, reduce, then y streamed and dx stored.
// At most 64 registers per lane, as in the library's kernel, so that two workgroups share a compute unit and all 512 columns are resident at once.
__global__ __launch_bounds__(1024) __attribute__((amdgpu_waves_per_eu(8, 8))) void lsb_tl(int m, const float* __restrict__ y, const float* __restrict__ dy, float* __restrict__ dx, Stamp* st) {
  constexpr int BT = 1024, ITEMS = 8;
  __shared__ float lds[16];
  const unsigned long long t0 = wall_clock64();
  const int tl = threadIdx.x;
  const long base = (long)blockIdx.x * m;
  const v4* dc = reinterpret_cast<const v4*>(dy + base);
  const v4* yc = reinterpret_cast<const v4*>(y + base);
  v4* oc = reinterpret_cast<v4*>(dx + base);
  const int nb = m / 4;
  v4 rd[ITEMS];
#pragma unroll
  for (int i = 0; i < ITEMS; i++) { const int r = tl + i * BT; rd[i] = r < nb ? ld_stream(dc + r) : v4{0, 0, 0, 0}; }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < ITEMS; i++) s += (rd[i][0] + rd[i][1]) + (rd[i][2] + rd[i][3]);
  s = block_reduce<float, 16>(s, lds, AddFn(), 0.f);
  const unsigned long long t1 = wall_clock64();
#pragma unroll
  for (int i = 0; i < ITEMS; i++) {
    const int r = tl + i * BT;
    if (r < nb) {
      const v4 a = ld_stream(yc + r);
      v4 o;
      for (int e = 0; e < 4; e++) { const float ex = dev_exp(a[e]); const float p = ex * s; o[e] = rd[i][e] - p; }
      st_stream(oc + r, o);
    }
  }
  wait_all();
  if (tl == 0) put_stamp(st, blockIdx.x, t0, t1, wall_clock64());
}

// (c) fused nll backward, one column per 1024-lane workgroup: x held in registers, (max, sum) reduce, dx stored
__global__ __launch_bounds__(1024) __attribute__((amdgpu_waves_per_eu(8, 8))) void nll_tl(int m, const float* a, float* out, const int* labels, float scale, float* loss, Stamp* st) {
  constexpr int BT = 1024, ITEMS = 8, NW = 16;
  __shared__ float lds_m[16], lds_s[16];
  const unsigned long long t0 = wall_clock64();
  const int tl = threadIdx.x;
  const long col = blockIdx.x;
  const v4* ac = reinterpret_cast<const v4*>(a + col * m);
  v4* oc = reinterpret_cast<v4*>(out + col * m);
  const int nb = m / 4;
  const float ninf = -INFINITY;
  int lab = labels[col];
  if (lab < 0 || lab > m) lab = 0;
  const float alab = (tl == 0 && lab > 0) ? a[col * m + lab - 1] : 0.f;
  v4 rv[ITEMS];
#pragma unroll
  for (int i = 0; i < ITEMS; i++) { const int r = tl + i * BT; rv[i] = r < nb ? ld_stream(ac + r) : v4{ninf, ninf, ninf, ninf}; }
  float mt = ninf;
#pragma unroll
  for (int i = 0; i < ITEMS; i++) for (int e = 0; e < 4; e++) mt = mt > rv[i][e] ? mt : rv[i][e];
  float s = 0.f;
  const float mref = mt == ninf ? 0.f : mt;
#pragma unroll
  for (int i = 0; i < ITEMS; i++) for (int e = 0; e < 4; e++) { const float ex = dev_exp(rv[i][e] - mref); rv[i][e] = ex; s += ex; }
  const unsigned long long t1 = wall_clock64();
  MaxSum<float> ms = {mt, s};
  ms = ms_wave_reduce(ms);
  const int lane = tl & 63, wave = tl >> 6;
  if (lane == 0) { lds_m[wave] = ms.m; lds_s[wave] = ms.s; }
  __syncthreads();
  MaxSum<float> t = {lane < NW ? lds_m[lane] : ninf, lane < NW ? lds_s[lane] : 0.f};
  ms = ms_wave_reduce(t);
  const float logS = dev_log(ms.s);
  const float f = (mt == ninf ? 0.f : dev_exp(mt - ms.m) / ms.s) * scale;
  if (tl == 0) loss[col] = lab > 0 ? -((alab - ms.m) - logS) : 0.f;
#pragma unroll
  for (int i = 0; i < ITEMS; i++) {
    const int r = tl + i * BT;
    if (r < nb) {
      v4 vo;
      for (int e = 0; e < 4; e++) { const float p = rv[i][e] * f; const float dlp = (r * 4 + e + 1 == lab) ? -scale : 0.f; vo[e] = lab == 0 ? 0.f : dlp + p; }
      st_stream(oc + r, vo);
    }
  }
  wait_all();
  if (tl == 0) put_stamp(st, blockIdx.x, t0, t1, wall_clock64());
}

// (d) sum over the strided dimension: 256-row tiles, 16 waves on the columns of one of P parts, partial tiles combined by the last
// workgroup of each tile (ticket)
__global__ __launch_bounds__(1024) void strided_tl(const float* __restrict__ x, long s1, long d, long atiles, long kchunk, unsigned P, float* __restrict__ y,
                                                   float* partial, unsigned* counters, Stamp* st) {
  typedef RedSum<float> Op;
  constexpr int NV = 4, TILE = 256, NW = 16, U = 2;
  __shared__ float lds[NW][TILE];
  __shared__ unsigned flag;
  const unsigned long long t0 = wall_clock64();
  const long group = blockIdx.x / P;
  const unsigned p = blockIdx.x % P;
  const long at = group % atiles;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const long a0 = at * TILE + (long)lane * NV;
  const long k0 = (long)p * kchunk;
  long k1 = k0 + kchunk;
  if (k1 > d) k1 = d;
  float acc[NV] = {0, 0, 0, 0};
  strided_walk<float, Op, NV, true, NW, U, false>(x + a0, s1, k0, k1, wave, acc, ~0u);
  const float sink = (acc[0] + acc[1]) + (acc[2] + acc[3]);
  asm volatile("" ::"v"(sink));
  const unsigned long long t1 = wall_clock64();
  for (int e = 0; e < NV; e++) lds[wave][lane * NV + e] = acc[e];
  __syncthreads();
  if (threadIdx.x < TILE) { float r = 0; for (int w = 0; w < NW; w++) r += lds[w][threadIdx.x]; st_coherent(partial + (group * P + p) * TILE + threadIdx.x, r); }
  if (last_block_ticket(counters + group, P, &flag)) {
    for (int e = 0; e < NV; e++) acc[e] = 0;
    strided_walk<float, Op, NV, false, NW, U, false>(partial + group * P * TILE + lane * NV, TILE, 0, P, wave, acc);
    if (threadIdx.x == 0) st_coherent(counters + group, 0u);
    for (int e = 0; e < NV; e++) lds[wave][lane * NV + e] = acc[e];
    __syncthreads();
    if (threadIdx.x < TILE) { float r = 0; for (int w = 0; w < NW; w++) r += lds[w][threadIdx.x]; y[at * TILE + threadIdx.x] = r; }
    wait_all();
  }
  if (threadIdx.x == 0) put_stamp(st, blockIdx.x, t0, t1, wall_clock64());
}

static void report(const char* tag, const std::vector<Stamp>& h, double bytes) {
  unsigned long long base = ~0ull, last = 0;
  for (auto& s : h) { base = std::min(base, s.t0); last = std::max(last, s.t2); }
  const double span = (last - base) * 0.01;
  printf("%s\n  first workgroup start to last workgroup end: %.2f us  (%.0f GB/s inside the launch)\n", tag, span, bytes / span * 1e-3);
  double xm[8] = {0}, xe[8] = {0};
  int xn[8] = {0};
  std::vector<double> st, mid, en;
  for (auto& s : h) {
    const int x = s.xcc & 7;
    xm[x] += (s.t1 - base) * 0.01; xe[x] += (s.t2 - base) * 0.01; xn[x]++;
    st.push_back((s.t0 - base) * 0.01); mid.push_back((s.t1 - base) * 0.01); en.push_back((s.t2 - base) * 0.01);
  }
  auto pct = [](std::vector<double> v, const char* nm) {
    std::sort(v.begin(), v.end());
    const size_t n = v.size();
    printf("  %-13s min %6.2f  p10 %6.2f  p50 %6.2f  p90 %6.2f  max %6.2f us\n", nm, v[0], v[n / 10], v[n / 2], v[n * 9 / 10], v[n - 1]);
  };
  pct(st, "start"); pct(mid, "loads arrived"); pct(en, "end");
  printf("  mean end per XCD:");
  for (int x = 0; x < 8; x++) if (xn[x]) printf(" %d: %.1f", x, xe[x] / xn[x]);
  printf("\n");
}

template <typename F> static float event_time(F launch, int nbuf, int reps = 48) {
  for (int i = 0; i < nbuf; i++) launch(i);
  CK(hipDeviceSynchronize());
  hipEvent_t e0, e1;
  CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
  float best = 1e30f;
  for (int rep = 0; rep < 3; rep++) {
    CK(hipEventRecord(e0));
    for (int i = 0; i < reps; i++) launch(i % nbuf);
    CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1));
    float ms;
    CK(hipEventElapsedTime(&ms, e0, e1));
    best = std::min(best, ms);
  }
  CK(hipEventDestroy(e0)); CK(hipEventDestroy(e1));
  return best / reps * 1e3f;
}

__global__ void fill_pattern(float* p, long n, unsigned seed) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i < n) { unsigned s = (unsigned)i * 2654435761u + seed; s ^= s >> 15; s *= 2246822519u; s ^= s >> 13; p[i] = ((float)(s >> 8) / 8388608.f - 1.f) * 4.f; }
}
__global__ void empty_kernel() {}

int main() {
  Stamp* st;
  CK(hipMalloc(&st, sizeof(Stamp) * 65536));
  printf("MI355X launch timelines, cold buffers (8-10 rotating sets, more than 1 GB per round); times in microseconds from the first workgroup's start.\n");
  {
    float us = event_time([&](int) { hipLaunchKernelGGL(empty_kernel, dim3(1), dim3(64), 0, 0); }, 1, 400);
    printf("an empty kernel, back to back: %.2f us per launch (the fixed cost of a launch on this stream)\n\n", us);
  }
  {
    const int m = 32000, n = 512, NBUF = 8;
    const size_t cnt = (size_t)m * n;
    float *y[NBUF], *dy[NBUF], *dx[NBUF];
    for (int b = 0; b < NBUF; b++) {
      CK(hipMalloc(&y[b], cnt * 4)); CK(hipMalloc(&dy[b], cnt * 4)); CK(hipMalloc(&dx[b], cnt * 4));
      hipLaunchKernelGGL(fill_pattern, dim3((unsigned)((cnt + 255) / 256)), dim3(256), 0, 0, y[b], (long)cnt, 3u * b + 1);
      hipLaunchKernelGGL(fill_pattern, dim3((unsigned)((cnt + 255) / 256)), dim3(256), 0, 0, dy[b], (long)cnt, 3u * b + 2);
    }
    int* labels; float* loss;
    CK(hipMalloc(&labels, n * 4)); CK(hipMemset(labels, 0, n * 4)); CK(hipMalloc(&loss, n * 4));
    const long nv = cnt / 4;
    const int nwg = (int)(nv / 256);
    for (int pass = 0; pass < 2; pass++) {   // the first pass warms the code objects; the second is reported
      for (int b = 0; b < NBUF; b++) hipLaunchKernelGGL(oneshot_tl, dim3(nwg), dim3(256), 0, 0, (const v4*)y[b], (const v4*)dy[b], (v4*)dx[b], st);
      CK(hipDeviceSynchronize());
      std::vector<Stamp> h(nwg / 64);
      CK(hipMemcpy(h.data(), st, sizeof(Stamp) * h.size(), hipMemcpyDeviceToHost));
      if (pass) report("(a) one-shot elementwise 2R+1W over the bytes of logsoftmaxback (32000,512): 16000 workgroups of 256 lanes, every 64th stamped", h, 12.0 * cnt);
    }
    float us = event_time([&](int i) { hipLaunchKernelGGL(oneshot_tl, dim3(nwg), dim3(256), 0, 0, (const v4*)y[i], (const v4*)dy[i], (v4*)dx[i], st); }, NBUF);
    printf("  the same launch back to back, HIP events: %.2f us per launch\n\n", us);
    for (int pass = 0; pass < 2; pass++) {
      for (int b = 0; b < NBUF; b++) hipLaunchKernelGGL(lsb_tl, dim3(n), dim3(1024), 0, 0, m, y[b], dy[b], dx[b], st);
      CK(hipDeviceSynchronize());
      std::vector<Stamp> h(n);
      CK(hipMemcpy(h.data(), st, sizeof(Stamp) * n, hipMemcpyDeviceToHost));
      if (pass) report("(b) logsoftmaxback (32000,512): 512 workgroups of 1024 lanes, one column each, all resident at once (two per CU)", h, 12.0 * cnt);
    }
    us = event_time([&](int i) { hipLaunchKernelGGL(lsb_tl, dim3(n), dim3(1024), 0, 0, m, y[i], dy[i], dx[i], st); }, NBUF);
    printf("  the same launch back to back, HIP events: %.2f us per launch\n\n", us);
    for (int pass = 0; pass < 2; pass++) {
      for (int b = 0; b < NBUF; b++) hipLaunchKernelGGL(nll_tl, dim3(n), dim3(1024), 0, 0, m, y[b], dx[b], labels, 1.f / n, loss, st);
      CK(hipDeviceSynchronize());
      std::vector<Stamp> h(n);
      CK(hipMemcpy(h.data(), st, sizeof(Stamp) * n, hipMemcpyDeviceToHost));
      if (pass) report("(c) fused nll backward (32000,512): 512 workgroups of 1024 lanes, one column each", h, 8.0 * cnt);
    }
    us = event_time([&](int i) { hipLaunchKernelGGL(nll_tl, dim3(n), dim3(1024), 0, 0, m, y[i], dx[i], labels, 1.f / n, loss, st); }, NBUF);
    printf("  the same launch back to back, HIP events: %.2f us per launch\n\n", us);
    for (int b = 0; b < NBUF; b++) { CK(hipFree(y[b])); CK(hipFree(dy[b])); CK(hipFree(dx[b])); }
  }
  {
    const long s1 = 4096, d = 8192, n = s1 * d;
    const int NBUF = 10;
    float* X[NBUF];
    float *Y, *partial;
    unsigned* counters;
    for (int b = 0; b < NBUF; b++) { CK(hipMalloc(&X[b], n * 4)); hipLaunchKernelGGL(fill_pattern, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, 0, X[b], n, 5u * b + 1); }
    CK(hipMalloc(&Y, s1 * 4)); CK(hipMalloc(&partial, 8 << 20)); CK(hipMalloc(&counters, 1 << 16)); CK(hipMemset(counters, 0, 1 << 16));
    const unsigned P = 16;
    const long atiles = 16, kchunk = d / P;
    for (int pass = 0; pass < 2; pass++) {
      for (int b = 0; b < NBUF; b++) hipLaunchKernelGGL(strided_tl, dim3((unsigned)(atiles * P)), dim3(1024), 0, 0, X[b], s1, d, atiles, kchunk, P, Y, partial, counters, st);
      CK(hipDeviceSynchronize());
      std::vector<Stamp> h(atiles * P);
      CK(hipMemcpy(h.data(), st, sizeof(Stamp) * h.size(), hipMemcpyDeviceToHost));
      if (pass) report("(d) sum over dims=2 of (4096,8192): 16 row tiles x 16 parts = 256 workgroups of 1024 lanes; 'loads arrived' = own columns summed, 'end' = after the ticket (and the combine, for the last of a tile)", h, 4.0 * (n + s1));
    }
    float us = event_time([&](int i) { hipLaunchKernelGGL(strided_tl, dim3((unsigned)(atiles * P)), dim3(1024), 0, 0, X[i], s1, d, atiles, kchunk, P, Y, partial, counters, st); }, NBUF);
    printf("  the same launch back to back, HIP events: %.2f us per launch\n", us);
  }
  return 0;
}
