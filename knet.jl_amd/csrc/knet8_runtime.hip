// Host runtime of libknet8: error slot, per-stream reduction scratch, device-memory pool for KnetArray
// storage, copies, stream/timer helpers and the hipBLASLt GEMM entry points.
#include "knet8_runtime.h"
#include "knet8_gemm_small.h"
#include "knet8_fused.h"

#include <hipblaslt/hipblaslt.h>
#include <hipblaslt/hipblaslt-ext.hpp>
#include <hipblaslt/hipblaslt-version.h>

#include <atomic>
#include <cstdio>
#include <cstring>
#include <map>
#include <mutex>
#include <random>
#include <string>
#include <tuple>
#include <unordered_map>
#include <vector>

namespace knet8 {

// ---- errors ------------------------------------------------------------------------------------------
static std::mutex g_err_mutex;
static std::string g_err;
static thread_local std::string g_err_out;

void record_error(const char* what) {
  std::lock_guard<std::mutex> lock(g_err_mutex);
  if (g_err.empty()) g_err = what;  // keep the first failure: later ones are usually consequences
}

void check_launch(const char* name) {
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    std::string msg = std::string(name) + ": " + hipGetErrorString(e);
    record_error(msg.c_str());
  }
}

static bool ok(hipError_t e, const char* what) {
  if (e == hipSuccess) return true;
  std::string msg = std::string(what) + ": " + hipGetErrorString(e);
  record_error(msg.c_str());
  return false;
}

// ---- every device allocation and release of the library goes through these two, which count the calls (knet8_stats): a test can
// then assert that an entry point that promises not to allocate made none.
static std::atomic<unsigned long long> g_malloc_calls{0}, g_free_calls{0};
static std::atomic<unsigned long long> g_held_bytes{0};         // scratch, workspaces and scalar slots the library holds outside the pool
static std::atomic<unsigned long long> g_gemm_left_vendor{0};   // plain products that ran on the library's own tiles because hipBLASLt had no algorithm
static hipError_t dev_malloc(void** p, size_t n, bool held = false) {
  g_malloc_calls.fetch_add(1, std::memory_order_relaxed);
  const hipError_t e = hipMalloc(p, n);
  if (held && e == hipSuccess) g_held_bytes.fetch_add(n, std::memory_order_relaxed);
  return e;
}
static void dev_free(void* p, size_t held_bytes = 0) {
  g_free_calls.fetch_add(1, std::memory_order_relaxed);
  g_held_bytes.fetch_sub(held_bytes, std::memory_order_relaxed);
  (void)hipFree(p);
}

// ---- launch-heuristic knobs ------------------------------------------------------------------------------
// Default random stream: seed and the next unused generator counter.  Unseeded, the seed comes from the operating system's
// entropy source at first use, as the reference's generators start from a random seed until seed! is called.
static std::mutex g_rng_mu;
static unsigned long long g_rng_seed = 0, g_rng_offset = 0;
static bool g_rng_seeded = false;
void rng_take(unsigned long long blocks, unsigned long long* seed, unsigned long long* offset) {
  std::lock_guard<std::mutex> lock(g_rng_mu);
  if (!g_rng_seeded) {
    std::random_device rd;
    g_rng_seed = ((unsigned long long)rd() << 32) ^ (unsigned long long)rd();
    g_rng_offset = 0;
    g_rng_seeded = true;
  }
  *seed = g_rng_seed;
  *offset = g_rng_offset;
  g_rng_offset += blocks;
}

static int g_tune[kTuneCount] = {0, 0, 0, 0, 0, 0, 0, 0, 0};
int tuning(int key) {
  if (key < 0 || key >= kTuneCount) return 0;
  if (key == kTuneNumCUs && g_tune[key] == 0) {  // compute units of the current device, asked once
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
      g_tune[key] = n;
    else {
      (void)hipGetLastError();
      g_tune[key] = 256;
    }
  }
  // kTuneGemmSmallMflop stays 0 unless a caller opts in: gemm_S and gemm_bias_act_S go to hipBLASLt (the matrix cores are used through the
  // vendor library only).  A positive value sends products of up to that many MFLOP (2mnk) to the library's own small-product kernels.
  if (key == kTuneDenseBackMflop && g_tune[key] == 0) g_tune[key] = 270;  // dense_back_S and its relatives accept layers whose products have up to this many MFLOP each
  return g_tune[key];
}

// ---- per-stream scratch for split reductions ------------------------------------------------------------
struct StreamScratch {
  void* partial = nullptr;
  size_t partial_bytes = 0;
  unsigned* counters = nullptr;
  size_t ncounters = 0;
  std::vector<void*> retired;
  std::vector<size_t> retired_bytes;
  bool in_graph = false;   // handed out while the stream was being captured: a graph holds the addresses, so knet8_trim leaves them alone
  hipEvent_t t0 = nullptr, t1 = nullptr;
};
static std::mutex g_scratch_mutex;
static std::map<std::pair<int, hipStream_t>, StreamScratch> g_scratch;

static StreamScratch& scratch_of(hipStream_t stream) {
  int dev = 0;
  (void)hipGetDevice(&dev);
  return g_scratch[std::make_pair(dev, stream)];
}

static bool stream_is_capturing(hipStream_t stream) {
  hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
  if (stream == nullptr || hipStreamIsCapturing(stream, &cap) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  return cap != hipStreamCaptureStatusNone;
}

// hipBLASLt workspaces, one per (device, stream), defined with the GEMM entry points below: release the one of a stream that is being
// destroyed, or (every = true) all that no captured graph holds; returns the bytes released.
static size_t gemm_release(int dev, hipStream_t stream, bool every);

static size_t release_scratch(StreamScratch& s) {
  size_t released = s.partial_bytes + s.ncounters * sizeof(unsigned);
  if (s.partial) dev_free(s.partial, s.partial_bytes);
  if (s.counters) dev_free(s.counters, s.ncounters * sizeof(unsigned));
  for (size_t i = 0; i < s.retired.size(); i++) { dev_free(s.retired[i], s.retired_bytes[i]); released += s.retired_bytes[i]; }
  s.partial = nullptr; s.partial_bytes = 0;
  s.counters = nullptr; s.ncounters = 0;
  s.retired.clear(); s.retired_bytes.clear();
  return released;
}

__global__ __launch_bounds__(256) void zero_counters_kernel(unsigned* c, size_t n) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) c[i] = 0u;
}

Workspace workspace_for(hipStream_t stream, size_t partial_bytes, size_t ncounters) {
  if (g_tune[kTuneFailScratch] != 0) {   // set by tests: behave as if the device were out of memory, without touching it
    record_error("reduction scratch: allocation refused (knet8_tune key 5 is set)");
    Workspace none = {nullptr, nullptr};
    return none;
  }
  const bool capturing = stream_is_capturing(stream);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  StreamScratch& s = scratch_of(stream);
  if (capturing) s.in_graph = true;
  // Buffers that have become too small are retired, not freed: launches already queued on the stream, and graphs
  // captured on it, keep using their addresses.  Sizes grow geometrically, so the retired ones add up to less than
  // the current one.  knet8_trim (after a device-wide wait) and knet8_stream_destroy release them.
  if (s.partial_bytes < partial_bytes) {
    if (s.partial) { s.retired.push_back(s.partial); s.retired_bytes.push_back(s.partial_bytes); }
    size_t want = partial_bytes < (size_t(1) << 20) ? (size_t(1) << 20) : 2 * partial_bytes;
    s.partial = nullptr;
    s.partial_bytes = ok(dev_malloc(&s.partial, want, true), "hipMalloc(reduction partials)") ? want : 0;
  }
  if (s.ncounters < ncounters) {
    if (s.counters) { s.retired.push_back(s.counters); s.retired_bytes.push_back(s.ncounters * sizeof(unsigned)); }
    size_t want = ncounters < 4096 ? 4096 : 2 * ncounters;
    s.counters = nullptr;
    s.ncounters = 0;
    // Zeroed by a fill kernel on the launching stream itself, so that the zeroing is ordered before the kernel that is about to
    // use the counters.  (A hipMemset goes to the null stream, which a non-blocking stream does not wait for: on recycled memory
    // the first split kernel on a new stream could then count on top of garbage and leave its tickets non-zero for good.  A fill
    // kernel is also what a stream capture can record safely.)
    if (ok(dev_malloc(reinterpret_cast<void**>(&s.counters), want * sizeof(unsigned), true), "hipMalloc(reduction counters)")) {
      hipLaunchKernelGGL(zero_counters_kernel, dim3((unsigned)((want + 255) / 256)), dim3(256), 0, stream, s.counters, want);
      if (ok(hipGetLastError(), "zero_counters_kernel")) s.ncounters = want;
    }
  }
  Workspace w = {s.partial, s.counters};
  return w;
}

// ---- scratch for callers that cannot allocate ---------------------------------------------------------------------
// sum_32_21_noalloc runs the same kernels as sum_32_21 with the partial results and tickets of a split launch in this fixed array
// instead of the per-stream buffers above (which grow through hipMalloc).  Every GPU the library runs on holds its own copy, at its
// own address, until the process ends.  In host code the array's name is only a handle for hipGetSymbolAddress: the address a kernel
// can use is asked from the runtime once per device and kept.
constexpr size_t kStaticPartialBytes = size_t(1) << 20;
constexpr size_t kStaticCounters = 16384;   // tickets sit 64 apart: 256 output groups
static __device__ __align__(256) unsigned char scratch[kStaticPartialBytes + kStaticCounters * sizeof(unsigned)];

constexpr int kMaxDevices = 64;
static std::mutex g_static_mutex;
static unsigned char* g_static_ptr[kMaxDevices] = {nullptr};

static unsigned char* static_scratch_ptr() {
  int dev = -1;
  if (!ok(hipGetDevice(&dev), "hipGetDevice") || dev < 0 || dev >= kMaxDevices) {
    record_error("sum_32_21_noalloc: no current device");
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(g_static_mutex);
  if (g_static_ptr[dev] == nullptr) {
    unsigned char* ptr = nullptr;
    if (!ok(hipGetSymbolAddress(reinterpret_cast<void**>(&ptr), HIP_SYMBOL(scratch)), "hipGetSymbolAddress(scratch)") || ptr == nullptr) return nullptr;
    g_static_ptr[dev] = ptr;
  }
  return g_static_ptr[dev];
}

static Workspace static_scratch_get(void*, hipStream_t stream, size_t partial_bytes, size_t ncounters) {
  Workspace none = {nullptr, nullptr};
  if (partial_bytes > kStaticPartialBytes || ncounters > kStaticCounters) {
    char buf[256];
    snprintf(buf, sizeof(buf), "sum_32_21_noalloc: the split of this shape needs %zu bytes of partial results and %zu tickets; the library's fixed scratch "
             "holds %zu bytes and %zu tickets (use sum_32_21)", partial_bytes, ncounters, kStaticPartialBytes, kStaticCounters);
    record_error(buf);
    return none;
  }
  unsigned char* base = static_scratch_ptr();
  if (base == nullptr) return none;
  unsigned* counters = reinterpret_cast<unsigned*>(base + kStaticPartialBytes);
  // The array keeps whatever the last call on this GPU left in it: the tickets this launch draws start from zero by a fill kernel on
  // the same stream (a kernel, not a memset node, so the call can be captured into a graph).
  if (ncounters > 0) {
    hipLaunchKernelGGL(zero_counters_kernel, dim3((unsigned)((ncounters + 255) / 256)), dim3(256), 0, stream, counters, ncounters);
    if (!ok(hipGetLastError(), "zero_counters_kernel")) return none;
  }
  Workspace w = {base, counters};
  return w;
}

// One slot per (host thread, device, stream): two threads that call a `_20` entry point on the same stream (the plain twins all use the
// null stream; the reference builds with --default-stream per-thread, src/libknet8/build.jl:5) must not read each other's result.
// 256 bytes each, kept until the process ends.
void* scalar_slot(hipStream_t stream) {
  thread_local std::map<std::pair<int, hipStream_t>, void*> slots;
  int dev = 0;
  (void)hipGetDevice(&dev);
  void*& p = slots[std::make_pair(dev, stream)];
  if (!p && !ok(dev_malloc(&p, 256, true), "hipMalloc(scalar slot)")) p = nullptr;
  return p;
}

void fetch_scalar(hipStream_t stream, const void* dev, void* host, size_t nbytes) {
  if (!dev) return;
  if (ok(hipMemcpyAsync(host, dev, nbytes, hipMemcpyDeviceToHost, stream), "hipMemcpyAsync(scalar)"))
    ok(hipStreamSynchronize(stream), "hipStreamSynchronize(scalar)");
}

// ---- device-memory pool ---------------------------------------------------------------------------------
// Freed blocks are kept on per-size free lists and handed out again without touching the driver, as the
// reference's KnetPtr pool does (src/knetarrays/kptr.jl:105-142; an uncached allocation costs ~0.5 ms there,
// kptr.jl:187).  Sizes are rounded up to {1, 1.25, 1.5, 1.75} x 2^k (>= 256 bytes), so at most 25 % is lost
// to rounding.  When hipMalloc fails the free lists are released and the allocation retried once.
//
// Placement of large blocks.  Measured on MI355X with the 2R+1W gradient kernels on 1 GiB operands (a 16 x 16 map of the start
// offsets of y and dx relative to dy, in KB): the time depends on where the three arrays start relative to each other modulo
// 16 KB -- 499-513 us when the output starts at the same residue as dy (what page-aligned allocations give; 522-529 us at odd
// multiples of 16 KB), 480-485 us when it starts 5-7 KB later and y 1-5 KB later: same-index accesses of the streams then do not
// meet in the same memory channel and bank.  Blocks of 1 MB and more are therefore handed out at a start address whose residue
// modulo 16 KB advances by 21*256 bytes (5.25 KB) from one new block to the next (all 64 multiples of 256 come up before any
// repeats), so arrays allocated one after the other -- a layer's dy and then its dx -- sit in the good region of that map.
struct Pool {
  std::mutex mutex;
  std::unordered_map<size_t, std::vector<void*>> free_lists;  // rounded size -> blocks (as handed out)
  std::unordered_map<void*, size_t> live;                     // block -> rounded size
  std::unordered_map<void*, void*> base_of;                   // block handed out at an offset -> what hipMalloc returned
  size_t bytes_live = 0, bytes_cached = 0, nmalloc = 0, nhit = 0;
  unsigned next_color = 0;
};
static Pool g_pool;
constexpr size_t kColorPeriod = 16384, kColorStep = 21 * 256, kColorMinBytes = size_t(1) << 20;

static hipError_t pool_device_malloc(Pool& pool, void** out, size_t sz) {
  if (sz < kColorMinBytes) return dev_malloc(out, sz);
  void* base = nullptr;
  const hipError_t e = dev_malloc(&base, sz + kColorPeriod);
  if (e != hipSuccess) return e;
  const size_t want = (pool.next_color++ * kColorStep) % kColorPeriod;
  const size_t have = reinterpret_cast<uintptr_t>(base) % kColorPeriod;
  const size_t off = ((want + kColorPeriod - have) % kColorPeriod + 255) / 256 * 256 % kColorPeriod;
  *out = static_cast<char*>(base) + off;
  if (off) pool.base_of[*out] = base;
  return hipSuccess;
}

static void pool_device_free(Pool& pool, void* p) {
  auto it = pool.base_of.find(p);
  if (it != pool.base_of.end()) {
    dev_free(it->second);
    pool.base_of.erase(it);
  } else {
    dev_free(p);
  }
}

static size_t round_size(size_t n) {
  if (n <= 256) return 256;
  size_t p = 256;
  while (p * 2 < n) p *= 2;  // p < n <= 2p
  const size_t q = p / 4;
  for (int k = 1; k <= 4; k++)
    if (p + k * q >= n) return p + k * q;
  return 2 * p;
}

static size_t trim_locked(Pool& pool) {
  size_t released = 0;
  for (auto& kv : pool.free_lists) {
    for (void* p : kv.second) {
      pool_device_free(pool, p);
      released += kv.first;
    }
    kv.second.clear();
  }
  pool.bytes_cached = 0;
  return released;
}

}  // namespace knet8

using namespace knet8;

extern "C" {

KNET8_API void* knet8_malloc(size_t nbytes) {
  const size_t sz = round_size(nbytes);
  std::lock_guard<std::mutex> lock(g_pool.mutex);
  void* p = nullptr;
  auto it = g_pool.free_lists.find(sz);
  if (it != g_pool.free_lists.end() && !it->second.empty()) {
    p = it->second.back();
    it->second.pop_back();
    g_pool.bytes_cached -= sz;
    g_pool.nhit++;
  } else {
    hipError_t e = pool_device_malloc(g_pool, &p, sz);
    if (e != hipSuccess) {
      (void)hipGetLastError();
      trim_locked(g_pool);
      e = pool_device_malloc(g_pool, &p, sz);
    }
    if (e != hipSuccess) {
      (void)hipGetLastError();
      record_error("knet8_malloc: out of device memory");
      return nullptr;
    }
    g_pool.nmalloc++;
  }
  g_pool.live[p] = sz;
  g_pool.bytes_live += sz;
  return p;
}

KNET8_API void knet8_free(void* ptr) {
  if (!ptr) return;
  std::lock_guard<std::mutex> lock(g_pool.mutex);
  auto it = g_pool.live.find(ptr);
  if (it == g_pool.live.end()) {
    record_error("knet8_free: pointer was not allocated by knet8_malloc");
    return;
  }
  const size_t sz = it->second;
  g_pool.live.erase(it);
  g_pool.bytes_live -= sz;
  g_pool.free_lists[sz].push_back(ptr);
  g_pool.bytes_cached += sz;
}

KNET8_API size_t knet8_trim(void) {
  (void)hipDeviceSynchronize();
  size_t released = 0;
  {
    std::lock_guard<std::mutex> lock(g_pool.mutex);
    released += trim_locked(g_pool);
  }
  // Nothing is queued any more: the reduction scratch of every stream (current and retired buffers) and the hipBLASLt workspaces go back
  // too, except those a captured graph may still name (handed out while their stream was being captured); the next launch that needs
  // scratch allocates it afresh.
  {
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    for (auto& kv : g_scratch)
      if (!kv.second.in_graph) released += release_scratch(kv.second);
  }
  released += gemm_release(0, nullptr, true);
  return released;
}

KNET8_API void knet8_stats(unsigned long long* out6) {
  size_t free_b = 0, total_b = 0;
  if (hipMemGetInfo(&free_b, &total_b) != hipSuccess) { (void)hipGetLastError(); free_b = total_b = 0; }
  out6[0] = g_malloc_calls.load();
  out6[1] = g_free_calls.load();
  out6[2] = g_held_bytes.load();
  out6[3] = g_gemm_left_vendor.load();
  out6[4] = free_b;
  out6[5] = total_b;
}

KNET8_API void knet8_meminfo(size_t* out4) {
  std::lock_guard<std::mutex> lock(g_pool.mutex);
  out4[0] = g_pool.bytes_live;
  out4[1] = g_pool.bytes_cached;
  out4[2] = g_pool.nmalloc;
  out4[3] = g_pool.nhit;
}

KNET8_API int knet8_memcpy(void* dst, const void* src, size_t nbytes, int kind, hipStream_t stream) {
  if (nbytes == 0) return 0;
  hipMemcpyKind k;
  switch (kind) {
    case 1: k = hipMemcpyHostToDevice; break;
    case 2: k = hipMemcpyDeviceToHost; break;
    case 3: k = hipMemcpyDeviceToDevice; break;
    default: record_error("knet8_memcpy: kind must be 1 (h2d), 2 (d2h) or 3 (d2d)"); return -1;
  }
  if (!ok(hipMemcpyAsync(dst, src, nbytes, k, stream), "hipMemcpyAsync")) return -1;
  if (kind != 3 && !ok(hipStreamSynchronize(stream), "hipStreamSynchronize")) return -1;
  return 0;
}

KNET8_API int knet8_device_count(void) {
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess) {
    (void)hipGetLastError();
    return 0;
  }
  return n;
}

KNET8_API int knet8_set_device(int dev) { return ok(hipSetDevice(dev), "hipSetDevice") ? 0 : -1; }

KNET8_API hipStream_t knet8_stream_create(void) {
  hipStream_t s = nullptr;
  ok(hipStreamCreateWithFlags(&s, hipStreamNonBlocking), "hipStreamCreate");
  return s;
}

KNET8_API void knet8_stream_destroy(hipStream_t stream) {
  if (!stream) return;
  // The stream's reduction scratch goes with it (a later stream may get the same handle and must start from its own, freshly
  // zeroed counters).  Graphs captured on the stream hold the scratch addresses: destroy them first.
  ok(hipStreamSynchronize(stream), "hipStreamSynchronize");
  {
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    int dev = 0;
    (void)hipGetDevice(&dev);
    auto it = g_scratch.find(std::make_pair(dev, stream));
    if (it != g_scratch.end()) {
      StreamScratch& s = it->second;
      release_scratch(s);
      if (s.t0) (void)hipEventDestroy(s.t0);
      if (s.t1) (void)hipEventDestroy(s.t1);
      g_scratch.erase(it);
    }
    gemm_release(dev, stream, false);   // the stream's hipBLASLt workspace: a later stream with the same handle starts without one
  }
  ok(hipStreamDestroy(stream), "hipStreamDestroy");
}

KNET8_API int knet8_synchronize(hipStream_t stream) { return ok(hipStreamSynchronize(stream), "hipStreamSynchronize") ? 0 : -1; }

KNET8_API void knet8_timer_start(hipStream_t stream) {
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  StreamScratch& s = scratch_of(stream);
  if (!s.t0) {
    ok(hipEventCreate(&s.t0), "hipEventCreate");
    ok(hipEventCreate(&s.t1), "hipEventCreate");
  }
  ok(hipEventRecord(s.t0, stream), "hipEventRecord");
}

KNET8_API float knet8_timer_stop(hipStream_t stream) {
  hipEvent_t t0, t1;
  {
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    StreamScratch& s = scratch_of(stream);
    t0 = s.t0;
    t1 = s.t1;
  }
  if (!t0) return -1.f;
  float ms = -1.f;
  if (ok(hipEventRecord(t1, stream), "hipEventRecord") && ok(hipEventSynchronize(t1), "hipEventSynchronize"))
    ok(hipEventElapsedTime(&ms, t0, t1), "hipEventElapsedTime");
  return ms;
}

KNET8_API void* knet8_event_create(void) {
  hipEvent_t e = nullptr;
  ok(hipEventCreate(&e), "hipEventCreate");
  return e;
}

KNET8_API void knet8_event_destroy(void* event) {
  if (event) ok(hipEventDestroy(static_cast<hipEvent_t>(event)), "hipEventDestroy");
}

KNET8_API void knet8_event_record(void* event, hipStream_t stream) { ok(hipEventRecord(static_cast<hipEvent_t>(event), stream), "hipEventRecord"); }

KNET8_API float knet8_event_elapsed(void* start, void* stop) {
  float ms = -1.f;
  if (ok(hipEventSynchronize(static_cast<hipEvent_t>(stop)), "hipEventSynchronize"))
    ok(hipEventElapsedTime(&ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)), "hipEventElapsedTime");
  return ms;
}

// ---- hipGraph capture of a launch sequence ------------------------------------------------------------------
// A backward step over small arrays is bound by launch latency, not bandwidth: capture the whole sequence once and
// replay it with one call.  Capture needs a caller-created stream; everything the sequence needs
// from the driver (pool blocks, reduction scratch, GEMM plans) should exist already, i.e. the sequence has run once
// eagerly on the same stream (relaxed mode tolerates a late hipMalloc, but not the synchronisation a new GEMM plan needs).  No memset nodes are recorded: the library clears memory with fill kernels only.
KNET8_API int knet8_graph_begin(hipStream_t stream) {
  if (!stream) {
    record_error("knet8_graph_begin: capture needs a stream created with knet8_stream_create");
    return -1;
  }
  return ok(hipStreamBeginCapture(stream, hipStreamCaptureModeRelaxed), "hipStreamBeginCapture") ? 0 : -1;
}

KNET8_API void* knet8_graph_end(hipStream_t stream) {
  hipGraph_t graph = nullptr;
  if (!ok(hipStreamEndCapture(stream, &graph), "hipStreamEndCapture") || !graph) return nullptr;
  hipGraphExec_t exec = nullptr;
  const bool inst = ok(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0), "hipGraphInstantiate");
  (void)hipGraphDestroy(graph);
  return inst ? exec : nullptr;
}

KNET8_API int knet8_graph_launch(void* graph, hipStream_t stream) {
  return ok(hipGraphLaunch(static_cast<hipGraphExec_t>(graph), stream), "hipGraphLaunch") ? 0 : -1;
}

KNET8_API void knet8_graph_destroy(void* graph) {
  if (graph) ok(hipGraphExecDestroy(static_cast<hipGraphExec_t>(graph)), "hipGraphExecDestroy");
}

KNET8_API const char* knet8_last_error(void) {
  std::lock_guard<std::mutex> lock(g_err_mutex);
  if (g_err.empty()) return nullptr;
  g_err_out = g_err;
  g_err.clear();
  return g_err_out.c_str();
}

KNET8_API int knet8_version(void) { return 200; }

// Hash of the sources this binary was built from (csrc/*.h, *.hip, gen_knet8.py, build.py), written by build.py: lets a loader refuse a
// stale library.
#ifndef KNET8_BUILD_ID
#define KNET8_BUILD_ID "unknown"
#endif
KNET8_API const char* knet8_build_id(void) { return KNET8_BUILD_ID; }

KNET8_API void sum_32_21_noalloc(int nx, float* x, int sy, int ny, float* y, hipStream_t stream) {
  const ScratchSource src = {static_scratch_get, nullptr, kStaticPartialBytes, kStaticCounters};
  reduce_21<float, RedSum<float>>(stream, nx, x, sy, ny, y, &src);
  check_launch("sum_32_21_noalloc");
}

KNET8_API void knet8_seed(unsigned long long seed) {
  std::lock_guard<std::mutex> lock(g_rng_mu);
  g_rng_seed = seed;
  g_rng_offset = 0;
  g_rng_seeded = true;
}

#ifdef KNET8_TIMELINE
// Measurement build only: the device buffer (kTlSlots stamps of 32 bytes) the stamped kernels write to from now on; null switches the stamps off.
static knet8::TlStamp* g_timeline = nullptr;
KNET8_API void knet8_timeline_set(void* buffer) { g_timeline = static_cast<knet8::TlStamp*>(buffer); }
#endif

KNET8_API int knet8_tune(int key, int value) {
  if (key < 0 || key >= kTuneCount) return -1;
  const int old = g_tune[key];
  if (value >= 0) g_tune[key] = value;  // 0 restores the default
  return old;
}

}  // extern "C"

// ---- GEMM through hipBLASLt ----------------------------------------------------------------------------------
namespace knet8 {

#ifdef KNET8_TIMELINE
TlStamp* timeline_buffer() { return g_timeline; }
#endif

struct GemmBatch {   // strided batch: product b uses A + b*sa, B + b*sb, C + b*sc (elements)
  int count = 1;
  long long sa = 0, sb = 0, sc = 0;
};
struct GemmKey {
  int dev, dtype, ta, tb, m, n, k, lda, ldb, ldc, batch, epilogue;
  long long sa, sb, sc;
  bool operator<(const GemmKey& o) const {
    return std::tie(dev, dtype, ta, tb, m, n, k, lda, ldb, ldc, batch, epilogue, sa, sb, sc) <
           std::tie(o.dev, o.dtype, o.ta, o.tb, o.m, o.n, o.k, o.lda, o.ldb, o.ldc, o.batch, o.epilogue, o.sa, o.sb, o.sc);
  }
};
struct GemmPlan {
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatrixLayout_t la = nullptr, lb = nullptr, lc = nullptr;
  hipblasLtMatmulAlgo_t algo;
  size_t workspace = 0;
  bool valid = false;        // descriptors and an algorithm exist
  bool timed = false;        // the algorithm was chosen by timing the candidates (not possible while the stream is being captured)
  bool unsupported = false;  // the vendor library has no kernel for this problem with this epilogue: callers take the separate bias pass
};
struct GemmWs {
  void* p = nullptr;
  bool in_graph = false;   // used by a product recorded into a graph: knet8_trim leaves it alone
};
static std::mutex g_gemm_mutex;
static std::map<int, hipblasLtHandle_t> g_lt;
static std::map<GemmKey, GemmPlan> g_plans;
static std::map<std::pair<int, hipStream_t>, GemmWs> g_gemm_ws;
static const size_t kGemmWorkspace = size_t(64) << 20;
// Bumped whenever a workspace is released: the per-thread shortcut below then forgets what it remembered.
static std::atomic<unsigned long long> g_gemm_generation{1};

static size_t gemm_release(int dev, hipStream_t stream, bool every) {
  std::lock_guard<std::mutex> lock(g_gemm_mutex);
  size_t released = 0;
  for (auto it = g_gemm_ws.begin(); it != g_gemm_ws.end();) {
    const bool hit = every ? !it->second.in_graph : (it->first.first == dev && it->first.second == stream);
    if (hit) {
      if (it->second.p) { dev_free(it->second.p, kGemmWorkspace); released += kGemmWorkspace; }
      it = g_gemm_ws.erase(it);
    } else {
      ++it;
    }
  }
  if (released) g_gemm_generation.fetch_add(1);
  return released;
}

// The last plain products of this thread: problem, stream, operands, and everything the vendor call needs.  A repeat of the problem (the
// same layer of the same model in the next step) goes straight to the vendor call: no map lookups, the lock held for the call only.  When
// the operands repeat as well -- the pool hands a steady-state training step the same blocks every time -- the call is *prepared*: the
// vendor library's extension interface builds the kernel's arguments once (hipblaslt_ext::Gemm::initialize) and every later call only
// launches them (run), which costs a caller about what a plain kernel launch costs instead of a full hipblasLtMatmul.  Only plans that are
// final (algorithm chosen by timing) and carry no bias pointer are remembered; plans are never destroyed once valid.
struct GemmRecent {
  GemmKey key;
  hipStream_t stream = nullptr;
  const GemmPlan* plan = nullptr;
  hipblasLtHandle_t handle = nullptr;
  void* ws = nullptr;
  unsigned long long generation = 0;   // 0: empty
  const void *A = nullptr, *B = nullptr;
  void* C = nullptr;
  double alpha = 0, beta = 0;          // the scalars of the prepared call (a float is held exactly)
  union { float f; double d; } alpha_t, beta_t;   // what the prepared arguments point to
  int repeats = 0;                     // calls in a row with these operands and scalars
  bool no_prepare = false;             // the extension interface refused this problem: stay with hipblasLtMatmul
  hipblaslt_ext::Gemm* prepared = nullptr;
  void reset() {
    delete prepared;
    prepared = nullptr;
    generation = 0; repeats = 0; no_prepare = false;
  }
  ~GemmRecent() { delete prepared; }
};
// The extension interface is a C++ class whose layout belongs to one build of the vendor library.  A process may have resolved libhipblaslt.so.1 to
// another build than the one whose headers this file was compiled against (a Python process that imported PyTorch first gets the copy PyTorch
// bundles): prepared calls are used only when the loaded library reports the very revision of those headers, otherwise every product stays on the
// C interface (hipblasLtMatmul), whose ABI is stable.
#define KNET8_STR2(x) #x
#define KNET8_STR(x) KNET8_STR2(x)
static bool ext_interface_matches(hipblasLtHandle_t h) {
  static int state = -1;   // (called under g_gemm_mutex)
  if (state < 0) {
    char rev[256] = {0};
    int version = 0;
    const bool ok = hipblasLtGetVersion(h, &version) == HIPBLAS_STATUS_SUCCESS && hipblasLtGetGitRevision(h, rev) == HIPBLAS_STATUS_SUCCESS &&
                    version == HIPBLASLT_VERSION_MAJOR * 100000 + HIPBLASLT_VERSION_MINOR * 100 + HIPBLASLT_VERSION_PATCH &&
                    std::string(rev) == KNET8_STR(HIPBLASLT_VERSION_TWEAK);
    state = ok ? 1 : 0;
  }
  return state == 1;
}
constexpr int kGemmRecent = 32;
static thread_local GemmRecent t_recent[kGemmRecent];
static thread_local int t_recent_next = 0;
static bool same_key(const GemmKey& a, const GemmKey& b) {
  return a.m == b.m && a.n == b.n && a.k == b.k && a.ta == b.ta && a.tb == b.tb && a.lda == b.lda && a.ldb == b.ldb && a.ldc == b.ldc && a.dtype == b.dtype &&
         a.dev == b.dev && a.batch == b.batch && a.epilogue == b.epilogue && a.sa == b.sa && a.sb == b.sb && a.sc == b.sc;
}

static bool lt_ok(hipblasStatus_t s, const char* what) {
  if (s == HIPBLAS_STATUS_SUCCESS) return true;
  char buf[128];
  snprintf(buf, sizeof(buf), "hipBLASLt %s failed with status %d", what, (int)s);
  record_error(buf);
  return false;
}

static void destroy_plan(GemmPlan& p) {
  if (p.la) (void)hipblasLtMatrixLayoutDestroy(p.la);
  if (p.lb) (void)hipblasLtMatrixLayoutDestroy(p.lb);
  if (p.lc) (void)hipblasLtMatrixLayoutDestroy(p.lc);
  if (p.desc) (void)hipblasLtMatmulDescDestroy(p.desc);
  p = GemmPlan();
}

// bias != nullptr / act != 0: the dense-layer form C = act(alpha*op(A)*op(B) + bias[i]) (beta must be 0).
struct EpiNone { template <typename T> __device__ __forceinline__ T operator()(T zb, T) const { return zb; } };
// relu of gemm_bias_act_S: z > 0 ? z : 0 -- what hipBLASLt's RELU_BIAS output stage computes and what the reference's device relu computes
// (src/libknet8/ops.jl:63), so that a NaN comes out as 0 whichever route the product takes.
struct EpiRelu { template <typename T> __device__ __forceinline__ T operator()(T zb, T) const { return zb > T(0) ? zb : T(0); } };

enum { kEpiNone = 0, kEpiBias = 1, kEpiReluBias = 2 };
constexpr int kGemmNoFusedForm = 2;   // gemm_lt: the vendor library has no kernel for this problem (with this epilogue); nothing was launched

// One product through hipBLASLt.  epilogue != kEpiNone: bias (length m, added to every column) and optionally relu are applied by the
// product kernel's own output stage, so the m x n result is written once and never read back.
template <typename T>
static int gemm_lt(bool ta, bool tb, int m, int n, int k, T alpha, const T* A, int lda, const T* B, int ldb, T beta, T* C, int ldc, hipStream_t stream,
                   int epilogue, const T* bias, GemmBatch batch) {
  const hipDataType dt = sizeof(T) == 4 ? HIP_R_32F : HIP_R_64F;
  const hipblasComputeType_t ct = sizeof(T) == 4 ? HIPBLAS_COMPUTE_32F : HIPBLAS_COMPUTE_64F;
  int dev = 0;
  (void)hipGetDevice(&dev);
  const GemmKey key = {dev, (int)sizeof(T), ta, tb, m, n, k, lda, ldb, ldc, batch.count, epilogue, batch.sa, batch.sb, batch.sc};
  const bool dry = g_tune[kTuneGemmDryRun] != 0;   // measurements of the library's own share of a call: everything but the vendor call
  const bool capturing = stream_is_capturing(stream);
  if (epilogue == kEpiNone && !capturing) {   // (a product being recorded into a graph takes the full path, which notes that a graph now names the workspace)
    const unsigned long long gen = g_gemm_generation.load(std::memory_order_acquire);
    for (int i = 0; i < kGemmRecent; i++) {
      GemmRecent& r = t_recent[i];
      if (r.generation != gen || r.stream != stream || r.A != A || r.B != B || r.C != C || !same_key(r.key, key)) continue;
      if (dry) return 0;
      const bool same_scalars = r.alpha == (double)alpha && r.beta == (double)beta;
      r.repeats = same_scalars ? r.repeats + 1 : 0;
      r.alpha = (double)alpha; r.beta = (double)beta;
      // (the vendor calls stay under the lock: concurrent calls on one handle from several host threads gave wrong products in the
      //  library's own multi-thread test)
      std::lock_guard<std::mutex> lock(g_gemm_mutex);
      const bool allowed = g_tune[kTuneGemmNoPrepared] == 0 && ext_interface_matches(r.handle);
      if ((!same_scalars || !allowed) && r.prepared) { delete r.prepared; r.prepared = nullptr; }
      if (!r.prepared && !r.no_prepare && r.repeats >= 1 && allowed) {
        if (sizeof(T) == 4) { r.alpha_t.f = (float)alpha; r.beta_t.f = (float)beta; } else { r.alpha_t.d = (double)alpha; r.beta_t.d = (double)beta; }
        auto* g = new hipblaslt_ext::Gemm(r.handle, r.plan->desc, &r.alpha_t, A, r.plan->la, B, r.plan->lb, &r.beta_t, C, r.plan->lc, C, r.plan->lc);
        hipblasLtMatmulAlgo_t algo = r.plan->algo;
        size_t need = 0;
        if (g->isAlgoSupported(algo, need) == HIPBLAS_STATUS_SUCCESS && need <= kGemmWorkspace &&
            g->initialize(algo, r.ws, false, stream) == HIPBLAS_STATUS_SUCCESS) {
          r.prepared = g;
        } else {
          delete g;
          r.no_prepare = true;
        }
      }
      if (r.prepared) return lt_ok(r.prepared->run(stream), "prepared matmul") ? 0 : -1;
      return lt_ok(hipblasLtMatmul(r.handle, r.plan->desc, &alpha, A, r.plan->la, B, r.plan->lb, &beta, C, r.plan->lc, C, r.plan->lc, &r.plan->algo, r.ws,
                                   kGemmWorkspace, stream), "matmul") ? 0 : -1;
    }
  }
  std::lock_guard<std::mutex> lock(g_gemm_mutex);
  hipblasLtHandle_t& h = g_lt[dev];
  if (!h && !lt_ok(hipblasLtCreate(&h), "create")) return -1;
  GemmWs& wsrec = g_gemm_ws[std::make_pair(dev, stream)];
  if (!wsrec.p && !ok(dev_malloc(&wsrec.p, kGemmWorkspace, true), "hipMalloc(gemm workspace)")) return -1;
  if (capturing) wsrec.in_graph = true;
  void* const ws = wsrec.p;
  GemmPlan& p = g_plans[key];
  if (p.unsupported) return kGemmNoFusedForm;
  // A plan whose creation fails half way is taken out of the cache again: the next call must not find a descriptor without layouts.
  auto fail = [&]() { destroy_plan(p); g_plans.erase(key); return -1; };
  if (!p.desc) {
    const hipblasOperation_t opa = ta ? HIPBLAS_OP_T : HIPBLAS_OP_N, opb = tb ? HIPBLAS_OP_T : HIPBLAS_OP_N;
    if (!lt_ok(hipblasLtMatmulDescCreate(&p.desc, ct, dt), "desc create")) return fail();
    if (!lt_ok(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &opa, sizeof(opa)), "set transa")) return fail();
    if (!lt_ok(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &opb, sizeof(opb)), "set transb")) return fail();
    if (epilogue != kEpiNone) {
      const hipblasLtEpilogue_t ep = epilogue == kEpiReluBias ? HIPBLASLT_EPILOGUE_RELU_BIAS : HIPBLASLT_EPILOGUE_BIAS;
      if (hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_EPILOGUE, &ep, sizeof(ep)) != HIPBLAS_STATUS_SUCCESS ||
          hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_BIAS_DATA_TYPE, &dt, sizeof(dt)) != HIPBLAS_STATUS_SUCCESS) {
        destroy_plan(p);
        p.unsupported = true;
        return kGemmNoFusedForm;
      }
    }
    if (!lt_ok(hipblasLtMatrixLayoutCreate(&p.la, dt, ta ? k : m, ta ? m : k, lda), "layout A")) return fail();
    if (!lt_ok(hipblasLtMatrixLayoutCreate(&p.lb, dt, tb ? n : k, tb ? k : n, ldb), "layout B")) return fail();
    if (!lt_ok(hipblasLtMatrixLayoutCreate(&p.lc, dt, m, n, ldc), "layout C")) return fail();
    if (batch.count > 1) {
      const int32_t bc = batch.count;
      const int64_t st[3] = {batch.sa, batch.sb, batch.sc};
      hipblasLtMatrixLayout_t lay[3] = {p.la, p.lb, p.lc};
      for (int q = 0; q < 3; q++) {
        if (!lt_ok(hipblasLtMatrixLayoutSetAttribute(lay[q], HIPBLASLT_MATRIX_LAYOUT_BATCH_COUNT, &bc, sizeof(bc)), "batch count")) return fail();
        if (!lt_ok(hipblasLtMatrixLayoutSetAttribute(lay[q], HIPBLASLT_MATRIX_LAYOUT_STRIDED_BATCH_OFFSET, &st[q], sizeof(st[q])), "batch stride")) return fail();
      }
    }
  }
  if (epilogue != kEpiNone) {   // the bias vector changes from call to call; the descriptor is only used under this lock
    const void* bp = bias;
    if (!lt_ok(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &bp, sizeof(bp)), "set bias pointer")) return fail();
  }
  // Choose the algorithm: at the first call, and again at the first call that is allowed to time the candidates if the earlier
  // choice had to be made without (a stream under capture cannot be synchronised; a call with beta != 0 would accumulate into C).
  const bool can_time = !capturing && beta == T(0);
  if (!p.valid || (!p.timed && can_time)) {
    hipblasLtMatmulPreference_t pref = nullptr;
    if (!lt_ok(hipblasLtMatmulPreferenceCreate(&pref), "pref create")) return fail();
    size_t wsbytes = kGemmWorkspace;
    lt_ok(hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &wsbytes, sizeof(wsbytes)), "pref workspace");
    // Ask for several candidates and time each once on this problem: the first heuristic answer is far from the
    // best for small shapes (the 64x100x784 products of the MNIST MLP ran 5x slower than the best candidate).
    constexpr int kCand = 8;
    hipblasLtMatmulHeuristicResult_t res[kCand];
    int found = 0;
    const hipblasStatus_t hs = hipblasLtMatmulAlgoGetHeuristic(h, p.desc, p.la, p.lb, p.lc, p.lc, pref, kCand, res, &found);
    hipblasLtMatmulPreferenceDestroy(pref);
    if (hs != HIPBLAS_STATUS_SUCCESS && hs != HIPBLAS_STATUS_NOT_SUPPORTED) {   // a failure of the query itself is an error, not "no kernel"
      lt_ok(hs, "algorithm query");
      return fail();
    }
    if (hs == HIPBLAS_STATUS_NOT_SUPPORTED || found < 1) {
      destroy_plan(p);   // not an error: the caller falls back on the library's own product kernels, and remembers it
      p.unsupported = true;
      return kGemmNoFusedForm;
    }
    int best = 0;
    if (found > 1 && can_time) {
      // The timing runs write C exactly as the caller's own call does (beta = 0); the real call below produces its final content.
      hipEvent_t e0 = nullptr, e1 = nullptr;
      if (hipEventCreate(&e0) == hipSuccess && hipEventCreate(&e1) == hipSuccess) {
        float best_ms = 1e30f;
        for (int c = 0; c < found; c++) {
          if (res[c].workspaceSize > kGemmWorkspace) continue;
          float ms = 1e30f;
          bool okc = true;
          for (int rep = 0; rep < 4 && okc; rep++) {  // first run warms the code object, the best of three counts
            (void)hipEventRecord(e0, stream);
            okc = hipblasLtMatmul(h, p.desc, &alpha, A, p.la, B, p.lb, &beta, C, p.lc, C, p.lc, &res[c].algo, ws, kGemmWorkspace, stream) == HIPBLAS_STATUS_SUCCESS;
            (void)hipEventRecord(e1, stream);
            if (hipEventSynchronize(e1) != hipSuccess) okc = false;
            float t = 1e30f;
            if (okc) (void)hipEventElapsedTime(&t, e0, e1);
            if (rep > 0 && t < ms) ms = t;
          }
          if (okc && ms < best_ms) { best_ms = ms; best = c; }
        }
      }
      if (e0) (void)hipEventDestroy(e0);
      if (e1) (void)hipEventDestroy(e1);
      (void)hipGetLastError();
    }
    p.algo = res[best].algo;
    p.workspace = res[best].workspaceSize;
    p.valid = true;
    p.timed = can_time;
  }
  if (epilogue == kEpiNone && p.timed && !capturing) {
    GemmRecent& r = t_recent[t_recent_next];
    t_recent_next = (t_recent_next + 1) % kGemmRecent;
    r.reset();
    r.key = key; r.stream = stream; r.plan = &p; r.handle = h; r.ws = ws;
    r.A = A; r.B = B; r.C = C; r.alpha = (double)alpha; r.beta = (double)beta;
    r.generation = g_gemm_generation.load(std::memory_order_acquire);
  }
  if (dry) return 0;
  return lt_ok(hipblasLtMatmul(h, p.desc, &alpha, A, p.la, B, p.lb, &beta, C, p.lc, C, p.lc, &p.algo, ws, kGemmWorkspace, stream), "matmul") ? 0 : -1;
}

template <typename T>
static int gemm(char transa, char transb, int m, int n, int k, T alpha, const T* A, int lda, const T* B, int ldb, T beta, T* C, int ldc,
                hipStream_t stream, const T* bias = nullptr, int act = 0, GemmBatch batch = GemmBatch()) {
  if (m <= 0 || n <= 0 || batch.count <= 0) return 0;
  const bool ta = (transa == 'T' || transa == 't' || transa == 'C' || transa == 'c');
  const bool tb = (transb == 'T' || transb == 't' || transb == 'C' || transb == 'c');
  if (batch.count > 1 && (bias || act)) { record_error("gemm: the bias/activation form takes no batch"); return -1; }
  // The library's own kernels index their operands with 32 bits; the vendor route (64-bit layouts) has no such limit.
  auto own_kernels_reach = [&]() {
    if ((long long)m * n < (1LL << 31) && (long long)m * k < (1LL << 31) && (long long)k * n < (1LL << 31)) return true;
    record_error("gemm: an operand has 2^31 or more elements; the 32-bit indices of the library's own kernels do not reach that far");
    return false;
  };
  if (batch.count == 1 && (k <= 0 || gemm_is_small(m, n, k))) {   // empty products (C = beta*C [+ bias]), and small ones when a caller has opted in (knet8_tune key 3)
    if (!own_kernels_reach()) return -1;
    launch_gemm_small<T>(stream, ta, tb, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc, bias, act);
    check_launch("gemm (small)");
    return 0;
  }
  // Products the vendor library has no kernel for (seen with some fp64 shapes) run on the library's own tiles, whatever their size.
  auto plain = [&](T bt) {
    int rc = gemm_lt<T>(ta, tb, m, n, k, alpha, A, lda, B, ldb, bt, C, ldc, stream, kEpiNone, nullptr, batch);
    if (rc != kGemmNoFusedForm) return rc;
    if (batch.count > 1) { record_error("hipBLASLt: no algorithm for this batched product"); return -1; }
    if (!own_kernels_reach()) return -1;
    g_gemm_left_vendor.fetch_add(1, std::memory_order_relaxed);
    launch_gemm_small<T>(stream, ta, tb, m, n, k, alpha, A, lda, B, ldb, bt, C, ldc, nullptr, 0);
    check_launch("gemm (own kernel: no vendor algorithm)");
    return 0;
  };
  if (!bias && !act) return plain(beta);
  if (!bias) { record_error("gemm_bias_act: an activation without a bias is not provided"); return -1; }
  int rc = gemm_lt<T>(ta, tb, m, n, k, alpha, A, lda, B, ldb, T(0), C, ldc, stream, act == 1 ? kEpiReluBias : kEpiBias, bias, batch);
  if (rc != kGemmNoFusedForm) return rc;
  // no fused form in the vendor library for this type or shape: the product, then one in-place pass over it
  if (ldc != m) { record_error("gemm_bias_act: ldc must equal m when the vendor library has no fused form for the product"); return -1; }
  rc = plain(T(0));
  if (rc != 0) return rc;
  if (act == 1) launch_bias_act<T, false>(stream, m, n, C, bias, C, EpiRelu());
  else launch_bias_act<T, false>(stream, m, n, C, bias, C, EpiNone());
  check_launch("gemm_bias_act (bias pass)");
  return 0;
}


// Strided batch of products C_b = alpha*op(A_b)*op(B_b) + beta*C_b, b = 0..batch-1, operand b at base + b*stride (elements).
template <typename T>
static int bmm_entry(char transa, char transb, int m, int n, int k, T alpha, const T* A, int lda, long long sa, const T* B, int ldb, long long sb, T beta,
                     T* C, int ldc, long long sc, int batch, hipStream_t stream) {
  if (batch < 0 || sa < 0 || sb < 0 || sc < 0) { record_error("bmm: negative batch count or stride"); return -1; }
  if (batch <= 1 || k <= 0) {   // nothing to batch, or empty products (C = beta*C): the plain entry handles both
    for (int b = 0; b < batch; b++) {
      const int rc = gemm<T>(transa, transb, m, n, k, alpha, A + b * sa, lda, B + b * sb, ldb, beta, C + b * sc, ldc, stream);
      if (rc != 0) return rc;
    }
    return 0;
  }
  GemmBatch gb;
  gb.count = batch; gb.sa = sa; gb.sb = sb; gb.sc = sc;
  return gemm<T>(transa, transb, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc, stream, nullptr, 0, gb);
}

}  // namespace knet8

extern "C" {
KNET8_API int gemm_32_stream(char transa, char transb, int m, int n, int k, float alpha, float* A, int lda, float* B, int ldb, float beta,
                             float* C, int ldc, hipStream_t stream) {
  return knet8::gemm<float>(transa, transb, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc, stream);
}
KNET8_API int gemm_32(char transa, char transb, int m, int n, int k, float alpha, float* A, int lda, float* B, int ldb, float beta, float* C,
                      int ldc) {
  return gemm_32_stream(transa, transb, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc, 0);
}
KNET8_API int gemm_64_stream(char transa, char transb, int m, int n, int k, double alpha, double* A, int lda, double* B, int ldb, double beta,
                             double* C, int ldc, hipStream_t stream) {
  return knet8::gemm<double>(transa, transb, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc, stream);
}
KNET8_API int gemm_64(char transa, char transb, int m, int n, int k, double alpha, double* A, int lda, double* B, int ldb, double beta,
                      double* C, int ldc) {
  return gemm_64_stream(transa, transb, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc, 0);
}

KNET8_API int bmm_32_stream(char transa, char transb, int m, int n, int k, float alpha, float* A, int lda, long long strideA, float* B, int ldb,
                            long long strideB, float beta, float* C, int ldc, long long strideC, int batch, hipStream_t stream) {
  return knet8::bmm_entry<float>(transa, transb, m, n, k, alpha, A, lda, strideA, B, ldb, strideB, beta, C, ldc, strideC, batch, stream);
}
KNET8_API int bmm_32(char transa, char transb, int m, int n, int k, float alpha, float* A, int lda, long long strideA, float* B, int ldb, long long strideB,
                     float beta, float* C, int ldc, long long strideC, int batch) {
  return bmm_32_stream(transa, transb, m, n, k, alpha, A, lda, strideA, B, ldb, strideB, beta, C, ldc, strideC, batch, 0);
}
KNET8_API int bmm_64_stream(char transa, char transb, int m, int n, int k, double alpha, double* A, int lda, long long strideA, double* B, int ldb,
                            long long strideB, double beta, double* C, int ldc, long long strideC, int batch, hipStream_t stream) {
  return knet8::bmm_entry<double>(transa, transb, m, n, k, alpha, A, lda, strideA, B, ldb, strideB, beta, C, ldc, strideC, batch, stream);
}
KNET8_API int bmm_64(char transa, char transb, int m, int n, int k, double alpha, double* A, int lda, long long strideA, double* B, int ldb, long long strideB,
                     double beta, double* C, int ldc, long long strideC, int batch) {
  return bmm_64_stream(transa, transb, m, n, k, alpha, A, lda, strideA, B, ldb, strideB, beta, C, ldc, strideC, batch, 0);
}

static int check_epilogue(int act) {
  if (act == 0 || act == 1) return 0;
  knet8::record_error("gemm_bias_act: act must be 0 (none) or 1 (relu)");
  return -1;
}
KNET8_API int gemm_bias_act_32_stream(char transa, char transb, int m, int n, int k, float alpha, float* A, int lda, float* B, int ldb, float* bias,
                                      int act, float* C, int ldc, hipStream_t stream) {
  if (check_epilogue(act) != 0) return -1;
  return knet8::gemm<float>(transa, transb, m, n, k, alpha, A, lda, B, ldb, 0.0f, C, ldc, stream, bias, act);
}
KNET8_API int gemm_bias_act_32(char transa, char transb, int m, int n, int k, float alpha, float* A, int lda, float* B, int ldb, float* bias, int act,
                               float* C, int ldc) {
  return gemm_bias_act_32_stream(transa, transb, m, n, k, alpha, A, lda, B, ldb, bias, act, C, ldc, 0);
}
KNET8_API int gemm_bias_act_64_stream(char transa, char transb, int m, int n, int k, double alpha, double* A, int lda, double* B, int ldb, double* bias,
                                      int act, double* C, int ldc, hipStream_t stream) {
  if (check_epilogue(act) != 0) return -1;
  return knet8::gemm<double>(transa, transb, m, n, k, alpha, A, lda, B, ldb, 0.0, C, ldc, stream, bias, act);
}
KNET8_API int gemm_bias_act_64(char transa, char transb, int m, int n, int k, double alpha, double* A, int lda, double* B, int ldb, double* bias, int act,
                               double* C, int ldc) {
  return gemm_bias_act_64_stream(transa, transb, m, n, k, alpha, A, lda, B, ldb, bias, act, C, ldc, 0);
}
}
