// Host-side services shared by the generated entry points: error recording, per-stream reduction
// scratch, launch-heuristic knobs.  Implemented in knet8_runtime.hip.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>

#ifndef KNET8_API
#define KNET8_API __attribute__((visibility("default")))
#endif

namespace knet8 {

// The entry points return void like the reference's (errors there are unchecked, src/libknet8/LibKnet8.jl:54);
// failures are kept as text for knet8_last_error() instead of being dropped.
void record_error(const char* what);
void check_launch(const char* name);  // records hipGetLastError() if a launch failed

// Scratch that split reductions need beyond their inputs and outputs: `partial` holds the per-workgroup
// partial results, `counters` the per-output-group tickets (all zero between launches; the kernel that
// uses them resets them).  One Workspace per stream, so launches on different streams never share it;
// launches on one stream are ordered and may.
struct Workspace {
  void* partial;
  unsigned* counters;
};
Workspace workspace_for(hipStream_t stream, size_t partial_bytes, size_t ncounters);
// Where a split launch takes its scratch from: the per-stream buffers above (a null source) or a caller-supplied provider.  A provider
// that cannot serve the request records why and returns null pointers.
struct ScratchSource {
  Workspace (*get)(void* ctx, hipStream_t stream, size_t partial_bytes, size_t ncounters);
  void* ctx;
  size_t partial_capacity, counter_capacity;   // what the provider can serve at most (0: it grows as needed); launch planners that have a choice stay within it
};
inline bool scratch_fits(const ScratchSource* src, size_t partial_bytes, size_t ncounters) {
  return src == nullptr || ((src->partial_capacity == 0 || partial_bytes <= src->partial_capacity) &&
                            (src->counter_capacity == 0 || ncounters <= src->counter_capacity));
}
// Tickets of different output groups sit 256 bytes apart: atomics on one 64-byte line are carried out one after the other (11-12 ns each on MI355X,
// measured: 256 workgroups drawing from 16 counters 4 bytes apart take 1.9 us longer than from counters 256 bytes apart).
constexpr int kTicketStride = 64;   // in counters

inline Workspace take_scratch(const ScratchSource* src, hipStream_t stream, size_t partial_bytes, size_t ncounters) {
  return src ? src->get(src->ctx, stream, partial_bytes, ncounters) : workspace_for(stream, partial_bytes, ncounters);
}
// A launch split over several workgroups stores partial results and draws tickets through these pointers: without them it must not be
// issued at all (out of device memory is an error to report, src/knetarrays/kptr.jl:114-141, not a fault on the device).
inline bool scratch_ready(const Workspace& ws, const char* who) {
  if (ws.partial != nullptr && ws.counters != nullptr) return true;
  record_error(who);   // the allocation's own failure, recorded first, is the message that is kept
  return false;
}
// Device slot for the result of a `_20` reduction on this stream, and the blocking copy that fetches it.
void* scalar_slot(hipStream_t stream);
void fetch_scalar(hipStream_t stream, const void* dev, void* host, size_t nbytes);

// State of the default random stream (knet8_seed): hands out `blocks` consecutive generator counters under the current seed.
void rng_take(unsigned long long blocks, unsigned long long* seed, unsigned long long* offset);

enum { kTuneNumCUs = 0, kTuneSoftmaxResidentRows = 1, kTuneGemmSmallMflop = 3, kTuneDenseBackMflop = 4, kTuneFailScratch = 5, kTuneSoftmaxNoLdsSlots = 6, kTuneGemmDryRun = 7, kTuneGemmNoPrepared = 8, kTuneCount = 9 };
int tuning(int key);

#ifdef KNET8_TIMELINE
struct TlStamp;
TlStamp* timeline_buffer();   // measurement build: where the stamped kernels write (null: nowhere), set by knet8_timeline_set
#endif

}  // namespace knet8
