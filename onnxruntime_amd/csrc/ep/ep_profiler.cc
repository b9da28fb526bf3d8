// OrtEpProfilerImpl of the MI355X plugin EP (include/onnxruntime/core/session/onnxruntime_ep_c_api.h:449-631,
// OrtEp::CreateProfiler :2460-2482; how ONNX Runtime drives it: onnxruntime/core/session/plugin_ep/ep_event_profiling.cc).
//
// ONNX Runtime brackets every profiled event of its own (session initialisation, the execution of one node) with
// StartEvent / StopEvent on the thread that runs it.  The profiler keeps those brackets on a per-thread stack; while
// a thread is inside one, every kernel of this provider times what it enqueues with a pair of hipEvents on its
// compute stream (KernelTimer) and files the pair under the bracket's correlation id.  EndProfiling waits for the
// events, converts the device times to ONNX Runtime's timeline
//   timestamp_us = (ep_profiling_start_offset_ns + (event_time - start_time)) / 1000
// with both times read from the same device clock (an origin event recorded in StartProfiling), and reports one
// KERNEL event per launch group.  Outside a bracket KernelTimer does nothing, so unprofiled runs pay one
// thread-local read per kernel call.
#include <unistd.h>

#include <atomic>
#include <functional>
#include <thread>

#include "ep_kernel_util.h"

namespace mi355x_ep {

namespace {

struct Launch {
  std::string name;      // what ran on the device, e.g. mnb_skinny_kernel
  std::string op;        // operator the kernel belongs to
  std::string shape;     // "M x N x K"
  uint64_t correlation;  // ORT event the launch happened under
  int64_t thread;
  hipEvent_t start, stop;
};

struct Profiler : OrtEpProfilerImpl {
  Apis apis;
  std::mutex mutex;
  std::vector<Launch> launches;
  int64_t start_offset_ns = 0;
  hipEvent_t origin = nullptr;
  std::atomic<bool> started{false};
};

struct Bracket {
  Profiler* profiler;
  uint64_t correlation;
};

// ORT events open on the calling thread, innermost last
thread_local std::vector<Bracket> tl_brackets;

Profiler* Self(OrtEpProfilerImpl* p) { return static_cast<Profiler*>(p); }

void DestroyLaunches(std::vector<Launch>& launches) {
  for (Launch& l : launches) {
    (void)hipEventDestroy(l.start);
    (void)hipEventDestroy(l.stop);
  }
  launches.clear();
}

void ORT_API_CALL ReleaseImpl(OrtEpProfilerImpl* this_ptr) noexcept {
  Profiler* p = Self(this_ptr);
  DestroyLaunches(p->launches);
  if (p->origin != nullptr) (void)hipEventDestroy(p->origin);
  delete p;
}

OrtStatus* ORT_API_CALL StartProfilingImpl(OrtEpProfilerImpl* this_ptr, int64_t ep_profiling_start_offset_ns) noexcept {
  Profiler& p = *Self(this_ptr);
  std::lock_guard<std::mutex> lock(p.mutex);
  DestroyLaunches(p.launches);
  p.start_offset_ns = ep_profiling_start_offset_ns;
  if (p.origin == nullptr) MI_RETURN_IF_HIP(p.apis, hipEventCreate(&p.origin));
  // the device clock's reading of "now": every later launch is timed against this event
  MI_RETURN_IF_HIP(p.apis, hipEventRecord(p.origin, nullptr));
  MI_RETURN_IF_HIP(p.apis, hipEventSynchronize(p.origin));
  p.started = true;
  return nullptr;
}

OrtStatus* ORT_API_CALL StartEventImpl(OrtEpProfilerImpl* this_ptr, uint64_t ort_event_correlation_id) noexcept {
  tl_brackets.push_back({Self(this_ptr), ort_event_correlation_id});
  return nullptr;
}

OrtStatus* ORT_API_CALL StopEventImpl(OrtEpProfilerImpl* this_ptr, uint64_t ort_event_correlation_id,
                                      const OrtProfilingEvent* /*ort_event*/) noexcept {
  // brackets nest, but be lenient about a Stop without its Start: remove the innermost match only
  for (size_t i = tl_brackets.size(); i-- > 0;) {
    if (tl_brackets[i].profiler == Self(this_ptr) && tl_brackets[i].correlation == ort_event_correlation_id) {
      tl_brackets.erase(tl_brackets.begin() + static_cast<std::ptrdiff_t>(i));
      break;
    }
  }
  return nullptr;
}

OrtStatus* ORT_API_CALL EndProfilingImpl(OrtEpProfilerImpl* this_ptr, OrtProfilingEventsContainer* container) noexcept {
  Profiler& p = *Self(this_ptr);
  const Apis& a = p.apis;
  std::vector<Launch> launches;
  {
    std::lock_guard<std::mutex> lock(p.mutex);
    launches.swap(p.launches);
    p.started = false;
  }
  OrtStatus* result = nullptr;
  const int32_t pid = static_cast<int32_t>(getpid());
  for (const Launch& l : launches) {
    if (result != nullptr) break;
    float since_origin_ms = 0.f, duration_ms = 0.f;
    hipError_t e = hipEventSynchronize(l.stop);
    if (e == hipSuccess) e = hipEventElapsedTime(&since_origin_ms, p.origin, l.start);
    if (e == hipSuccess) e = hipEventElapsedTime(&duration_ms, l.start, l.stop);
    if (e != hipSuccess) {
      (void)hipGetLastError();
      continue;  // a launch whose events cannot be read is left out; the others are still reported
    }
    const int64_t timestamp_us =
        (p.start_offset_ns + static_cast<int64_t>(static_cast<double>(since_origin_ms) * 1e6)) / 1000;
    const int64_t duration_us = static_cast<int64_t>(static_cast<double>(duration_ms) * 1e3 + 0.5);
    const std::string correlation = std::to_string(l.correlation);
    const char* keys[3] = {"op_name", "shape", "ort_event_correlation_id"};
    const char* values[3] = {l.op.c_str(), l.shape.c_str(), correlation.c_str()};
    OrtProfilingEvent* event = nullptr;
    result = a.ep->CreateProfilingEvent(OrtProfilingEventCategory_KERNEL, pid, static_cast<int32_t>(l.thread),
                                        l.name.c_str(), timestamp_us, duration_us, keys, values, 3, &event);
    if (result != nullptr) break;
    const OrtProfilingEvent* events[1] = {event};
    result = a.ep->ProfilingEventsContainer_AddEvents(container, events, 1);
    a.ep->ReleaseProfilingEvent(event);
  }
  DestroyLaunches(launches);
  return result;
}

}  // namespace

OrtStatus* CreateEpProfiler(const Apis& a, OrtEpProfilerImpl** out) {
  *out = nullptr;
  Profiler* p = new (std::nothrow) Profiler{};
  if (p == nullptr) return a.ort->CreateStatus(ORT_FAIL, "out of memory creating the profiler");
  p->ort_version_supported = ORT_API_VERSION;
  p->Release = ReleaseImpl;
  p->StartProfiling = StartProfilingImpl;
  p->StartEvent = StartEventImpl;
  p->StopEvent = StopEventImpl;
  p->EndProfiling = EndProfilingImpl;
  p->apis = a;
  *out = p;
  return nullptr;
}

KernelTimer::KernelTimer(hipStream_t stream, const char* op, const char* kernel_name, int64_t M, int64_t N, int64_t K)
    : stream_(stream) {
  if (tl_brackets.empty()) return;
  const Bracket& bracket = tl_brackets.back();
  Profiler& p = *bracket.profiler;
  if (!p.started) return;
  Launch l;
  if (hipEventCreate(&l.start) != hipSuccess) return;
  if (hipEventCreate(&l.stop) != hipSuccess) {
    (void)hipEventDestroy(l.start);
    return;
  }
  if (hipEventRecord(l.start, stream) != hipSuccess) {
    (void)hipEventDestroy(l.start);
    (void)hipEventDestroy(l.stop);
    return;
  }
  l.name = kernel_name != nullptr ? kernel_name : op;
  l.op = op;
  l.shape = std::to_string(M) + " x " + std::to_string(N) + " x " + std::to_string(K);
  l.correlation = bracket.correlation;
  l.thread = static_cast<int64_t>(std::hash<std::thread::id>{}(std::this_thread::get_id()) & 0x7fffffff);
  hipEvent_t start = l.start, stop = l.stop;
  pending_ = new (std::nothrow) Launch(std::move(l));
  if (pending_ == nullptr) {
    (void)hipEventDestroy(start);
    (void)hipEventDestroy(stop);
    return;
  }
  profiler_ = &p;
}

KernelTimer::~KernelTimer() {
  if (pending_ == nullptr) return;
  Launch* l = static_cast<Launch*>(pending_);
  Profiler& p = *static_cast<Profiler*>(profiler_);
  if (hipEventRecord(l->stop, stream_) == hipSuccess) {
    std::lock_guard<std::mutex> lock(p.mutex);
    p.launches.push_back(std::move(*l));
  } else {
    (void)hipEventDestroy(l->start);
    (void)hipEventDestroy(l->stop);
  }
  delete l;
}

}  // namespace mi355x_ep
