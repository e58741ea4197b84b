// See runtime.h.
#include "runtime.h"

#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <map>
#include <mutex>

namespace mobula_hip {

CallState& call_state() {
  static thread_local CallState state;
  return state;
}

void set_error(const char* fmt, ...) {
  CallState& st = call_state();
  if (!st.error.empty()) return;  // keep the first error of a call
  char buf[1024];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  st.error = buf;
}

long long arg_extent(int index) {
  const auto& e = call_state().extents;
  return (index >= 0 && index < static_cast<int>(e.size())) ? e[index] : -1;
}

namespace {
// One scratch buffer per calling thread and device: calls of different threads
// never share one.  Calls of one thread are ordered by their stream; when a
// thread moves to another stream while the buffer may still be in use on the
// previous one (asynchronous calls), the new stream waits for `idle`.
struct Scratch {
  void* ptr = nullptr;
  size_t bytes = 0;
  hipStream_t last = nullptr;   // stream of the last call that used the buffer
  hipEvent_t idle = nullptr;    // recorded on `last` when a call on another stream has to wait for it
  bool busy = false;            // work on `last` may still use the buffer
  bool pinned = false;          // a call was recorded into a HIP graph while using the buffer:
                                // replays use this very address, so it is neither freed nor moved
};
struct ScratchOfThread {
  std::map<int, Scratch> per_device;
  ~ScratchOfThread() {
    for (auto& it : per_device) {
      if (it.second.ptr != nullptr) (void)hipFree(it.second.ptr);
      if (it.second.idle != nullptr) (void)hipEventDestroy(it.second.idle);
    }
  }
};
Scratch* scratch_of_current_device() {
  static thread_local ScratchOfThread mine;
  int device = 0;
  MOBULA_HIP_TRY(hipGetDevice(&device));
  return failed() ? nullptr : &mine.per_device[device];
}
std::mutex g_mutex;
std::map<std::string, long long> g_options;
}  // namespace

void* workspace(size_t bytes) {
  Scratch* const s = scratch_of_current_device();
  if (s == nullptr) return nullptr;
  CallState& st = call_state();
  auto is_capturing = [](hipStream_t stream) {
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    if (stream == nullptr) return false;
    if (hipStreamIsCapturing(stream, &status) != hipSuccess) {
      (void)hipGetLastError();
      return false;
    }
    return status == hipStreamCaptureStatusActive;
  };
  const bool capturing = is_capturing(st.stream);
  if (s->busy && s->last != st.stream) {
    // The previous call went to another stream and did not wait: this stream waits for what that
    // one holds now (an event is only recorded here, when the stream changes; an event behind
    // every call costs each call boundary some ten microseconds).  The handle of that stream is
    // used here: a caller that makes asynchronous calls keeps a stream alive until the next call
    // of the same thread on the device has returned.  A call that was recorded into a graph (or
    // a stream that is being recorded now) is left to the owner of the graph to order: an
    // event there would become part of the recording.
    if (!s->pinned && !is_capturing(s->last)) {
      if (s->idle == nullptr && hipEventCreateWithFlags(&s->idle, hipEventDisableTiming) != hipSuccess)
        s->idle = nullptr;
      if (s->idle == nullptr || hipEventRecord(s->idle, s->last) != hipSuccess ||
          hipStreamWaitEvent(st.stream, s->idle, 0) != hipSuccess) {
        (void)hipGetLastError();
        if (capturing) {   // (a device-wide wait would break the recording)
          set_error("the previous call of this thread ran on another stream and cannot be waited for while "
                    "this stream is being captured: synchronise that stream before recording");
          return nullptr;
        }
        MOBULA_HIP_TRY(hipDeviceSynchronize());
      }
      if (failed()) return nullptr;
    }
    s->busy = false;   // ordered behind it from here on (finish_call marks the new call)
  }
  if (s->bytes < bytes && (capturing || s->pinned)) {
    set_error("the workspace of this thread (%zu bytes) is too small for the call (%zu bytes) and cannot be "
              "replaced %s: make one ordinary call of the largest shape before recording, or call "
              "mobula_hip_unpin_workspace() once the graphs are gone", s->bytes, bytes,
              capturing ? "while the stream is being captured" : "because a recorded graph uses it");
    return nullptr;
  }
  if (capturing) s->pinned = true;
  if (s->bytes < bytes) {
    if (s->ptr != nullptr) MOBULA_HIP_TRY(hipFree(s->ptr));  // waits for pending work
    s->ptr = nullptr;
    s->bytes = 0;
    size_t want = bytes + bytes / 4 + (1u << 20);
    MOBULA_HIP_TRY(hipMalloc(&s->ptr, want));
    if (failed()) { s->ptr = nullptr; return nullptr; }
    s->bytes = want;
  }
  s->last = st.stream;
  st.used_workspace = true;
  return s->ptr;
}

// Frees the calling thread's scratch buffer on the current device (hipFree waits
// for the work that still uses it); returns the bytes given back.
long long release_workspace() {
  Scratch* const s = scratch_of_current_device();
  if (s == nullptr || s->ptr == nullptr) return 0;
  if (s->pinned) {
    set_error("the workspace of this thread is used by a recorded graph: call mobula_hip_unpin_workspace() "
              "once the graph is gone");
    return 0;
  }
  const long long bytes = static_cast<long long>(s->bytes);
  MOBULA_HIP_TRY(hipFree(s->ptr));
  s->ptr = nullptr;
  s->bytes = 0;
  s->busy = false;
  s->last = nullptr;
  return failed() ? 0 : bytes;
}

void unpin_workspace() {
  Scratch* const s = scratch_of_current_device();
  if (s != nullptr) s->pinned = false;
}

long long workspace_bytes() {
  Scratch* const s = scratch_of_current_device();
  return s == nullptr ? 0 : static_cast<long long>(s->bytes);
}

long long option(const char* name, long long fallback) {
  std::lock_guard<std::mutex> lock(g_mutex);
  auto it = g_options.find(name);
  return it == g_options.end() ? fallback : it->second;
}

DeviceScope::DeviceScope(int device) {
  if (device < 0) return;
  MOBULA_HIP_TRY(hipGetDevice(&previous_));
  if (failed()) { ok_ = false; return; }
  if (previous_ != device) {
    MOBULA_HIP_TRY(hipSetDevice(device));
    if (failed()) { ok_ = false; return; }
    changed_ = true;
  }
}

DeviceScope::~DeviceScope() {
  if (changed_) (void)hipSetDevice(previous_);
}

HostStaging::~HostStaging() {
  for (auto& it : items_) (void)hipFree(it.dev);
}

void* HostStaging::in(const void* host, size_t bytes, bool upload) {
  void* dev = inout(const_cast<void*>(host), bytes, upload);
  items_.back().download = false;
  return dev;
}

void* HostStaging::inout(void* host, size_t bytes, bool upload) {
  Item item{nullptr, host, bytes, true};
  MOBULA_HIP_TRY(hipMalloc(&item.dev, bytes > 0 ? bytes : 1));
  if (!failed() && upload && bytes > 0)
    MOBULA_HIP_TRY(hipMemcpy(item.dev, host, bytes, hipMemcpyHostToDevice));
  items_.push_back(item);
  return item.dev;
}

bool HostStaging::flush(hipStream_t stream) {
  MOBULA_HIP_TRY(hipStreamSynchronize(stream));
  for (auto& it : items_) {
    if (failed()) break;
    if (it.download && it.bytes > 0)
      MOBULA_HIP_TRY(hipMemcpy(it.host, it.dev, it.bytes, hipMemcpyDeviceToHost));
  }
  return !failed();
}

namespace {
struct SideState { hipStream_t stream = nullptr; hipEvent_t fork = nullptr, join = nullptr; bool tried = false; };
SideState& side_state(int device) {
  static thread_local std::map<int, SideState> states;
  return states[device];
}
}  // namespace

namespace {
std::string& export_list() {
  static std::string names = "set_device";
  return names;
}
}  // namespace

ExportRegistrar::ExportRegistrar(const char* names) {
  export_list() += " ";
  export_list() += names;
}

SideStream::SideStream(hipStream_t main, bool wanted) : main_(main), side_(main) {
  if (!wanted || option("side_stream", 1) == 0) return;
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) return;
  SideState& st = side_state(device);
  if (!st.tried) {
    st.tried = true;
    if (hipStreamCreateWithFlags(&st.stream, hipStreamNonBlocking) != hipSuccess ||
        hipEventCreateWithFlags(&st.fork, hipEventDisableTiming) != hipSuccess ||
        hipEventCreateWithFlags(&st.join, hipEventDisableTiming) != hipSuccess) {
      st.stream = nullptr;
      (void)hipGetLastError();
    }
  }
  if (st.stream == nullptr) return;
  if (hipEventRecord(st.fork, main_) != hipSuccess || hipStreamWaitEvent(st.stream, st.fork, 0) != hipSuccess) {
    (void)hipGetLastError();
    return;
  }
  side_ = st.stream;
  joined_ = st.join;
}

SideStream::~SideStream() {
  // a path that left early: the caller's stream still has to wait for the helpers
  if (side_ != main_ && (hipEventRecord(joined_, side_) != hipSuccess ||
                         hipStreamWaitEvent(main_, joined_, 0) != hipSuccess))
    (void)hipGetLastError();
}

void SideStream::join() {
  if (side_ == main_) return;
  MOBULA_HIP_TRY(hipEventRecord(joined_, side_));
  MOBULA_HIP_TRY(hipStreamWaitEvent(main_, joined_, 0));
  side_ = main_;
}

namespace {
struct TimerState {
  hipEvent_t start = nullptr, stop = nullptr;
  const char* name = "";
  bool pending = false;
};
TimerState& timer_state() {
  static thread_local TimerState t;
  return t;
}
}  // namespace

KernelTimer::KernelTimer(const char* name, hipStream_t stream, bool wanted)
    : stream_(stream), on_(wanted && option("kernel_timing", 0) != 0) {
  if (!on_) return;
  TimerState& t = timer_state();
  if (t.start == nullptr) {
    if (hipEventCreate(&t.start) != hipSuccess || hipEventCreate(&t.stop) != hipSuccess) {
      t.start = t.stop = nullptr;
      on_ = false;
      return;
    }
  }
  t.name = name;
  t.pending = false;
  if (hipEventRecord(t.start, stream_) != hipSuccess) on_ = false;
}

KernelTimer::~KernelTimer() {
  if (!on_) return;
  TimerState& t = timer_state();
  t.pending = hipEventRecord(t.stop, stream_) == hipSuccess;
}

void begin_call() { call_state().error.clear(); }

void finish_call() {
  CallState& st = call_state();
  if (st.synchronous && !failed()) MOBULA_HIP_TRY(hipStreamSynchronize(st.stream));
  if (st.used_workspace) {
    st.used_workspace = false;
    Scratch* const s = scratch_of_current_device();
    if (s != nullptr) s->busy = !st.synchronous;   // the buffer stays in use until the stream gets here
  }
  st.extents.clear();
}

}  // namespace mobula_hip

using mobula_hip::call_state;

extern "C" {

void mobula_hip_set_stream(void* stream, int synchronous) {
  auto& st = call_state();
  st.stream = static_cast<hipStream_t>(stream);
  st.synchronous = synchronous != 0;
}

void mobula_hip_set_arg_extents(const long long* numel, int n) {
  auto& st = call_state();
  st.extents.assign(numel, numel + (n > 0 ? n : 0));
}

const char* mobula_hip_last_error(void) {
  auto& st = call_state();
  return st.error.empty() ? nullptr : st.error.c_str();
}

void mobula_hip_clear_error(void) { call_state().error.clear(); }

int mobula_hip_set_option(const char* name, long long value) {
  static const char* known[] = {"roialign_impl", "host_staging_device", "kernel_timing", "side_stream",
                                "conv_compute", "roialign_tile_columns", "roialign_row_split", "roialign_row_quads", nullptr};
  for (int i = 0; known[i] != nullptr; ++i) {
    if (std::strcmp(known[i], name) == 0) {
      std::lock_guard<std::mutex> lock(mobula_hip::g_mutex);
      mobula_hip::g_options[name] = value;
      return 0;
    }
  }
  return -1;
}

long long mobula_hip_get_option(const char* name) { return mobula_hip::option(name, -1); }

const char* mobula_hip_exports(void) { return mobula_hip::export_list().c_str(); }

double mobula_hip_last_kernel_ms(const char** name) {
  mobula_hip::TimerState& t = mobula_hip::timer_state();
  if (name != nullptr) *name = t.name;
  if (!t.pending) return -1.0;
  float ms = 0.0f;
  if (hipEventSynchronize(t.stop) != hipSuccess || hipEventElapsedTime(&ms, t.start, t.stop) != hipSuccess)
    return -1.0;
  return ms;
}

long long mobula_hip_workspace_bytes(void) { return mobula_hip::workspace_bytes(); }
long long mobula_hip_release_workspace(void) {
  mobula_hip::begin_call();
  return mobula_hip::release_workspace();
}
// The calling thread's workspace on the current device is no longer used by any recorded graph.
void mobula_hip_unpin_workspace(void) { mobula_hip::unpin_workspace(); }

// 1 if a kernel may dereference p: device memory, or host memory the device
// reaches (pinned, managed); 0 for ordinary host memory and for null.
int mobula_hip_device_can_read(const void* p) {
  if (p == nullptr) return 0;
  hipPointerAttribute_t attr;
  if (hipPointerGetAttributes(&attr, p) != hipSuccess) {
    (void)hipGetLastError();
    return 0;
  }
  return attr.type == hipMemoryTypeDevice || attr.type == hipMemoryTypeHost ||
                 attr.type == hipMemoryTypeManaged
             ? 1
             : 0;
}

int mobula_hip_device_count(void) {
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess) return 0;
  return n;
}

// Reference: mobula/cpp/src/context.cpp:9-15.
void set_device(const int device_id) {
  int current = -1;
  MOBULA_HIP_TRY(hipGetDevice(&current));
  if (current != device_id) MOBULA_HIP_TRY(hipSetDevice(device_id));
}
}
