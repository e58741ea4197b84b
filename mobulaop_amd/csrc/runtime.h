// Launcher runtime shared by every operator in the library: per-thread call
// state (stream, argument extents, error text), scratch memory per thread and
// device, and staging of host buffers through device memory.
//
// Replaces the reference's HIP "context" (mobula/cpp/include/context/hip_ctx.h:
// 36-106): that one creates, synchronises and destroys a stream around every
// launch and terminates the process on a HIP error; this one launches on a
// caller-chosen stream, synchronises only when asked to, and records errors
// for the caller to pick up.
#pragma once
#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>
#include <string>
#include <vector>

namespace mobula_hip {

struct CallState {
  hipStream_t stream = nullptr;
  bool synchronous = true;          // wait for completion before returning
  std::vector<long long> extents;   // element count per argument, -1 = unknown
  std::string error;                // empty = no error
  bool used_workspace = false;      // the call took the scratch buffer (see workspace())
};

CallState& call_state();

void set_error(const char* fmt, ...) __attribute__((format(printf, 1, 2)));
inline bool failed() { return !call_state().error.empty(); }

// Element count the caller declared for argument `index` (0-based, device id
// not counted); -1 if it declared none.  Consumed extents are cleared by
// finish_call().
long long arg_extent(int index);

// Grow-only scratch buffer of the calling thread on the current device, for
// work on the call's stream.  The pointer stays valid until a later call of the
// thread asks for more bytes on the same device.  A thread that changes streams
// between asynchronous calls is ordered behind its previous call; every entry
// point ends with finish_call(), which keeps the book for that.
void* workspace(size_t bytes);
long long release_workspace();   // frees the calling thread's buffer on the current device
// A call recorded into a HIP graph pins the buffer (replays use its address): it is then
// neither grown nor released (an error instead) until unpin_workspace().
void unpin_workspace();
long long workspace_bytes();

long long option(const char* name, long long fallback);

// Makes `device` current for the lifetime of the object (no-op for -1).
class DeviceScope {
 public:
  explicit DeviceScope(int device);
  ~DeviceScope();
  bool ok() const { return ok_; }

 private:
  int previous_ = -1;
  bool changed_ = false;
  bool ok_ = true;
};

// Device mirrors of host buffers for calls that arrive with device id -1.
class HostStaging {
 public:
  ~HostStaging();
  // Device copy of `bytes` bytes at `host` (uploaded when `upload`).
  void* in(const void* host, size_t bytes, bool upload = true);
  // Device buffer that is downloaded to `host` by flush().
  void* inout(void* host, size_t bytes, bool upload);
  bool flush(hipStream_t stream);  // download outputs, wait for completion

 private:
  struct Item { void* dev; void* host; size_t bytes; bool download; };
  std::vector<Item> items_;
};

// Every entry point starts a call with begin_call() -- the error text of the
// thread's previous call is dropped, so an error is reported for the call that
// caused it and never makes a later one return early -- and ends it with
// finish_call(), which synchronises if the call is synchronous and clears the
// per-call extents.
void begin_call();
void finish_call();
struct CallBegin { CallBegin() { begin_call(); } };   // begin_call() as a first member / first local

// A second stream of the current device on which independent helper kernels of
// a call run beside the work on the caller's stream:
//   SideStream side(stream);   work launched on side.get() starts after what
//                              `stream` holds so far
//   side.join();               `stream` waits for what the side stream holds
// Both streams have the default priority.  With the option "side_stream" set to
// 0 (or if the stream cannot be created) get() is the caller's stream itself.
class SideStream {
 public:
  explicit SideStream(hipStream_t main, bool wanted = true);   // !wanted: get() is `main`
  ~SideStream();                       // joins if join() was not reached
  SideStream(const SideStream&) = delete;
  SideStream& operator=(const SideStream&) = delete;
  hipStream_t get() const { return side_; }
  void join();

 private:
  hipStream_t main_, side_;
  hipEvent_t joined_ = nullptr;
};

// Every operator source adds the names of its entry points to the list that
// mobula_hip_exports() returns:  static ExportRegistrar r("name_a name_b");
struct ExportRegistrar {
  explicit ExportRegistrar(const char* names);
};

// With the option "kernel_timing" set, brackets the launches issued during its
// lifetime with HIP events on `stream`; mobula_hip_last_kernel_ms() then
// reports the elapsed time of the calling thread's last bracket.
class KernelTimer {
 public:
  KernelTimer(const char* name, hipStream_t stream, bool wanted = true);   // !wanted: no bracket
  ~KernelTimer();

 private:
  hipStream_t stream_;
  bool on_;
};

}  // namespace mobula_hip

#define MOBULA_HIP_TRY(expr)                                                        \
  do {                                                                              \
    hipError_t mobula_hip_status_ = (expr);                                         \
    if (mobula_hip_status_ != hipSuccess) {                                         \
      ::mobula_hip::set_error("%s failed: %s (%s:%d)", #expr,                       \
                              hipGetErrorString(mobula_hip_status_), __FILE__, __LINE__); \
    }                                                                               \
  } while (0)

// Launcher functions are ordinary host functions; the macro only marks them
// for the Python-side declaration scanner.  (Sources in the kernel dialect,
// compiled on load, define the macros themselves before this header is seen.)
#ifndef MOBULA_KERNEL
#define MOBULA_KERNEL void
#define MOBULA_FUNC
#endif
