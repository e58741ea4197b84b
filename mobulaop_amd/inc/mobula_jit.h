// Launch glue for operator sources compiled at load time (one small shared
// object per function instantiation, see mobulaop_amd/op/jit.py).  A generated
// entry point
//     extern "C" void axpy_<hash>(const int device_id, const int n, ...)
// creates a KernelCall, maps its pointer arguments (device pointers pass
// through; host pointers, device id -1, are mirrored on the staging device using
// the element counts the binding declared for the call) and launches the
// kernel on the calling thread's stream.  Errors are recorded for the binding
// to raise; nothing terminates the process.
#pragma once
#include <algorithm>
#include <type_traits>

#include "runtime.h"

namespace mobula_jit {

class KernelCall {
 public:
  KernelCall(const char* name, int device_id)
      : name_(name), host_(device_id < 0),
        scope_(device_id < 0 ? static_cast<int>(mobula_hip::option("host_staging_device", 0)) : device_id) {
    auto& st = mobula_hip::call_state();
    saved_stream_ = st.stream;
    if (host_) st.stream = nullptr;   // the caller's stream belongs to another device, if to any
  }
  ~KernelCall() {
    auto& st = mobula_hip::call_state();
    if (host_) {
      if (!mobula_hip::failed()) stage_.flush(nullptr);
      st.stream = saved_stream_;
      st.extents.clear();
    } else {
      if (copies_ && !mobula_hip::failed()) stage_.flush(st.stream);   // structures come back
      mobula_hip::finish_call();
    }
  }
  bool ok() const { return scope_.ok() && !mobula_hip::failed(); }

  // Pointer argument number `index` (0-based, device id not counted) of
  // elem_bytes-sized elements; writable ones are copied back for host callers.
  template <typename T>
  T* arg(T* p, int index, bool writable) {
    if (!host_ || p == nullptr) return p;
    const long long count = mobula_hip::arg_extent(index);
    if (count < 0) {
      mobula_hip::set_error("%s: host memory needs the element count of argument %d", name_, index);
      return p;
    }
    typedef typename std::remove_const<T>::type M;
    const size_t bytes = sizeof(T) * static_cast<size_t>(count);
    void* dev = writable ? stage_.inout(const_cast<M*>(p), bytes, /*upload=*/true)
                         : stage_.in(p, bytes);
    return static_cast<T*>(dev);
  }

  // A structure the caller passes by address (host memory, whatever the device
  // id): the kernel gets a copy in device memory, and the caller's structure is
  // updated from it afterwards.  Pointers inside it are used as they are.
  template <typename T>
  T* struct_arg(T* p) {
    if (p == nullptr || !ok()) return p;
    typedef typename std::remove_const<T>::type M;
    copies_ = true;
    return static_cast<T*>(stage_.inout(const_cast<M*>(p), sizeof(T), /*upload=*/true));
  }

  // kernel<<<one workgroup of 1024 threads>>>(args...): for kernels whose threads
  // synchronise with each other (Reduce, __syncthreads).
  template <typename Kernel, typename... Args>
  void launch_together(long long n, Kernel kernel, Args... args) {
    if (!ok() || n <= 0) return;
    hipLaunchKernelGGL(kernel, dim3(1), dim3(1024), 0, mobula_hip::call_state().stream, args...);
    const hipError_t status = hipGetLastError();
    if (status != hipSuccess) mobula_hip::set_error("%s: launch failed: %s", name_, hipGetErrorString(status));
  }

  // kernel<<<blocks of 256 threads for n iterations>>>(args...) on the call's stream.
  template <typename Kernel, typename... Args>
  void launch(long long n, Kernel kernel, Args... args) {
    if (!ok() || n <= 0) return;
    int cus = 0, device = 0;
    if (hipGetDevice(&device) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || cus <= 0) {
      (void)hipGetLastError();
      cus = 256;
    }
    const long long blocks = std::min<long long>((n + 255) / 256, static_cast<long long>(cus) * 8);
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0,
                       mobula_hip::call_state().stream, args...);
    const hipError_t status = hipGetLastError();
    if (status != hipSuccess) mobula_hip::set_error("%s: launch failed: %s", name_, hipGetErrorString(status));
  }

 private:
  mobula_hip::CallBegin begin_;   // (first member: the previous call's error goes before anything can fail)
  const char* name_;
  bool host_;
  bool copies_ = false;
  mobula_hip::DeviceScope scope_;
  mobula_hip::HostStaging stage_;
  hipStream_t saved_stream_ = nullptr;
};

// True if a kernel may dereference `p`: null, device memory, or host memory the
// device can reach (pinned or managed).  Ordinary host memory is refused: a
// kernel that touched it would fault.
template <typename T>
bool device_can_read(T* p) {
  if (p == nullptr) return true;
  hipPointerAttribute_t attr;
  if (hipPointerGetAttributes(&attr, p) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  return attr.type == hipMemoryTypeDevice || attr.type == hipMemoryTypeHost ||
         attr.type == hipMemoryTypeManaged;
}
template <typename T>
bool device_can_read(T) { return true; }   // passed by value

}  // namespace mobula_jit

// KERNEL_RUN(kernel)(n, args...) in a host function of an operator source
// (reference: context/hip_ctx.h:62-106): launches over n iterations on the
// calling thread's stream and waits, as the reference does.  Every pointer
// argument must be memory the device can reach; otherwise nothing is launched
// and the call fails with an error.
namespace mobula {
template <typename Kernel>
class KernelRunner {
 public:
  explicit KernelRunner(Kernel kernel, void* stream = nullptr) : kernel_(kernel), stream_(stream) {}
  template <typename... Args>
  void operator()(const int n, Args... args) {
    if (mobula_hip::failed() || n <= 0) return;
    const bool reachable = (mobula_jit::device_can_read(args) && ...);
    if (!reachable) {
      mobula_hip::set_error("KERNEL_RUN: a pointer argument is ordinary host memory; pass device tensors");
      return;
    }
    int cus = 0, device = 0;
    if (hipGetDevice(&device) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || cus <= 0) {
      (void)hipGetLastError();
      cus = 256;
    }
    const hipStream_t stream = stream_ != nullptr ? static_cast<hipStream_t>(stream_)
                                                  : mobula_hip::call_state().stream;
    const long long blocks = std::min<long long>((static_cast<long long>(n) + 255) / 256,
                                                 static_cast<long long>(cus) * 8);
    hipLaunchKernelGGL(kernel_, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream, n, args...);
    MOBULA_HIP_TRY(hipGetLastError());
    if (!mobula_hip::failed()) MOBULA_HIP_TRY(hipStreamSynchronize(stream));
  }

 private:
  Kernel kernel_;
  void* stream_;
};
}  // namespace mobula

// Device memory helpers for host functions of an operator source (reference:
// context/hip_ctx.h:116-148).  A failure is recorded as the call's error; the
// pointer is then null.
namespace mobula {
template <typename T>
T* new_array(size_t size) {
  void* p = nullptr;
  MOBULA_HIP_TRY(hipMalloc(&p, sizeof(T) * (size > 0 ? size : 1)));
  return mobula_hip::failed() ? nullptr : static_cast<T*>(p);
}
template <typename T>
void del_array(T* p) {
  if (p != nullptr) MOBULA_HIP_TRY(hipFree(p));
}
template <typename T>
T* MemcpyHostToDev(T* dst, const T* src, size_t size) {
  MOBULA_HIP_TRY(hipMemcpy(dst, src, size, hipMemcpyHostToDevice));
  return dst;
}
template <typename T>
T* MemcpyDevToHost(T* dst, const T* src, size_t size) {
  MOBULA_HIP_TRY(hipMemcpy(dst, src, size, hipMemcpyDeviceToHost));
  return dst;
}
template <typename T>
T* MemcpyDevToDev(T* dst, const T* src, size_t size) {
  MOBULA_HIP_TRY(hipMemcpy(dst, src, size, hipMemcpyDeviceToDevice));
  return dst;
}
}  // namespace mobula

#define KERNEL_RUN(a) (mobula::KernelRunner<decltype(&(a))>(&(a)))
#define KERNEL_RUN_STREAM(a, strm) (mobula::KernelRunner<decltype(&(a))>(&(a), strm))
#define KERNEL_RUN_BEGIN(device_id) \
  {                                 \
    mobula_hip::DeviceScope mobula_kernel_run_scope_(device_id);
#define KERNEL_RUN_END() }
