// The kernel dialect of MobulaOP operator sources, for gfx950.
//
// An operator source written for MobulaOP, e.g.
//     template <typename T>
//     MOBULA_KERNEL axpy_kernel(const int n, const T a, const T* x, T* y) {
//       parfor(n, [&](int i) { y[i] += a * x[i]; });
//     }
// includes "mobula_op.h" and uses MOBULA_KERNEL / MOBULA_DEVICE / MOBULA_FUNC,
// parfor and atomic_add (reference: mobula/cpp/include/mobula_op.h,
// context/hip_ctx.h:4-5,108-114,155-168).  This header gives those names their
// meaning on the GPU: a MOBULA_KERNEL is a __global__ function launched over a
// one-dimensional grid of 256-thread workgroups (four wavefronts), and parfor
// hands out the iterations [0, n) in a grid-stride loop, so consecutive lanes
// take consecutive iterations.  The first parameter of a kernel is the number
// of iterations it is launched for (the reference's convention).
//
// Kernels that synchronise their threads (Reduce, __syncthreads, or their own
// use of get_num_threads / get_thread_num) are launched as ONE workgroup of
// 1024 threads, so that "all threads of the launch" and "all threads a barrier
// reaches" are the same set (the reference launches several workgroups and
// its barrier then reaches only one of them: context/hip_ctx.h:62-90,
// helper.h:10-49); the loader sees which kernels these are from their text.
//
// Also here: LOG(INFO|WARNING|FATAL) and the CHECK macros (logging.h:10-62).
// A failed CHECK or a LOG(FATAL) in host code ends the call with an error the
// binding raises (the reference exits the process); in kernel code they
// compile to nothing.  KERNEL_RUN for host functions is in mobula_jit.h.
//
// Not provided: the reference's host BLAS helper (blas_gemm); sources that need
// it do not build.  new_array / del_array / Memcpy* are in mobula_jit.h.
#pragma once
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cfloat>
#include <cmath>
#include <cstddef>
#include <cstdint>
#include <sstream>
#include <stdexcept>
#include <string>

#define MOBULA_KERNEL __global__ void
#define MOBULA_DEVICE __device__
#define MOBULA_FUNC

namespace mobula {

// C type names as the Python side spells them (reference: ctypes.h:6-18).
typedef wchar_t wchar;
typedef char byte;
typedef unsigned char ubyte;
typedef unsigned short ushort;
typedef unsigned int uint;
typedef unsigned long ulong;
typedef long long longlong;
typedef unsigned long long ulonglong;
typedef long double longdouble;
typedef char* char_p;
typedef wchar_t* wchar_p;
typedef void* void_p;

template <typename... Args>
__host__ __device__ inline void UNUSED(Args&&...) {}

// ---- logging ---------------------------------------------------------------
struct FatalError : std::runtime_error {
  using std::runtime_error::runtime_error;
};

// Collects one message with <<; prints it when the statement ends.  A fatal one
// is thrown as FatalError on the host (generated entry points catch it).
class MobulaLogger {
 public:
  __host__ __device__ MobulaLogger(const char* kind, bool fatal) : kind_(kind), fatal_(fatal) {
#if !defined(__HIP_DEVICE_COMPILE__)
    text_ = new std::ostringstream();
#endif
  }
  template <typename T>
  __host__ __device__ MobulaLogger& operator<<(const T& piece) {
#if !defined(__HIP_DEVICE_COMPILE__)
    *text_ << piece;
#else
    (void)piece;
#endif
    return *this;
  }
  __host__ __device__ ~MobulaLogger() noexcept(false) {
#if !defined(__HIP_DEVICE_COMPILE__)
    const std::string line = std::string("[") + kind_ + "] " + text_->str();
    delete text_;
    if (fatal_) throw FatalError(line);
    fprintf(stdout, "%s\n", line.c_str());
    fflush(stdout);
#endif
  }
  MobulaLogger(const MobulaLogger&) = delete;
  MobulaLogger& operator=(const MobulaLogger&) = delete;

 private:
  const char* kind_;
  bool fatal_;
  std::ostringstream* text_ = nullptr;
};

#define LOG_INFO mobula::MobulaLogger("INFO", false) << __FILE__ << ":" << __LINE__ << " "
#define LOG_WARNING mobula::MobulaLogger("WARNING", false) << __FILE__ << ":" << __LINE__ << " "
#define LOG_FATAL mobula::MobulaLogger("FATAL", true) << __FILE__ << ":" << __LINE__ << " "
#define LOG(KIND) LOG_##KIND
#define CHECK(x) \
  if (!(x)) LOG(FATAL)
#define CHECK_BINARY_OP(op, x, y) \
  if (!((x)op(y))) LOG(FATAL) << " Check Failed: " #x " " #op " " #y " " << " " << x << " vs " << y
#define CHECK_EQ(x, y) CHECK_BINARY_OP(==, x, y)
#define CHECK_NE(x, y) CHECK_BINARY_OP(!=, x, y)
#define CHECK_LE(x, y) CHECK_BINARY_OP(<=, x, y)
#define CHECK_GE(x, y) CHECK_BINARY_OP(>=, x, y)
#define CHECK_LT(x, y) CHECK_BINARY_OP(<, x, y)
#define CHECK_GT(x, y) CHECK_BINARY_OP(>, x, y)

// ---- threads of a launch ---------------------------------------------------
__device__ __forceinline__ int get_num_threads() { return static_cast<int>(gridDim.x * blockDim.x); }
__device__ __forceinline__ int get_thread_num() {
  return static_cast<int>(blockIdx.x * blockDim.x + threadIdx.x);
}

// The contiguous share [*start, *end) of n iterations that thread_id of
// num_threads takes when they are dealt out in blocks, the first n % num_threads
// threads getting one more (reference: context/common.h:29-39).
template <typename index_t>
__host__ __device__ inline void get_parfor_range(const size_t n, const int num_threads, const int thread_id,
                                                 index_t* start, index_t* end) {
  const index_t share = static_cast<index_t>(n / num_threads), extra = static_cast<index_t>(n % num_threads);
  const index_t lead = thread_id < extra ? thread_id : extra;
  *start = share * thread_id + lead;
  *end = *start + share + (thread_id < extra ? 1 : 0);
}

// f(i) for every i in [0, n), iterations shared out over the whole launch.
template <typename Func>
__device__ __forceinline__ void parfor(const size_t n, Func f) {
  const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
  for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += stride)
    f(static_cast<int>(i));
}

// *address += val, atomically; returns the value before (float, double, int,
// unsigned: hardware atomics).
template <typename T>
__device__ __forceinline__ T atomic_add(const T val, T* address) {
  return atomicAdd(address, val);
}

// Sequential helpers operator sources use inside a parfor body.
template <typename T>
struct CArray {
  size_t size;
  T* data;
  __host__ __device__ T& operator[](int i) const { return data[i]; }
};

// a[outer][0][inner] as an offset, for flat index i over [outer][inner].
__device__ __forceinline__ int get_middle_loop_offset(const int i, const int middle_size, const int inner_size) {
  return (i / inner_size) * middle_size * inner_size + i % inner_size;
}

template <typename T>
__device__ __forceinline__ T ADD_FUNC(const T& a, const T& b) { return a + b; }
template <typename T>
__device__ __forceinline__ T MAX_FUNC(const T& a, const T& b) { return a > b ? a : b; }

// out[j] = func(data[j]) for n elements `stride` apart (in place by default).
template <typename F, typename T>
__device__ __forceinline__ void mobula_map(F func, const T* data, const int n, const int stride = 1,
                                           T* out = nullptr) {
  T* dst = out == nullptr ? const_cast<T*>(data) : out;
  for (int i = 0; i < n; ++i) dst[i * stride] = func(data[i * stride]);
}

// out[0] = func(... func(func(data[0], data[stride]), data[2 stride]) ...).
template <typename F, typename T>
__device__ __forceinline__ void mobula_reduce(F func, const T* data, const int n, const int stride = 1,
                                              T* out = nullptr) {
  T* dst = out == nullptr ? const_cast<T*>(data) : out;
  T acc = data[0];
  for (int i = 1; i < n; ++i) acc = func(acc, data[i * stride]);
  dst[0] = acc;
}

// ---- reductions over the whole launch (one workgroup, see the head) ---------
// Combining functions of Reduce (reference: helper.h:96-124).
template <typename T>
__device__ void max_func(T& dst, const T& src) {
  if (src > dst) dst = src;
}
template <typename T>
__device__ void add_func(T& dst, const T& src) {
  dst += src;
}
// Compensated addition: `residual` carries what the rounded sum lost.
template <typename T>
__device__ void add_residual_reduce_func(T& dst, const T& src, T& residual) {
  const T term = src - residual;
  const T sum = dst + term;
  residual = (sum - dst) - term;
  dst = sum;
}
// (dst, dst_residual) += (src, src_residual), both compensated sums in the
// convention of add_residual_reduce_func: the exact value of a pair is
// sum - residual.  (The reference's merge, helper.h:114-124, adds the residuals
// with the other sign; the two agree to a few units in the last place.)
template <typename T>
__device__ void add_residual_merge_func(T& dst, T& dst_residual, const T& src, const T& src_residual) {
  const T sum = dst + src;
  const T part = sum - dst;
  const T lost = (src - part) + (dst - (sum - part));   // dst + src == sum + lost, exactly
  const T fix = lost - dst_residual - src_residual;
  dst = sum + fix;
  dst_residual = (dst - sum) - fix;
}

namespace detail {
constexpr int kMaxLaunchThreads = 1024;
// Shared slots of a reduction, one per thread, for any trivially copyable T.
template <typename T, int WHICH>
__device__ __forceinline__ T* reduce_slots() {
  __shared__ __align__(16) unsigned char raw[kMaxLaunchThreads * sizeof(T)];
  return reinterpret_cast<T*>(raw);
}
}  // namespace detail

// out[0] = func folded over init and data[0..n), by all threads of the launch
// together (every thread must call it; the launch is one workgroup).  Only
// out[0] is written.
template <typename T>
__device__ void Reduce(const int n, const T* data, T* out, void (*func)(T&, const T&), T init) {
  T* const slot = detail::reduce_slots<T, 0>();
  const int threads = static_cast<int>(blockDim.x), me = static_cast<int>(threadIdx.x);
  T acc = init;
  for (int i = me; i < n; i += threads) func(acc, data[i]);
  __syncthreads();            // the slots may still be read by a previous reduction
  slot[me] = acc;
  __syncthreads();
  for (int width = 1; width < threads; width <<= 1) {
    if ((me & (2 * width - 1)) == 0 && me + width < threads) func(slot[me], slot[me + width]);
    __syncthreads();
  }
  if (me == 0) out[0] = slot[0];
  __syncthreads();            // out[0] is visible to every thread of the launch on return
}

// The same with a compensation term per partial result: func_reduce(acc, x,
// residual) adds one element, func_merge(acc, acc_residual, other,
// other_residual) joins two partial results.
template <typename T>
__device__ void Reduce(const int n, const T* data, T* out, void (*func_reduce)(T&, const T&, T&),
                       void (*func_merge)(T&, T&, const T&, const T&), T init) {
  T* const slot = detail::reduce_slots<T, 1>();
  T* const lost = detail::reduce_slots<T, 2>();
  const int threads = static_cast<int>(blockDim.x), me = static_cast<int>(threadIdx.x);
  T acc = init, residual = T(0);
  for (int i = me; i < n; i += threads) func_reduce(acc, data[i], residual);
  __syncthreads();
  slot[me] = acc;
  lost[me] = residual;
  __syncthreads();
  for (int width = 1; width < threads; width <<= 1) {
    if ((me & (2 * width - 1)) == 0 && me + width < threads)
      func_merge(slot[me], lost[me], slot[me + width], lost[me + width]);
    __syncthreads();
  }
  if (me == 0) out[0] = slot[0];
  __syncthreads();
}

}  // namespace mobula
