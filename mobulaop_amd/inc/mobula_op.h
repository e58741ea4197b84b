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
// Not provided: the reference's host-side helpers (blas_gemm, new_array, ...)
// and its block-level Reduce; sources that need them do not build.
#pragma once
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cfloat>
#include <cmath>
#include <cstddef>
#include <cstdint>

#define MOBULA_KERNEL __global__ void
#define MOBULA_DEVICE __device__
#define MOBULA_FUNC

namespace mobula {

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

}  // namespace mobula
