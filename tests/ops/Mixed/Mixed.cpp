// Test input for the compile-on-load path: argument kinds of the binding
// (several template parameters, scalars whose type follows a tensor, untyped
// pointers, templated host functions) and several loops in one kernel.
#include "mobula_op.h"

namespace mobula {

// five loops of different lengths in one launch: a[i] = i, b[i] = 2i for half of
// n, c[i] = 3i for a third, d and e over 2n and 3n
template <typename T>
MOBULA_KERNEL five_loops_kernel(const int n, T* a, T* b, T* c, T* d, T* e) {
  parfor(n, [&](int i) { a[i] = i; });
  parfor(n / 2, [&](int i) { b[i] = 2 * i; });
  parfor(n / 3, [&](int i) { c[i] = 3 * i; });
  parfor(2 * n, [&](int i) { d[i] = 2 * i; });
  parfor(3 * n, [&](int i) { e[i] = 3 * i; });
}

// two template parameters: the scalar's type comes from the caller, the tensor's from the tensor
template <typename S, typename T>
MOBULA_KERNEL broadcast_kernel(const int n, const S value, T* out) {
  parfor(n, [&](int i) { out[i] = static_cast<T>(value); });
}

// a scalar that shares its template parameter with a tensor takes the tensor's type
template <typename T>
MOBULA_KERNEL fill_like_kernel(const int n, T value, T* out) {
  parfor(n, [&](int i) { out[i] = value; });
}

// an untyped pointer is passed through as an address
template <typename T>
MOBULA_KERNEL address_of_kernel(const int n, const void* p, T* out) {
  parfor(n, [&](int i) { out[i] = static_cast<T>(reinterpret_cast<uintptr_t>(p)); });
}

// host function with a template parameter and a return value
template <typename T>
MOBULA_FUNC T copy_first(const T* from, T* to) {
  to[0] = from[0];
  return from[0];
}

// out[I][J] += a[I][U] * b[U][J], one thread per u: every thread adds to every element
template <typename T>
MOBULA_KERNEL product_by_atomics_kernel(const int U, const int I, const int J, const T* a, const T* b,
                                        T* out) {
  parfor(U, [&](int u) {
    for (int i = 0; i < I; ++i)
      for (int j = 0; j < J; ++j) atomic_add(a[i * U + u] * b[u * J + j], out + i * J + j);
  });
}

// steps[k] = k for k < rounds, written by thread k % threads after k barriers:
// wrong if a barrier lets any thread run ahead
MOBULA_KERNEL ordered_steps_kernel(const int rounds, int* counter, int* steps) {
  const int me = get_thread_num(), all = get_num_threads();
  for (int k = 0; k < rounds; ++k) {
    if (k % all == me) {
      steps[k] = counter[0];
      counter[0] += 1;
    }
    __syncthreads();
  }
}

}  // namespace mobula
