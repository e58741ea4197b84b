// Test input for the compile-on-load path: kernels whose threads work together
// (reductions over the whole launch, barriers, their own split of the work).
#include "mobula_op.h"

namespace mobula {

// out[0] = the largest of x[0..n)
template <typename T>
MOBULA_KERNEL largest_kernel(const int n, const T* x, T* out) {
  Reduce(n, x, out, max_func<T>, x[0]);
}

// out[0] = x[0] + ... + x[n-1], plain and compensated
template <typename T>
MOBULA_KERNEL plain_total_kernel(const int n, const T* x, T* out) {
  Reduce(n, x, out, add_func<T>, T(0));
}
template <typename T>
MOBULA_KERNEL careful_total_kernel(const int n, const T* x, T* out) {
  Reduce(n, x, out, add_residual_reduce_func<T>, add_residual_merge_func<T>, T(0));
}

// Every row of x[rows][cols] becomes exp(x - max) / sum(exp(x - max)); `cell` is
// one element of scratch.  Two reductions and two elementwise passes per row,
// separated by barriers.
template <typename T>
MOBULA_KERNEL row_weights_kernel(const int cols, const int rows, const T* x, T* cell, T* w) {
  for (int r = 0; r < rows; ++r) {
    const T* src = x + static_cast<size_t>(r) * cols;
    T* dst = w + static_cast<size_t>(r) * cols;
    Reduce(cols, src, cell, max_func<T>, src[0]);
    const T top = cell[0];
    parfor(cols, [&](int i) { dst[i] = exp(src[i] - top); });
    __syncthreads();
    Reduce(cols, dst, cell, add_residual_reduce_func<T>, add_residual_merge_func<T>, T(0));
    const T total = cell[0];
    parfor(cols, [&](int i) { dst[i] /= total; });
    __syncthreads();
  }
}

// owner[i] = the thread that gets iteration i when n iterations are dealt out in
// contiguous shares; threads[0] = how many threads the launch has
MOBULA_KERNEL contiguous_shares_kernel(const int n, int* owner, int* threads) {
  const int me = get_thread_num(), all = get_num_threads();
  int first, last;
  get_parfor_range(n, all, me, &first, &last);
  for (int i = first; i < last; ++i) owner[i] = me;
  if (me == 0) threads[0] = all;
}

}  // namespace mobula
