// A user operator in MobulaOP's kernel dialect (test input for the compile-on-load path).
#include "mobula_op.h"

namespace mobula {

// y[i] += a * x[i]
template <typename T>
MOBULA_KERNEL axpy_kernel(const int n, const T a, const T* x, T* y) {
  parfor(n, [&](int i) { y[i] += a * x[i]; });
}

// hist[bin[i]] += w[i]: many iterations add to one address
template <typename T>
MOBULA_KERNEL weighted_histogram_kernel(const int n, const int* bin, const T* w, T* hist) {
  parfor(n, [&](int i) { atomic_add(w[i], hist + bin[i]); });
}

MOBULA_DEVICE float squared(const float v) { return v * v; }

// out[r] = sum over the row of x[r][c]^2, rows of `cols` elements
MOBULA_KERNEL row_energy_kernel(const int rows, const int cols, const float* x, float* out) {
  parfor(rows, [&](int r) {
    float acc = 0.0f;
    for (int c = 0; c < cols; ++c) acc += squared(x[r * cols + c]);
    out[r] = acc;
  });
}

// a host function, exported as it is
MOBULA_FUNC int padded_length(const int n, const int multiple) {
  return (n + multiple - 1) / multiple * multiple;
}

}  // namespace mobula
