// Test input for the compile-on-load path: structure arguments, host functions
// that log, check and launch kernels themselves.  (No #include of mobula_op.h:
// the loader supplies it, as for the reference's own test sources.)

struct Span {      // a view of `size` floats
  float* data;
  int size;
};

struct Pair {
  int count;
  float weight;
};

// span->data[i] *= factor; the structure's size field is doubled as a sign that it came back
MOBULA_KERNEL span_scale_kernel(const int n, Span* span, const float factor) {
  CHECK_EQ(n, 1);
  parfor(span->size, [&](int i) { span->data[i] *= factor; });
}

MOBULA_FUNC float pair_total(const Pair* p) {
  LOG(INFO) << "pair of " << p->count << " and " << p->weight;
  return p->count + p->weight;
}

MOBULA_FUNC int positive_or_fail(const int v) {
  CHECK_GT(v, 0) << "need a positive value";
  return v;
}

template <typename T>
MOBULA_KERNEL fill_kernel(const int n, const T v, T* out) {
  parfor(n, [&](int i) { out[i] = v; });
}

// a host function that launches a kernel itself
MOBULA_FUNC void fill_with_sevens(const int n, float* out) {
  KERNEL_RUN(fill_kernel<float>)(n, 7.0f, out);
}
