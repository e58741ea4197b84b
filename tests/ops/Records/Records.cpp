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

template <typename T>
MOBULA_KERNEL fill_plus_kernel(const int n, const T v, T* inout) {
  parfor(n, [&](int i) { inout[i] += v; });
}

// a host function that launches a kernel itself
MOBULA_FUNC void fill_with_sevens(const int n, float* out) {
  KERNEL_RUN(fill_kernel<float>)(n, 7.0f, out);
}

// a host function that keeps a scratch array on the device for the length of the call:
// out[i] = in[i] + 1 through a device copy made with the memory helpers
MOBULA_FUNC int round_trip_plus_one(const int n, const float* in, float* out) {
  float* scratch = new_array<float>(n);
  if (scratch == nullptr) return -1;
  MemcpyHostToDev(scratch, in, sizeof(float) * n);
  KERNEL_RUN(fill_plus_kernel<float>)(n, 1.0f, scratch);
  MemcpyDevToHost(out, scratch, sizeof(float) * n);
  del_array(scratch);
  return n;
}
