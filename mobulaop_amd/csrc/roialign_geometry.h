// ROI and sample geometry, evaluated in fp32 in exactly the operation order of
// the reference (opzoo/ROIAlign/ROIAlign.cpp:24-65, opzoo/ROIAlign/bilinear.h:
// 15-48).  The validity cut-offs are discontinuous (a sample at y == height
// counts, one a single ulp above does not), so these expressions must not be
// re-associated or fused: the translation unit is compiled with
// -ffp-contract=off and IEEE division.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

namespace roialign {

struct RoiGeom {
  int batch;
  float start_w, start_h;
  float bin_w, bin_h;
  int grid_h, grid_w;
  float count;
};

__device__ __forceinline__ RoiGeom roi_geometry(const float* __restrict__ roi, float scale,
                                                int pooled_h, int pooled_w, int sampling_ratio) {
  RoiGeom g;
  g.batch = static_cast<int>(roi[0]);  // truncation toward zero
  g.start_w = roi[1] * scale;
  g.start_h = roi[2] * scale;
  const float end_w = roi[3] * scale;
  const float end_h = roi[4] * scale;
  const float roi_w = fmaxf(end_w - g.start_w, 1.0f);  // malformed boxes become 1x1
  const float roi_h = fmaxf(end_h - g.start_h, 1.0f);
  g.bin_h = roi_h / static_cast<float>(pooled_h);
  g.bin_w = roi_w / static_cast<float>(pooled_w);
  g.grid_h = sampling_ratio > 0 ? sampling_ratio
                                : static_cast<int>(ceilf(roi_h / static_cast<float>(pooled_h)));
  g.grid_w = sampling_ratio > 0 ? sampling_ratio
                                : static_cast<int>(ceilf(roi_w / static_cast<float>(pooled_w)));
  g.count = static_cast<float>(g.grid_h * g.grid_w);
  return g;
}

// start + p*bin + ((i + .5)*bin)/grid, left to right.
__device__ __forceinline__ float sample_coord(float start, int p, float bin, int i, int grid) {
  const float a = static_cast<float>(p) * bin;
  float b = (static_cast<float>(i) + 0.5f) * bin;
  b = b / static_cast<float>(grid);
  return (start + a) + b;
}

// The samples i of pooled index p whose coordinate lies in [-1, size] -- the only
// ones that contribute (opzoo/ROIAlign/bilinear.h:15-18) -- as a range
// [*first, *last) of [0, grid).  The coordinate never decreases with i (every
// step of sample_coord is monotonic under rounding), so the range is found by
// bisection with that very function: the cut falls exactly where the
// reference's test does.  Grids of ordinary size are not searched (all of
// [0, grid) is returned); the point is to bound the work for boxes far larger
// than the map, or infinite, whose adaptive grid has up to 2^31 points per bin
// of which only about `size` can be valid.
constexpr int kSearchedGrid = 64;

__device__ __forceinline__ void valid_sample_range(float start, int p, float bin, int grid, int size,
                                                   int* first, int* last) {
  *first = 0;
  *last = grid;
  if (grid <= kSearchedGrid) return;
  int lo = 0, hi = grid;
  while (lo < hi) {   // first sample that is not left of -1
    const int mid = lo + (hi - lo) / 2;
    if (sample_coord(start, p, bin, mid, grid) < -1.0f) lo = mid + 1; else hi = mid;
  }
  *first = lo;
  hi = grid;
  while (lo < hi) {   // first sample right of `size`
    const int mid = lo + (hi - lo) / 2;
    if (sample_coord(start, p, bin, mid, grid) > static_cast<float>(size)) hi = mid; else lo = mid + 1;
  }
  *last = lo;
  // A box with infinite corners can give coordinates that are not numbers; they
  // pass the reference's test, every one of them makes the result NaN, and one
  // does so as well as 2^31.
  if (*first < *last && isnan(sample_coord(start, p, bin, *first, grid))) *last = *first + 1;
}

struct AxisSample {
  int low, high;  // the two neighbouring rows (or columns)
  float l, h;     // weight of `high` and of `low`
  bool valid;     // false: the whole sample contributes nothing
};

__device__ __forceinline__ AxisSample axis_sample(float v, int size) {
  AxisSample s;
  s.valid = !(v < -1.0f || v > static_cast<float>(size));
  if (v <= 0.0f) v = 0.0f;
  int lo = static_cast<int>(v);
  if (lo >= size - 1) {
    lo = size - 1;
    s.high = lo;
    v = static_cast<float>(lo);
  } else {
    s.high = lo + 1;
  }
  s.low = lo;
  s.l = v - static_cast<float>(lo);
  s.h = 1.0f - s.l;
  if (!s.valid) { s.low = s.high = 0; s.l = s.h = 0.0f; }
  return s;
}

// Storage types: binary32, binary16 and bfloat16 (the upper half of a binary32);
// arithmetic is always binary32, a result is rounded to nearest-even once.
typedef __bf16 bfloat16;

__device__ __forceinline__ float to_float(float v) { return v; }
__device__ __forceinline__ float to_float(__half v) { return __half2float(v); }
__device__ __forceinline__ float to_float(bfloat16 v) { return static_cast<float>(v); }
template <typename T> __device__ __forceinline__ T from_float(float v);
template <> __device__ __forceinline__ float from_float<float>(float v) { return v; }
template <> __device__ __forceinline__ __half from_float<__half>(float v) { return __float2half_rn(v); }
template <> __device__ __forceinline__ bfloat16 from_float<bfloat16>(float v) { return static_cast<bfloat16>(v); }

}  // namespace roialign
