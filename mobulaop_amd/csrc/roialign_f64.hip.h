// ROIAlign in binary64: the `double` instantiation of the reference kernels
// (opzoo/ROIAlign/ROIAlign.cpp:9-76 with T = double; boxes and scale are T as
// well).  The reference can build only the forward in double (its atomic_add
// takes float, mobula/cpp/include/context/cpu_ctx.h:37); the backward here uses
// the hardware's binary64 atomic add and is an extension.  One thread per
// output element, every expression in the reference's order; these are not
// tuned kernels (binary64 feature maps are a debugging aid, not a workload).
#pragma once
#include <hip/hip_runtime.h>

namespace roialign {

struct RoiGeom64 {
  int batch;
  double start_w, start_h;
  double bin_w, bin_h;
  int grid_h, grid_w;
  double count;
};

__device__ __forceinline__ RoiGeom64 roi_geometry64(const double* __restrict__ roi, double scale,
                                                    int pooled_h, int pooled_w, int sampling_ratio) {
  RoiGeom64 g;
  g.batch = static_cast<int>(roi[0]);
  g.start_w = roi[1] * scale;
  g.start_h = roi[2] * scale;
  const double roi_w = fmax(roi[3] * scale - g.start_w, 1.0);
  const double roi_h = fmax(roi[4] * scale - g.start_h, 1.0);
  g.bin_h = roi_h / static_cast<double>(pooled_h);
  g.bin_w = roi_w / static_cast<double>(pooled_w);
  g.grid_h = sampling_ratio > 0 ? sampling_ratio : static_cast<int>(ceil(roi_h / pooled_h));
  g.grid_w = sampling_ratio > 0 ? sampling_ratio : static_cast<int>(ceil(roi_w / pooled_w));
  g.count = static_cast<double>(g.grid_h * g.grid_w);
  return g;
}

// One axis of a bilinear sample at coordinate start + p*bin + (i+.5)*bin/grid.
struct AxisSample64 {
  int low, high;
  double l, h;   // weights of `high` and `low`
  bool valid;
};

__device__ __forceinline__ double sample_coord64(double start, int p, double bin, int i, int grid) {
  return start + p * bin + (static_cast<double>(i) + 0.5) * bin / static_cast<double>(grid);
}

// [*first, *last): the samples of pooled index p that can be valid; see
// valid_sample_range in roialign_geometry.h (same rule, binary64).
__device__ __forceinline__ void valid_sample_range64(double start, int p, double bin, int grid, int size,
                                                     int* first, int* last) {
  *first = 0;
  *last = grid;
  if (grid <= 64) return;
  int lo = 0, hi = grid;
  while (lo < hi) {
    const int mid = lo + (hi - lo) / 2;
    if (sample_coord64(start, p, bin, mid, grid) < -1.0) lo = mid + 1; else hi = mid;
  }
  *first = lo;
  hi = grid;
  while (lo < hi) {
    const int mid = lo + (hi - lo) / 2;
    if (sample_coord64(start, p, bin, mid, grid) > size) hi = mid; else lo = mid + 1;
  }
  *last = lo;
  if (*first < *last && isnan(sample_coord64(start, p, bin, *first, grid))) *last = *first + 1;
}

__device__ __forceinline__ AxisSample64 axis_sample64(double start, int p, double bin, int i,
                                                      int grid, int size) {
  double v = sample_coord64(start, p, bin, i, grid);
  AxisSample64 s;
  s.valid = !(v < -1.0 || v > size);
  if (v <= 0) v = 0;
  s.low = static_cast<int>(v);
  if (s.low >= size - 1) {
    s.high = s.low = size - 1;
    v = static_cast<double>(s.low);
  } else {
    s.high = s.low + 1;
  }
  s.l = v - s.low;
  s.h = 1.0 - s.l;
  return s;
}

// MODE 0: forward (y = pooled x).  MODE 1: backward (dx += scattered dy).
template <int MODE>
__global__ void __launch_bounds__(256)
roialign_f64_kernel(long long n_out, const double* __restrict__ in, double scale, int C, int H,
                    int W, int PH, int PW, int S, const double* __restrict__ rois,
                    double* __restrict__ out, long long num_images) {
  const long long stride = static_cast<long long>(gridDim.x) * blockDim.x;
  const long long bins = static_cast<long long>(PH) * PW;
  for (long long idx = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x; idx < n_out;
       idx += stride) {
    const int pw = static_cast<int>(idx % PW);
    const int ph = static_cast<int>((idx / PW) % PH);
    const int c = static_cast<int>((idx / bins) % C);
    const long long r = idx / (bins * C);
    const RoiGeom64 g = roi_geometry64(rois + r * 5, scale, PH, PW, S);
    const bool image_ok = g.batch >= 0 && g.batch < num_images;
    const long long plane = (static_cast<long long>(image_ok ? g.batch : 0) * C + c) * H * W;
    const double top = MODE == 1 ? in[idx] : 0.0;
    double acc = 0.0;
    int y0, y1, x0, x1;   // samples outside add nothing
    valid_sample_range64(g.start_h, ph, g.bin_h, g.grid_h, H, &y0, &y1);
    valid_sample_range64(g.start_w, pw, g.bin_w, g.grid_w, W, &x0, &x1);
    for (int iy = y0; image_ok && iy < y1; ++iy) {
      const AxisSample64 sy = axis_sample64(g.start_h, ph, g.bin_h, iy, g.grid_h, H);
      for (int ix = x0; ix < x1; ++ix) {
        const AxisSample64 sx = axis_sample64(g.start_w, pw, g.bin_w, ix, g.grid_w, W);
        if (!(sy.valid && sx.valid)) continue;
        const double w1 = sy.h * sx.h, w2 = sy.h * sx.l, w3 = sy.l * sx.h, w4 = sy.l * sx.l;
        const long long a = plane + static_cast<long long>(sy.low) * W, b = plane + static_cast<long long>(sy.high) * W;
        if (MODE == 0) {
          acc += w1 * in[a + sx.low] + w2 * in[a + sx.high] + w3 * in[b + sx.low] + w4 * in[b + sx.high];
        } else {
          atomicAdd(out + a + sx.low, top * w1 / g.count);
          atomicAdd(out + a + sx.high, top * w2 / g.count);
          atomicAdd(out + b + sx.low, top * w3 / g.count);
          atomicAdd(out + b + sx.high, top * w4 / g.count);
        }
      }
    }
    if (MODE == 0) out[idx] = acc / g.count;
  }
}

}  // namespace roialign
