/*
 * TEST INFRASTRUCTURE - NOT PRODUCT CODE.
 *
 * CPU restatement (plain C, fp32, no FMA contraction) of the reference
 * ROIAlign forward/backward arithmetic.  It exists only so that tests, the
 * smoke check and the CPU-baseline leg of the benchmark have something to
 * compare the HIP kernels with; the shipped library never links or calls it.
 *
 * Follows, operation for operation:
 *   opzoo/ROIAlign/ROIAlign.cpp:9-76    roi_align_forward_kernel
 *   opzoo/ROIAlign/ROIAlign.cpp:78-161  roi_align_backward_kernel
 *   opzoo/ROIAlign/bilinear.h:10-59     bilinear_interpolate
 *   opzoo/ROIAlign/bilinear.h:61-112    bilinear_interpolate_gradient
 *   mobula/cpp/include/context/common.h:29-39   parfor block partition
 *   mobula/cpp/include/context/cpu_ctx.h:35-41  atomic_add (omp atomic)
 *
 * Pins (see tests/test_oracle.py): bit-exact against the compiled reference
 * C++ (oracle/_ref) where that is built; the closed-form case of
 * examples/RunROIAlign.py; plane (affine) invariance; adjoint identity
 * <fwd(x),dy> == <x,bwd(dy)>; an independent NumPy brute-force loop on tiny
 * shapes.  No function here is "parity unpinned".
 *
 * Build: see oracle/Makefile (gcc -O2 -fopenmp -ffp-contract=off, no -march).
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* Geometry of one ROI, computed exactly as ROIAlign.cpp:24-54. */
typedef struct {
  int batch;
  float start_w, start_h;
  float bin_w, bin_h;
  int grid_h, grid_w;
  float count;
} roi_geom_t;

static roi_geom_t roi_geometry(const float* roi, float spatial_scale, int pooled_h,
                               int pooled_w, int sampling_ratio) {
  roi_geom_t g;
  g.batch = (int)roi[0]; /* truncation toward zero, ROIAlign.cpp:25 */
  g.start_w = roi[1] * spatial_scale;
  g.start_h = roi[2] * spatial_scale;
  float end_w = roi[3] * spatial_scale;
  float end_h = roi[4] * spatial_scale;
  /* malformed ROIs are forced to 1x1, ROIAlign.cpp:38-39 */
  float roi_w = fmaxf(end_w - g.start_w, 1.0f);
  float roi_h = fmaxf(end_h - g.start_h, 1.0f);
  g.bin_h = roi_h / (float)pooled_h;
  g.bin_w = roi_w / (float)pooled_w;
  g.grid_h = (sampling_ratio > 0) ? sampling_ratio : (int)ceilf(roi_h / (float)pooled_h);
  g.grid_w = (sampling_ratio > 0) ? sampling_ratio : (int)ceilf(roi_w / (float)pooled_w);
  g.count = (float)(g.grid_h * g.grid_w);
  return g;
}

/* Sample coordinate, ROIAlign.cpp:59-65: start + p*bin + ((i+.5)*bin)/grid. */
static inline float sample_coord(float start, int p, float bin, int i, int grid) {
  float a = (float)p * bin;
  float b = ((float)i + 0.5f) * bin;
  b = b / (float)grid;
  return (start + a) + b;
}

/* One axis of bilinear.h:15-48.  Returns 0 if the coordinate is outside
 * [-1, size] (sample contributes nothing), else fills low/high/l/h. */
static inline int axis_weights(float v, int size, int* low, int* high, float* l, float* h) {
  if (v < -1.0f || v > (float)size) return 0;
  if (v <= 0.0f) v = 0.0f;
  int lo = (int)v;
  int hi;
  if (lo >= size - 1) {
    hi = lo = size - 1;
    v = (float)lo;
  } else {
    hi = lo + 1;
  }
  *low = lo;
  *high = hi;
  *l = v - (float)lo;
  *h = 1.0f - *l;
  return 1;
}

static inline float forward_one(const float* plane, int height, int width,
                                const roi_geom_t* g, int ph, int pw) {
  float acc = 0.0f;
  for (int iy = 0; iy < g->grid_h; ++iy) {
    const float y = sample_coord(g->start_h, ph, g->bin_h, iy, g->grid_h);
    for (int ix = 0; ix < g->grid_w; ++ix) {
      const float x = sample_coord(g->start_w, pw, g->bin_w, ix, g->grid_w);
      int yl, yh, xl, xh;
      float ly, hy, lx, hx;
      float val = 0.0f;
      /* validity is a joint test in the reference (bilinear.h:15) */
      if (axis_weights(y, height, &yl, &yh, &ly, &hy) &&
          axis_weights(x, width, &xl, &xh, &lx, &hx)) {
        const float v1 = plane[(size_t)yl * width + xl];
        const float v2 = plane[(size_t)yl * width + xh];
        const float v3 = plane[(size_t)yh * width + xl];
        const float v4 = plane[(size_t)yh * width + xh];
        const float w1 = hy * hx, w2 = hy * lx, w3 = ly * hx, w4 = ly * lx;
        val = w1 * v1 + w2 * v2 + w3 * v3 + w4 * v4;
      }
      acc += val;
    }
  }
  return acc / g->count;
}

/* Same signature as the reference kernel, minus the device id.
 * One work item per output element, in flat (n, c, ph, pw) order. */
void oracle_roi_align_forward_f32(int nthreads, const float* bottom_data,
                                  float spatial_scale, int channels, int height,
                                  int width, int pooled_h, int pooled_w,
                                  int sampling_ratio, const float* bottom_rois,
                                  float* top_data) {
  const int bins = pooled_h * pooled_w;
  const int per_roi = channels * bins;
#pragma omp parallel for schedule(static)
  for (int index = 0; index < nthreads; ++index) {
    const int pw = index % pooled_w;
    const int ph = (index / pooled_w) % pooled_h;
    const int c = (index / bins) % channels;
    const int n = index / per_roi;
    const roi_geom_t g =
        roi_geometry(bottom_rois + (size_t)n * 5, spatial_scale, pooled_h, pooled_w, sampling_ratio);
    const float* plane = bottom_data + ((size_t)g.batch * channels + c) * height * width;
    top_data[index] = forward_one(plane, height, width, &g, ph, pw);
  }
}

static inline void backward_one(float* plane, int height, int width, const roi_geom_t* g,
                                int ph, int pw, float dtop, int use_atomic) {
  for (int iy = 0; iy < g->grid_h; ++iy) {
    const float y = sample_coord(g->start_h, ph, g->bin_h, iy, g->grid_h);
    for (int ix = 0; ix < g->grid_w; ++ix) {
      const float x = sample_coord(g->start_w, pw, g->bin_w, ix, g->grid_w);
      int yl, yh, xl, xh;
      float ly, hy, lx, hx;
      if (!(axis_weights(y, height, &yl, &yh, &ly, &hy) &&
            axis_weights(x, width, &xl, &xh, &lx, &hx)))
        continue; /* indices -1 in the reference: nothing is added */
      const float w1 = hy * hx, w2 = hy * lx, w3 = ly * hx, w4 = ly * lx;
      /* multiply first, then divide: ROIAlign.cpp:143-146 */
      const float g1 = dtop * w1 / g->count;
      const float g2 = dtop * w2 / g->count;
      const float g3 = dtop * w3 / g->count;
      const float g4 = dtop * w4 / g->count;
      float* p1 = plane + (size_t)yl * width + xl;
      float* p2 = plane + (size_t)yl * width + xh;
      float* p3 = plane + (size_t)yh * width + xl;
      float* p4 = plane + (size_t)yh * width + xh;
      if (use_atomic) {
#pragma omp atomic update
        *p1 += g1;
#pragma omp atomic update
        *p2 += g2;
#pragma omp atomic update
        *p3 += g3;
#pragma omp atomic update
        *p4 += g4;
      } else {
        *p1 += g1;
        *p2 += g2;
        *p3 += g3;
        *p4 += g4;
      }
    }
  }
}

/* The reference's own schedule: contiguous block of work items per thread
 * (context/common.h:29-39) and "omp atomic" adds (cpu_ctx.h:35-41).
 * Accumulates INTO bottom_diff; summation order varies from run to run. */
void oracle_roi_align_backward_f32(int nthreads, const float* top_diff, float spatial_scale,
                                   int channels, int height, int width, int pooled_h,
                                   int pooled_w, int sampling_ratio, float* bottom_diff,
                                   const float* bottom_rois) {
  const int bins = pooled_h * pooled_w;
  const int per_roi = channels * bins;
#pragma omp parallel for schedule(static)
  for (int index = 0; index < nthreads; ++index) {
    const int pw = index % pooled_w;
    const int ph = (index / pooled_w) % pooled_h;
    const int c = (index / bins) % channels;
    const int n = index / per_roi;
    const roi_geom_t g =
        roi_geometry(bottom_rois + (size_t)n * 5, spatial_scale, pooled_h, pooled_w, sampling_ratio);
    float* plane = bottom_diff + ((size_t)g.batch * channels + c) * height * width;
    backward_one(plane, height, width, &g, ph, pw, top_diff[index], 1);
  }
}

/* Deterministic schedule with the single-thread summation order of the
 * reference: every (image, channel) plane is owned by one thread, which walks
 * the work items in increasing flat index.  Used where a reproducible answer
 * is needed (golden fixtures, bit-level comparison with a 1-thread reference
 * build).  num_images bounds the batch index (ROIs outside are skipped). */
void oracle_roi_align_backward_f32_ordered(int nthreads, const float* top_diff,
                                           float spatial_scale, int channels, int height,
                                           int width, int pooled_h, int pooled_w,
                                           int sampling_ratio, float* bottom_diff,
                                           const float* bottom_rois, int num_images) {
  const int bins = pooled_h * pooled_w;
  const int per_roi = channels * bins;
  const int num_rois = per_roi > 0 ? nthreads / per_roi : 0;
  const int planes = num_images * channels;
#pragma omp parallel for schedule(dynamic, 1)
  for (int p = 0; p < planes; ++p) {
    const int b = p / channels, c = p % channels;
    float* plane = bottom_diff + (size_t)p * height * width;
    for (int n = 0; n < num_rois; ++n) {
      const roi_geom_t g = roi_geometry(bottom_rois + (size_t)n * 5, spatial_scale, pooled_h,
                                        pooled_w, sampling_ratio);
      if (g.batch != b) continue;
      const float* dy = top_diff + ((size_t)n * channels + c) * bins;
      for (int ph = 0; ph < pooled_h; ++ph)
        for (int pw = 0; pw < pooled_w; ++pw)
          backward_one(plane, height, width, &g, ph, pw, dy[ph * pooled_w + pw], 0);
    }
  }
}

int oracle_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}
