/*
 * TEST INFRASTRUCTURE - NOT PRODUCT CODE.
 *
 * CPU restatement of the reference ROIAlign arithmetic with T = double
 * (opzoo/ROIAlign/ROIAlign.cpp:9-76 forward, :78-161 backward;
 * opzoo/ROIAlign/bilinear.h:10-112), boxes and scale in double as well.  The
 * reference itself can only build the forward in double (its atomic_add takes
 * float, mobula/cpp/include/context/cpu_ctx.h:37); the backward here is the same
 * scatter written in double, one (image, channel) plane per thread so that no
 * atomics are needed.
 *
 * Pins (tests/test_oracle.py): the forward bit-exact against the compiled
 * reference <double> instantiation (oracle/_ref) where that is built and
 * against the float64 brute-force loop of oracle/roialign.py; the backward by
 * the adjoint identity <fwd(x),dy> == <x,bwd(dy)> and the same brute force.
 * No function here is "parity unpinned".
 *
 * Structure differs from the fp32 file on purpose: the samples of one axis of
 * one ROI are tabulated once (they do not depend on the channel).
 */
#include <math.h>
#include <stddef.h>
#include <stdlib.h>

typedef struct {
  int valid, low, high;
  double l, h;
} axis_t;

/* Samples of pooled index p = 0..pooled-1, i = 0..grid-1 along one axis.
 * Coordinate: start + p*bin + (i+.5)*bin/grid (ROIAlign.cpp:59-65), then the
 * per-axis half of bilinear.h:15-48. */
static void tabulate(axis_t* t, double start, double bin, int pooled, int grid, int size) {
  for (int p = 0; p < pooled; ++p)
    for (int i = 0; i < grid; ++i, ++t) {
      double v = start + p * bin + ((double)i + 0.5) * bin / (double)grid;
      t->valid = !(v < -1.0 || v > size);
      if (v <= 0) v = 0;
      t->low = (int)v;
      if (t->low >= size - 1) {
        t->high = t->low = size - 1;
        v = (double)t->low;
      } else {
        t->high = t->low + 1;
      }
      t->l = v - t->low;
      t->h = 1.0 - t->l;
    }
}

typedef struct {
  int batch, grid_h, grid_w;
  double count;
  axis_t *rows, *cols; /* [PH*grid_h], [PW*grid_w] */
} roi_tables_t;

static roi_tables_t make_tables(const double* roi, double scale, int H, int W, int PH, int PW, int S) {
  roi_tables_t r;
  r.batch = (int)roi[0];
  const double sw = roi[1] * scale, sh = roi[2] * scale;
  const double ew = roi[3] * scale, eh = roi[4] * scale;
  const double rw = fmax(ew - sw, 1.0), rh = fmax(eh - sh, 1.0);
  const double bh = rh / (double)PH, bw = rw / (double)PW;
  r.grid_h = S > 0 ? S : (int)ceil(rh / PH);
  r.grid_w = S > 0 ? S : (int)ceil(rw / PW);
  r.count = (double)(r.grid_h * r.grid_w);
  r.rows = (axis_t*)malloc(sizeof(axis_t) * (size_t)PH * r.grid_h);
  r.cols = (axis_t*)malloc(sizeof(axis_t) * (size_t)PW * r.grid_w);
  tabulate(r.rows, sh, bh, PH, r.grid_h, H);
  tabulate(r.cols, sw, bw, PW, r.grid_w, W);
  return r;
}

/* mode 0: top[n,c,ph,pw] = pooled bottom.  mode 1: bottom += scattered top. */
static void run(int mode, int num_rois, int num_images, const double* rois, double scale, int C, int H,
                int W, int PH, int PW, int S, double* bottom, double* top) {
  roi_tables_t* tab = (roi_tables_t*)malloc(sizeof(roi_tables_t) * (size_t)(num_rois > 0 ? num_rois : 1));
  for (int n = 0; n < num_rois; ++n) tab[n] = make_tables(rois + (size_t)n * 5, scale, H, W, PH, PW, S);
  const int planes = num_images * C;
#pragma omp parallel for schedule(dynamic, 1)
  for (int pl = 0; pl < planes; ++pl) {
    const int b = pl / C, c = pl % C;
    double* plane = bottom + (size_t)pl * H * W;
    for (int n = 0; n < num_rois; ++n) { /* increasing flat index: the 1-thread order of the reference */
      const roi_tables_t* r = &tab[n];
      if (r->batch != b) continue;
      double* t = top + ((size_t)n * C + c) * PH * PW;
      for (int ph = 0; ph < PH; ++ph)
        for (int pw = 0; pw < PW; ++pw) {
          double acc = 0.0;
          for (int iy = 0; iy < r->grid_h; ++iy) {
            const axis_t* y = &r->rows[ph * r->grid_h + iy];
            for (int ix = 0; ix < r->grid_w; ++ix) {
              const axis_t* x = &r->cols[pw * r->grid_w + ix];
              if (!(y->valid && x->valid)) continue;
              const double w1 = y->h * x->h, w2 = y->h * x->l, w3 = y->l * x->h, w4 = y->l * x->l;
              double* v1 = plane + (size_t)y->low * W + x->low;
              double* v2 = plane + (size_t)y->low * W + x->high;
              double* v3 = plane + (size_t)y->high * W + x->low;
              double* v4 = plane + (size_t)y->high * W + x->high;
              if (mode == 0) {
                acc += w1 * *v1 + w2 * *v2 + w3 * *v3 + w4 * *v4;
              } else {
                const double g = t[ph * PW + pw];
                *v1 += g * w1 / r->count;
                *v2 += g * w2 / r->count;
                *v3 += g * w3 / r->count;
                *v4 += g * w4 / r->count;
              }
            }
          }
          if (mode == 0) t[ph * PW + pw] = acc / r->count;
        }
    }
  }
  for (int n = 0; n < num_rois; ++n) {
    free(tab[n].rows);
    free(tab[n].cols);
  }
  free(tab);
}

/* Outputs of ROIs whose batch index is outside [0, num_images) are left as the
 * caller set them (the reference would read out of bounds). */
void oracle_roi_align_forward_f64(int num_rois, int num_images, const double* bottom_data,
                                  double spatial_scale, int channels, int height, int width,
                                  int pooled_h, int pooled_w, int sampling_ratio,
                                  const double* bottom_rois, double* top_data) {
  run(0, num_rois, num_images, bottom_rois, spatial_scale, channels, height, width, pooled_h, pooled_w,
      sampling_ratio, (double*)bottom_data, top_data);
}

/* Accumulates INTO bottom_diff. */
void oracle_roi_align_backward_f64(int num_rois, int num_images, const double* top_diff,
                                   double spatial_scale, int channels, int height, int width,
                                   int pooled_h, int pooled_w, int sampling_ratio, double* bottom_diff,
                                   const double* bottom_rois) {
  run(1, num_rois, num_images, bottom_rois, spatial_scale, channels, height, width, pooled_h, pooled_w,
      sampling_ratio, bottom_diff, (double*)top_diff);
}
