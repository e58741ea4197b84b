// Per-(tile, ROI) sample lists shared by the tiled forward and backward kernels.
//
// A sample at (y, x) touches rows {y_low, y_high} with weights {hy, ly} and
// columns {x_low, x_high} with weights {hx, lx}; the weight of a pixel is the
// product, and a sample outside [-1, size] on either axis contributes nothing
// (opzoo/ROIAlign/bilinear.h:15-48).  Because of this product structure the
// contribution of one ROI to one tile is fully described by two short lists,
//   axis units along y:  (pooled row ph,  local row r,  weights of rows r, r+1)
//   axis units along x:  (pooled col pw,  local col c,  weights of cols c, c+1)
// one unit per sample row / sample column that has a corner inside the tile.
// A corner outside the tile gets weight 0 here (its owner tile accounts for
// it), so local positions range over [-1, T-1].
// Sample coordinates come from roialign_geometry.h (reference operation order).
#pragma once
#include "roialign_tiles.hip.h"

namespace roialign {

// `bin` is the pooled row/column; `pos` the local position of the low corner.
struct alignas(16) AxisUnit { int bin; int pos; float w0, w1; };

// What the tile owners need of a RoiRec, plus the ROI index: 32 bytes.
struct alignas(16) TileRoi {
  float start_h, start_w, bin_h, bin_w;
  int grid_h, grid_w;
  float count;
  int roi;
};

// One wavefront lists the units of one axis: samples (p, i), p < pooled,
// i < grid, whose low or high corner lies in [t0, t0+tsize).  Order = sample
// order.  Returns the (lane-uniform) count, clamped to `cap`.
__device__ __forceinline__ int build_axis_units(float start, float bin, int pooled, int grid,
                                                int size, int t0, int tsize, int lane,
                                                AxisUnit* out, int cap) {
  const int total = pooled * grid;
  int n = 0;
  for (int s0 = 0; s0 < total; s0 += 64) {
    const int s = s0 + lane;
    AxisUnit u;
    bool live = false;
    if (s < total) {
      u.bin = s / grid;
      const AxisSample a = axis_sample(sample_coord(start, u.bin, bin, s - u.bin * grid, grid), size);
      u.pos = a.low - t0;
      const bool lo_in = u.pos >= 0 && u.pos < tsize;
      const bool hi_in = a.high != a.low && u.pos + 1 >= 0 && u.pos + 1 < tsize;
      u.w0 = lo_in ? a.h : 0.0f;
      u.w1 = hi_in ? a.l : 0.0f;
      live = a.valid && (u.w0 != 0.0f || u.w1 != 0.0f);
    }
    const unsigned long long m = __ballot(live);
    const int idx = n + __popcll(m & ((1ull << lane) - 1ull));
    if (live && idx < cap) out[idx] = u;
    n += __popcll(m);
  }
  return min(n, cap);
}

}  // namespace roialign
