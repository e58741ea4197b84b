// Tile bookkeeping shared by the tiled forward and backward kernels.
//
// The feature map of every image is cut into TH x TW pixel tiles.  A small
// pre-pass turns the ROI list into (a) one geometry record per ROI and (b) for
// every tile the ordered list of ROIs that have at least one sample corner in
// it.  The main kernels are "tile owners": one workgroup per (tile, channel
// block) keeps that piece of the map in LDS and walks its ROI list.
#pragma once
#include "roialign_geometry.h"

namespace roialign {

struct RoiRec {
  float start_h, start_w, bin_h, bin_w;
  int grid_h, grid_w;
  float count;
  int batch;
  // Inclusive pixel box of every corner pixel of every valid sample;
  // row_lo > row_hi means the ROI touches nothing.
  int row_lo, row_hi, col_lo, col_hi;
};

struct TileGrid {
  int th, tw;        // tile size in pixels
  int ty, tx;        // tiles per image along y and x
  int per_image;     // ty * tx
  long long total;   // per_image * num_images
};

// Samples per axis above which the exact scan of sample positions is replaced
// by "may touch anything" (the owners still test every sample exactly).
constexpr int kMaxScan = 4096;

__device__ __forceinline__ void axis_extent(float start, float bin, int pooled, int grid, int size,
                                            int* lo, int* hi) {
  const long long total = static_cast<long long>(pooled) * grid;
  if (total > kMaxScan) { *lo = 0; *hi = size - 1; return; }
  int mn = size, mx = -1;
  for (int p = 0; p < pooled; ++p)
    for (int i = 0; i < grid; ++i) {
      const AxisSample s = axis_sample(sample_coord(start, p, bin, i, grid), size);
      if (s.valid) { mn = min(mn, s.low); mx = max(mx, s.high); }
    }
  *lo = mn; *hi = mx;
}

// One thread per ROI: geometry record + per-tile counters.
__global__ void __launch_bounds__(256)
roi_prepare_kernel(const float* __restrict__ rois, int R, float scale, int PH, int PW, int S, int H,
                   int W, long long num_images, TileGrid tg, RoiRec* __restrict__ recs,
                   int* __restrict__ tile_count) {
  const int r = blockIdx.x * blockDim.x + threadIdx.x;
  if (r >= R) return;
  const RoiGeom g = roi_geometry(rois + static_cast<long long>(r) * 5, scale, PH, PW, S);
  RoiRec rec;
  rec.start_h = g.start_h; rec.start_w = g.start_w; rec.bin_h = g.bin_h; rec.bin_w = g.bin_w;
  rec.grid_h = g.grid_h; rec.grid_w = g.grid_w; rec.count = g.count; rec.batch = g.batch;
  rec.row_lo = rec.col_lo = 0; rec.row_hi = rec.col_hi = -1;
  if (g.batch >= 0 && g.batch < num_images) {
    axis_extent(g.start_h, g.bin_h, PH, g.grid_h, H, &rec.row_lo, &rec.row_hi);
    axis_extent(g.start_w, g.bin_w, PW, g.grid_w, W, &rec.col_lo, &rec.col_hi);
    if (rec.row_lo > rec.row_hi || rec.col_lo > rec.col_hi) {
      rec.row_lo = rec.col_lo = 0; rec.row_hi = rec.col_hi = -1;
    }
  }
  recs[r] = rec;
  if (rec.row_lo <= rec.row_hi) {
    int* base = tile_count + static_cast<long long>(g.batch) * tg.per_image;
    for (int ty = rec.row_lo / tg.th; ty <= rec.row_hi / tg.th; ++ty)
      for (int tx = rec.col_lo / tg.tw; tx <= rec.col_hi / tg.tw; ++tx)
        atomicAdd(base + ty * tg.tx + tx, 1);
  }
}

// Exclusive prefix sum of tile_count[0..n) into tile_offset[0..n]; one block.
__global__ void __launch_bounds__(1024)
tile_scan_kernel(const int* __restrict__ tile_count, long long n, int* __restrict__ tile_offset) {
  __shared__ int wave_sum[16];
  __shared__ int carry;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (threadIdx.x == 0) carry = 0;
  __syncthreads();
  for (long long base = 0; base < n; base += 1024) {
    const long long i = base + threadIdx.x;
    const int v = i < n ? tile_count[i] : 0;
    int incl = v;
    for (int off = 1; off < 64; off <<= 1) {
      const int up = __shfl_up(incl, off);
      if (lane >= off) incl += up;
    }
    if (lane == 63) wave_sum[wave] = incl;
    __syncthreads();
    int before = carry;
    for (int w = 0; w < wave; ++w) before += wave_sum[w];
    if (i < n) tile_offset[i] = before + incl - v;
    __syncthreads();
    if (threadIdx.x == 1023) carry = before + incl;
    __syncthreads();
  }
  if (threadIdx.x == 0) tile_offset[n] = carry;
}

// One wavefront per tile: writes the tile's ROI list in increasing ROI index.
__global__ void __launch_bounds__(256)
tile_fill_kernel(const RoiRec* __restrict__ recs, int R, TileGrid tg,
                 const int* __restrict__ tile_offset, int* __restrict__ tile_rois) {
  const long long tile = (static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x) >> 6;
  if (tile >= tg.total) return;
  const int lane = threadIdx.x & 63;
  const int n = static_cast<int>(tile / tg.per_image);
  const int t = static_cast<int>(tile % tg.per_image);
  const int r0 = (t / tg.tx) * tg.th, c0 = (t % tg.tx) * tg.tw;
  const int begin = tile_offset[tile], want = tile_offset[tile + 1] - begin;
  if (want == 0) return;
  int written = 0;
  for (int base = 0; base < R && written < want; base += 64) {
    const int r = base + lane;
    bool hit = false;
    if (r < R) {
      const RoiRec rec = recs[r];
      hit = rec.batch == n && rec.row_lo <= rec.row_hi && rec.row_hi >= r0 &&
            rec.row_lo < r0 + tg.th && rec.col_hi >= c0 && rec.col_lo < c0 + tg.tw;
    }
    const unsigned long long mask = __ballot(hit);
    if (hit) tile_rois[begin + written + __popcll(mask & ((1ull << lane) - 1ull))] = r;
    written += __popcll(mask);
  }
}

}  // namespace roialign
