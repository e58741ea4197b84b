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

struct TileGrid {
  int th, tw;        // tile size in pixels
  int ty, tx;        // tiles per image along y and x
  int per_image;     // ty * tx
  long long total;   // per_image * num_images
};

// The tiles a ROI touches: image (-1: none), first | last << 16 tile row, first |
// last << 16 tile column.
struct alignas(16) TileBox { int batch; int ty; int tx; int pad; };

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

// One workgroup of four wavefronts per tile: writes the tile's ROI list in
// increasing ROI index.  Each wavefront takes a quarter of the ROIs, counts its
// hits, and after one exchange writes them behind those of the quarters before.
__global__ void __launch_bounds__(256)
tile_fill_kernel(const TileBox* __restrict__ boxes, int R, TileGrid tg,
                 const int* __restrict__ tile_offset, int* __restrict__ tile_rois) {
  __shared__ int hits[4];
  const long long tile = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n = static_cast<int>(tile / tg.per_image);
  const int t = static_cast<int>(tile % tg.per_image);
  const int ty = t / tg.tx, tx = t % tg.tx;
  const int begin = tile_offset[tile], want = tile_offset[tile + 1] - begin;
  if (want == 0) return;
  const int quarter = ((R + 255) / 256) * 64;
  const int r_begin = wave * quarter, r_end = min(R, r_begin + quarter);
  auto hit_of = [&](int r) {
    if (r >= r_end) return false;
    const TileBox b = boxes[r];
    return b.batch == n && ty >= (b.ty & 0xffff) && ty <= (b.ty >> 16) && tx >= (b.tx & 0xffff) &&
           tx <= (b.tx >> 16);
  };
  int mine = 0;
  for (int base = r_begin; base < r_end; base += 64) mine += __popcll(__ballot(hit_of(base + lane)));
  if (lane == 0) hits[wave] = mine;
  __syncthreads();
  int written = begin;
  for (int w = 0; w < wave; ++w) written += hits[w];
  for (int base = r_begin; base < r_end && mine > 0; base += 64) {
    const bool hit = hit_of(base + lane);
    const unsigned long long mask = __ballot(hit);
    if (hit) tile_rois[written + __popcll(mask & ((1ull << lane) - 1ull))] = base + lane;
    written += __popcll(mask);
    mine -= __popcll(mask);
  }
}

}  // namespace roialign
