// Per-ROI sample lists shared by the tiled kernels.
//
// A sample at (y, x) touches rows {y_low, y_high} with weights {hy, ly} and
// columns {x_low, x_high} with weights {hx, lx}; the weight of a pixel is the
// product, and a sample outside [-1, size] on either axis contributes nothing
// (opzoo/ROIAlign/bilinear.h:15-48).  Because of this product structure the
// contribution of one ROI to one tile is fully described by two short lists,
//   units along y:  (pooled row ph,  local row r,  weights of rows r, r+1)
//   units along x:  (pooled col pw,  local col c,  weights of cols c, c+1)
// one unit per sample row / sample column.  A corner outside the tile gets
// weight 0 (its owner tile accounts for it), so local positions range over
// [-1, T-1]; a unit with both weights 0 is dead.
//
// The lists depend only on (ROI, tile row) and (ROI, tile column), so the
// pre-pass writes them once to memory and every tile owner that needs them
// reads them back:
//   row taps  of (roi, ty): for each of the tile's rows the (pooled row, weight)
//                           pairs that land on it, weights already divided by
//                           the sample count of the bin: a 16-entry index
//                           (start | count << 8) followed by the taps, sorted
//                           by tile row, then by sample order
//   col list  of (roi, tx): one 16-byte ColPair per pooled column (padded to a
//                           multiple of 8 columns): its one or two sample columns
// The lists hold one or two sample points per bin and axis.  A larger sampling
// grid (a ratio above 2, or the adaptive ceil(bin size)) is cut into pieces of
// 2 x 2 points: every piece is a list item of its own, with the box, the row
// taps and the column pairs of its own points, and the tile owners add the
// pieces up like so many ROIs that share one dy (the gradient is a sum over
// sample points).  `piece_offsets_kernel` numbers the pieces.
// Sample coordinates come from roialign_geometry.h (reference operation order).
#pragma once
#include "roialign_tiles.hip.h"

namespace roialign {

// `bin` is the pooled row/column; `pos` the local position of the low corner.
struct alignas(16) AxisUnit { int bin; int pos; float w0, w1; };

// The sample columns of one pooled column inside one tile column band.
//   cells  (pos0 + 1) | (pos1 + 1) << 16: index of the low corner's cell in a tile
//          row whose cell 0 is a dummy to the left of the tile (so a low corner
//          one column left of the tile is cell 0, its high corner cell 1)
//   flags  bit 0/1: low/high corner of sample 0 lies in the tile and has a
//          non-zero weight; bit 2/3: same for sample 1; bits 8..10: log2 of the
//          smallest power-of-two distance (in pooled columns, at most 8) at
//          which the first (and likewise the second) samples of two pooled
//          columns never share a cell: columns that far apart are added concurrently
//   l0/l1  weight of the high corner; the low corner weighs 1 - l
struct alignas(16) ColPair { int cells; int flags; float l0, l1; };
constexpr int kColStrideShift = 8;
constexpr int kColStrideMask = 7;

constexpr int kRowSlots = 64;   // PH * S <= 64 sample rows per ROI (one per lane of the list builder)
constexpr int kMaxListPW = 32;  // PW * S <= 64 sample columns, one or two sample points per bin
constexpr int kTileRows = 16;   // rows of a tile (fixed by the row-tap index)

struct RowTap { int ph; float wy; };
// Row taps of one (roi, tile row): 32-byte index + two taps per sample row.  In memory a
// table ends after the taps its shape can have (ListLayout::row_stride), not after taps[].
struct alignas(16) RowTapTable {
  unsigned short index[kTileRows];   // start | count << 8, per tile row
  RowTap taps[2 * kRowSlots];
};
// 16-byte units of a table for `slots` sample rows
inline int row_table_units(int slots) { return 2 + slots; }

struct ListLayout {
  int ty, tx;            // tiles per image
  int row_stride;        // 16-byte units per (roi, ty) row-tap table
  int col_stride;        // 16-byte units per (roi, tx) column list: PW rounded up to 8
  long long roi_stride;  // units per ROI: ty*row_stride + tx*col_stride
};

inline ListLayout make_list_layout(const TileGrid& tg, int PH, int PW, int S) {
  ListLayout l;
  l.ty = tg.ty; l.tx = tg.tx;
  l.row_stride = row_table_units(PH * (S == 1 ? 1 : 2));
  l.col_stride = (PW + 7) / 8 * 8;
  l.roi_stride = static_cast<long long>(l.ty) * l.row_stride + static_cast<long long>(l.tx) * l.col_stride;
  return l;
}

inline bool lists_in_pieces(int S) { return S != 1 && S != 2; }
inline bool lists_supported(int PH, int PW, int S) {
  return PH * (S == 1 ? 1 : 2) <= kRowSlots && PW <= kMaxListPW;
}

// offsets[r] = number of the first piece of ROI r, offsets[R] = their total;
// info[0] = the total, info[1] = 1 if some ROI's grid has more than
// kSearchedGrid points along an axis (such ROIs are not cut up: the caller
// takes another path).  One workgroup of 1024 threads.
__global__ void __launch_bounds__(1024)
piece_offsets_kernel(const float* __restrict__ rois, int R, float scale, int PH, int PW, int S,
                     int* __restrict__ offsets, int* __restrict__ info) {
  __shared__ int part[1024];
  __shared__ int too_big;
  const int t = threadIdx.x, share = (R + 1023) / 1024;
  const int first = min(R, t * share), last = min(R, first + share);
  if (t == 0) too_big = 0;
  __syncthreads();
  auto pieces_of = [&](int r) {
    const RoiGeom g = roi_geometry(rois + static_cast<long long>(r) * 5, scale, PH, PW, S);
    if (g.grid_h > kSearchedGrid || g.grid_w > kSearchedGrid || g.grid_h < 1 || g.grid_w < 1) {
      too_big = 1;
      return 0;
    }
    return ((g.grid_h + 1) / 2) * ((g.grid_w + 1) / 2);
  };
  int sum = 0;
  for (int r = first; r < last; ++r) sum += pieces_of(r);
  part[t] = sum;
  __syncthreads();
  if (t == 0) {   // exclusive prefix over the threads
    int run = 0;
    for (int i = 0; i < 1024; ++i) { const int c = part[i]; part[i] = run; run += c; }
    offsets[R] = run;
    info[0] = run;
  }
  __syncthreads();
  int at = part[t];
  for (int r = first; r < last; ++r) {
    offsets[r] = at;
    at += pieces_of(r);
  }
  __syncthreads();
  if (t == 0) info[1] = too_big;
}

__device__ __forceinline__ AxisUnit clip_unit(int bin, const AxisSample& a, int t0, int tsize,
                                              float scale) {
  AxisUnit u;
  u.bin = bin;
  u.pos = a.low - t0;
  const bool lo_in = a.valid && u.pos >= 0 && u.pos < tsize;
  const bool hi_in = a.valid && a.high != a.low && u.pos + 1 >= 0 && u.pos + 1 < tsize;
  u.w0 = lo_in ? a.h * scale : 0.0f;
  u.w1 = hi_in ? a.l * scale : 0.0f;
  // dead units point at the two dummy cells to the right of a tile row
  if (!(lo_in || hi_in) || (u.w0 == 0.0f && u.w1 == 0.0f)) { u.pos = tsize; u.w0 = u.w1 = 0.0f; }
  return u;
}

// One wavefront per ROI: lane s < PH*S evaluates sample row s once and clips it
// against every tile row of the ROI's box; likewise for sample columns.
// The wavefront also finds the ROI's box (the pixels any valid sample touches),
// and stores it as tile ranges for build_tile_work_kernel.
// `block`: index among the workgroups (of 256 threads) that build lists.
struct ListsArgs {
  const float* rois;
  int items, R;
  float scale;
  int PH, PW, S_given, H, W;
  long long num_images;
  TileGrid tg;
  ListLayout ll;
  TileBox* boxes;
  int* cursors;
  AxisUnit* lists;
  const int* piece_offsets;
};

__device__ __forceinline__ void build_lists_body(unsigned block, const ListsArgs& a) {
  const float* __restrict__ rois = a.rois;
  const int items = a.items, R = a.R, PH = a.PH, PW = a.PW, S_given = a.S_given, H = a.H, W = a.W;
  const float scale = a.scale;
  const long long num_images = a.num_images;
  const TileGrid tg = a.tg;
  const ListLayout ll = a.ll;
  TileBox* __restrict__ boxes = a.boxes;
  int* __restrict__ cursors = a.cursors;
  AxisUnit* __restrict__ lists = a.lists;
  const int* __restrict__ piece_offsets = a.piece_offsets;
  // the two bump pointers of build_tile_work_kernel, which runs after this one
  if (block == 0 && threadIdx.x < 2) cursors[threadIdx.x] = 0;
  // item: a ROI, or (piece_offsets given) one 2 x 2 piece of a ROI's sampling grid
  const int item = static_cast<int>((block * 256u + threadIdx.x) >> 6);
  if (item >= items) return;
  const int lane = threadIdx.x & 63;
  int roi = item;
  if (piece_offsets != nullptr) {   // the ROI whose pieces include this one
    int lo = 0, hi = R;
    while (hi - lo > 1) {
      const int mid = (lo + hi) / 2;
      if (piece_offsets[mid] <= item) lo = mid; else hi = mid;
    }
    roi = lo;
  }
  const RoiGeom g = roi_geometry(rois + static_cast<long long>(roi) * 5, scale, PH, PW, S_given);
  // S points per bin and axis in this item, the first of them point (y_first, x_first) of the grid
  const int S = piece_offsets != nullptr ? 2 : S_given;
  int y_first = 0, x_first = 0;
  if (piece_offsets != nullptr) {
    const int local = item - piece_offsets[roi], across = (g.grid_w + 1) / 2;
    y_first = 2 * (local / across);
    x_first = 2 * (local % across);
  }
  // one row sample and one column sample per lane
  const int iy = y_first + lane % S, ix_of_lane = x_first + lane % S;
  AxisSample ay = axis_sample(sample_coord(g.start_h, lane / S, g.bin_h, iy, g.grid_h), H);
  ay.valid = ay.valid && lane < PH * S && iy < g.grid_h;
  AxisSample ax = axis_sample(sample_coord(g.start_w, lane / S, g.bin_w, ix_of_lane, g.grid_w), W);
  ax.valid = ax.valid && lane < PW * S && ix_of_lane < g.grid_w;
  struct { int row_lo, row_hi, col_lo, col_hi; float start_h, start_w, bin_h, bin_w, count; } rec;
  rec.start_h = g.start_h; rec.start_w = g.start_w; rec.bin_h = g.bin_h; rec.bin_w = g.bin_w;
  rec.count = g.count;
  {
    int rlo = ay.valid ? ay.low : H, rhi = ay.valid ? ay.high : -1;
    int clo = ax.valid ? ax.low : W, chi = ax.valid ? ax.high : -1;
    for (int off = 32; off > 0; off >>= 1) {
      rlo = min(rlo, __shfl_xor(rlo, off)); rhi = max(rhi, __shfl_xor(rhi, off));
      clo = min(clo, __shfl_xor(clo, off)); chi = max(chi, __shfl_xor(chi, off));
    }
    const bool image_ok = g.batch >= 0 && g.batch < num_images;
    const bool any = image_ok && rlo <= rhi && clo <= chi;
    rec.row_lo = any ? rlo : 0; rec.row_hi = any ? rhi : -1;
    rec.col_lo = any ? clo : 0; rec.col_hi = any ? chi : -1;
    const int ty0 = rec.row_lo / tg.th, ty1 = any ? rec.row_hi / tg.th : -1;
    const int tx0 = rec.col_lo / tg.tw, tx1 = any ? rec.col_hi / tg.tw : -1;
    if (lane == 0) boxes[item] = TileBox{any ? g.batch : -1, ty0 | (ty1 << 16), tx0 | (tx1 << 16), roi};
    if (!any) return;
  }
  AxisUnit* const base = lists + static_cast<long long>(item) * ll.roi_stride;
  const float inv_count = 1.0f / rec.count;
  {
    const int ph = lane / S;
    const AxisSample a = ay;
    for (int ty = rec.row_lo / tg.th; ty <= rec.row_hi / tg.th; ++ty) {
      const AxisUnit u = clip_unit(ph, a, ty * tg.th, tg.th, inv_count);
      RowTapTable* const table = reinterpret_cast<RowTapTable*>(base + ty * ll.row_stride);
      // each unit lands on up to two tile rows; order the taps by row, then by lane
      const int row0 = u.w0 != 0.0f ? u.pos : -1, row1 = u.w1 != 0.0f ? u.pos + 1 : -1;
      int start = 0;
      for (int r = 0; r < kTileRows; ++r) {
        const unsigned long long m0 = __ballot(row0 == r), m1 = __ballot(row1 == r);
        const unsigned long long below = (1ull << lane) - 1ull;
        // a unit's high row is the next unit's low row: high parts first keeps sample order
        const int n1 = __popcll(m1), n0 = __popcll(m0);
        if (row1 == r) table->taps[start + __popcll(m1 & below)] = RowTap{ph, u.w1};
        if (row0 == r) table->taps[start + n1 + __popcll(m0 & below)] = RowTap{ph, u.w0};
        if (lane == 0) table->index[r] = static_cast<unsigned short>(start | ((n0 + n1) << 8));
        start += n0 + n1;
      }
    }
  }
  {
    // lane = sample column pw * S + ix
    const int pw = lane / S, ix = lane - pw * S;
    const bool real = lane < PW * S;
    const AxisSample a = ax;
    ColPair* const cols = reinterpret_cast<ColPair*>(base + static_cast<long long>(ll.ty) * ll.row_stride);
    for (int tx = rec.col_lo / tg.tw; tx <= rec.col_hi / tg.tw; ++tx) {
      int pos = a.low - tx * tg.tw;
      const bool lo_in = a.valid && pos >= 0 && pos < tg.tw && a.h != 0.0f;
      const bool hi_in = a.valid && a.high != a.low && pos + 1 >= 0 && pos + 1 < tg.tw && a.l != 0.0f;
      const bool live = lo_in || hi_in;
      if (!live) pos = -1;
      // smallest power-of-two distance at which no two live samples share a cell
      int lg = 0;
#pragma unroll
      for (int d = 1; d <= 16; d <<= 1) {
        const int pos_d = __shfl_down(pos, d);
        const bool live_d = __shfl_down(live ? 1 : 0, d) != 0;
        const bool clash = live && live_d && lane + d < PW * S && pos_d - pos >= -1 && pos_d - pos <= 1;
        if (__ballot(clash) != 0) lg = (d == 16) ? 5 : __builtin_ctz(d) + 1;
      }
      const int fl = (lo_in ? 1 : 0) | (hi_in ? 2 : 0);
      const int pos_n = __shfl_down(pos, 1), fl_n = __shfl_down(fl, 1);
      const float l_n = __shfl_down(a.l, 1);
      ColPair cp;
      cp.cells = (pos + 1) | ((S == 2 ? pos_n + 1 : 0) << 16);
      // Lanes take the first samples of their pooled columns together, then the
      // second ones: columns t apart are S * t samples apart.
      const int turns_log = max(0, min(3, lg - (S == 2 ? 1 : 0)));
      cp.flags = fl | ((S == 2 ? fl_n : 0) << 2) | (turns_log << kColStrideShift);
      cp.l0 = a.l;
      cp.l1 = S == 2 ? l_n : 0.0f;
      if (real && ix == 0) cols[tx * ll.col_stride + pw] = cp;
      // padding columns: nothing to add, same spacing
      if (lane < ll.col_stride - PW)
        cols[tx * ll.col_stride + PW + lane] = ColPair{0, turns_log << kColStrideShift, 0.0f, 0.0f};
    }
  }
}

__global__ void __launch_bounds__(256) build_lists_kernel(ListsArgs a) { build_lists_body(blockIdx.x, a); }


// One wavefront's share of a tile: the (ROI, pooled row, weight) taps that land
// on one tile row, in ROI order, so that the owner of that row streams through
// them without looking anything up.
struct alignas(16) WorkEntry {
  int roi;     // the list item (its column pairs are read from its lists)
  int ph;
  float wy;
  int flags;   // bit 0: continues the previous entry's item; bit 1: last entry of its item;
               // bits 2..: the ROI whose dy the entry reads (the item itself, or the ROI it is a piece of)
};
struct WorkRange { int begin; int count; };

// One workgroup per tile, one wavefront per tile row.
// First the tile's ROI list: every wavefront takes a sixteenth of the ROIs,
// counts those whose box covers the tile, and after one exchange writes them,
// in increasing ROI index, into space taken from cursors[0] with one atomic.
// Then the work lists: lane j looks at ROI j of the tile's list, takes its taps
// for this wavefront's row from the row-tap table, and all lanes append theirs
// in list order.  WorkRange::count includes the padding.  Space for the tile's
// sixteen lists comes from one bump-pointer allocation per tile (cursors[1]).
// The order in which tiles take their space varies from run to run; what is
// written into it does not.
__global__ void __launch_bounds__(kTileRows * 64)
build_tile_work_kernel(const TileBox* __restrict__ boxes, int R, int* __restrict__ tile_rois,
                       const AxisUnit* __restrict__ lists, TileGrid tg, ListLayout ll,
                       int* __restrict__ cursors, WorkRange* __restrict__ ranges,
                       WorkEntry* __restrict__ entries) {
  __shared__ int hits[kTileRows];
  __shared__ int row_total[kTileRows];
  __shared__ int list_base, tile_base;
  const long long tile = blockIdx.x;
  const int lane = threadIdx.x & 63, row = threadIdx.x >> 6;
  const int image = static_cast<int>(tile / tg.per_image);
  const int t = static_cast<int>(tile % tg.per_image);
  const int ty = t / tg.tx, tx = t % tg.tx;

  // ---- the tile's ROI list ----
  const int share = ((R + kTileRows * 64 - 1) / (kTileRows * 64)) * 64;
  const int r_begin = row * share, r_end = min(R, r_begin + share);
  auto hit_of = [&](int r) {
    if (r >= r_end) return false;
    const TileBox b = boxes[r];
    return b.batch == image && ty >= (b.ty & 0xffff) && ty <= (b.ty >> 16) && tx >= (b.tx & 0xffff) &&
           tx <= (b.tx >> 16);
  };
  int mine = 0;
  for (int base = r_begin; base < r_end; base += 64) mine += __popcll(__ballot(hit_of(base + lane)));
  if (lane == 0) hits[row] = mine;
  __syncthreads();
  if (threadIdx.x == 0) {
    int sum = 0;
    for (int r = 0; r < kTileRows; ++r) sum += hits[r];
    list_base = sum > 0 ? atomicAdd(cursors, sum) : 0;
  }
  __syncthreads();
  int written = list_base, count = 0;
  for (int r = 0; r < kTileRows; ++r) {
    if (r < row) written += hits[r];
    count += hits[r];
  }
  const int begin = list_base, end = list_base + count;
  for (int base = r_begin; base < r_end && mine > 0; base += 64) {
    const bool hit = hit_of(base + lane);
    const unsigned long long mask = __ballot(hit);
    if (hit) tile_rois[written + __popcll(mask & ((1ull << lane) - 1ull))] = base + lane;
    written += __popcll(mask);
    mine -= __popcll(mask);
  }
  __syncthreads();   // the list is complete and visible to the whole workgroup

  // ---- the work lists of the sixteen rows ----
  auto table_of = [&](int roi) {
    return reinterpret_cast<const RowTapTable*>(lists + static_cast<long long>(roi) * ll.roi_stride +
                                                static_cast<long long>(ty) * ll.row_stride);
  };
  int total = 0;
  for (int base = begin; base < end; base += 64) {
    int c = 0;
    if (base + lane < end) c = table_of(tile_rois[base + lane])->index[row] >> 8;
    for (int off = 32; off > 0; off >>= 1) c += __shfl_xor(c, off);
    total += c;
  }
  // Lists are padded to a multiple of eight entries (one turn of the consumer's
  // double-buffered pipeline) plus four more that it prefetches but never uses.
  const int padded = (total + 7) & ~7;
  const int reserved = total > 0 ? padded + 4 : 0;
  if (lane == 0) row_total[row] = reserved;
  __syncthreads();
  if (threadIdx.x == 0) {
    int sum = 0;
    for (int r = 0; r < kTileRows; ++r) sum += row_total[r];
    tile_base = sum > 0 ? atomicAdd(cursors + 1, sum) : 0;
  }
  __syncthreads();
  int out = tile_base;
  for (int r = 0; r < row; ++r) out += row_total[r];
  if (lane == 0) ranges[tile * kTileRows + row] = WorkRange{out, padded};
  for (int base = begin; base < end; base += 64) {
    int c = 0, roi = 0, owner = 0;
    const RowTap* taps = nullptr;
    if (base + lane < end) {
      roi = tile_rois[base + lane];
      owner = boxes[roi].roi << 2;
      const RowTapTable* tb = table_of(roi);
      const unsigned idx = tb->index[row];
      c = idx >> 8;
      taps = tb->taps + (idx & 0xffu);
    }
    int incl = c;
    for (int off = 1; off < 64; off <<= 1) {
      const int up = __shfl_up(incl, off);
      if (lane >= off) incl += up;
    }
    WorkEntry* dst = entries + out + incl - c;
    for (int q = 0; q < c; ++q)
      dst[q] = WorkEntry{roi, taps[q].ph, taps[q].wy, (q > 0 ? 1 : 0) | (q == c - 1 ? 2 : 0) | owner};
    out += __shfl(incl, 63);
  }
  // padding: taps of weight zero that continue the last ROI and never end it
  if (lane < reserved - total) {
    const int item = tile_rois[end - 1];
    entries[out + lane] = WorkEntry{item, 0, 0.0f, 1 | (boxes[item].roi << 2)};
  }
}

}  // namespace roialign
