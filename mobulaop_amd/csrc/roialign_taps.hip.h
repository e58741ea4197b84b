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
//                           the sample count of the bin (the two samples of a
//                           bin that share a map row give it one tap, their
//                           weights added up): a 16-entry index
//                           (start | count << 8) followed by the taps, sorted
//                           by tile row, then by sample order
//   col list  of (roi, tx): one 16-byte ColPair per pooled column (padded to a
//                           multiple of 8 columns): its one or two sample columns
// These lists hold one or two sample points per bin and axis.  A larger sampling
// grid (a ratio above 2, or the adaptive ceil(bin size)) is merged instead: the
// gradient of a pixel is dy times (sum of the row weights its row gets from the
// bin's sample rows) times (sum of the column weights its column gets from
// the bin's sample columns), so a bin is described by one weight per row and one
// per column it touches.  Rows become row taps as before (one per pooled row and
// tile row, the weights of that pooled row's samples added up).  The columns of a
// bin are cut into windows of kWindowCells cells, window j of every pooled column
// together forming list item j of the ROI: its column list holds one 32-byte
// ColWindow per pooled column, and the tile owners add the items up like so many
// ROIs that share one dy.  `window_offsets_kernel` numbers the items.
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
  int row_stride;        // 16-byte units per (item, ty) row-tap table
  int col_stride;        // 16-byte units per (item, tx) column list
  long long roi_stride;  // units per item: ty*row_stride + tx*col_stride
  int pw_padded;         // PW rounded up to 8: pooled columns of a column list
  int windows;           // 1: merged weights (WindowRowTable, ColWindow), 0: sample lists (RowTapTable, ColPair)
};

constexpr int kWindowCells = 7;   // cells of a column window (with its header: eight dwords)

inline bool lists_in_windows(int S) { return S != 1 && S != 2; }

inline ListLayout make_list_layout(const TileGrid& tg, int PH, int PW, int S) {
  ListLayout l;
  l.ty = tg.ty; l.tx = tg.tx;
  l.pw_padded = (PW + 7) / 8 * 8;
  l.windows = lists_in_windows(S) ? 1 : 0;
  if (l.windows) {
    l.row_stride = 4 + kTileRows * PH / 2 + 1;   // 64-byte index, then at most one tap per tile row and pooled row
    l.col_stride = 2 * l.pw_padded;
  } else {
    l.row_stride = row_table_units(PH * (S == 1 ? 1 : 2));
    l.col_stride = l.pw_padded;
  }
  l.roi_stride = static_cast<long long>(l.ty) * l.row_stride + static_cast<long long>(l.tx) * l.col_stride;
  return l;
}

inline bool lists_supported(int PH, int PW, int S) {
  return PH * (S == 1 ? 1 : 2) <= kRowSlots && PW <= kMaxListPW;
}

// ---- merged weights (sampling grids of more than two points per bin and axis) ----

// Grids up to this many points per axis are merged (sample numbers are found from
// coordinates in fp32: beyond this the search margin of one sample would not do).
constexpr int kMergedGrid = 1 << 15;

// The cells the samples of pooled index p can touch along one axis, [*low, *low + *span):
// a superset, found from the first and the last sample coordinate alone (coordinates never
// decrease with the sample number), clamped the way the interpolation clamps them
// (opzoo/ROIAlign/bilinear.h:15-40).
__device__ __forceinline__ void bin_cells(float start, int p, float bin, int grid, int size, int* low,
                                          int* span) {
  const float c0 = sample_coord(start, p, bin, 0, grid), c1 = sample_coord(start, p, bin, grid - 1, grid);
  *low = 0; *span = 0;
  if (c1 < -1.0f || c0 > static_cast<float>(size)) return;   // every sample lies outside [-1, size]
  // (a coordinate that is not a number passes the reference's test; fmaxf/fminf then give the bound)
  const AxisSample a = axis_sample(fmaxf(c0, -1.0f), size), b = axis_sample(fminf(c1, static_cast<float>(size)), size);
  *low = a.low;
  *span = max(b.high - a.low + 1, 1);
}

// Sum of the weights that the valid samples of pooled index p give to `cell`
// (samples in sample order; a sample whose two cells coincide at the border counts once).
__device__ __forceinline__ float merged_weight(float start, int p, float bin, int grid, int size, int cell) {
  // samples that can reach the cell have coordinates in (cell - 1, cell + 1); the border
  // cells also take what is clamped onto them.  Sample numbers from coordinates, one to
  // spare on either side; every candidate is then evaluated exactly.
  const float lo = cell == 0 ? -1.0f : static_cast<float>(cell - 1);
  const float hi = cell == size - 1 ? static_cast<float>(size) : static_cast<float>(cell + 1);
  const float origin = start + static_cast<float>(p) * bin, step = bin / static_cast<float>(grid);
  const float fa = (lo - origin) / step - 0.5f, fb = (hi - origin) / step - 0.5f;
  int first = 0, last = grid;
  if (fabsf(fa) < 1.0e9f && fabsf(fb) < 1.0e9f) {   // (false for coordinates that are not numbers)
    first = max(0, static_cast<int>(floorf(fa)) - 1);
    last = min(grid, static_cast<int>(ceilf(fb)) + 2);
  }
  float w = 0.0f;
  for (int i = first; i < last; ++i) {
    const AxisSample a = axis_sample(sample_coord(start, p, bin, i, grid), size);
    if (!a.valid) continue;
    if (a.low == cell) w += a.h;
    if (a.high == cell && a.high != a.low) w += a.l;
  }
  return w;
}

// What the window items of one ROI need: their number (windows per pooled column), the
// tile columns they span and an upper bound of the row taps of one of them.
struct WindowCount { int windows; int tiles_x; int taps; };
__device__ __forceinline__ WindowCount count_windows(const RoiGeom& g, int PH, int PW, int H, int W, int tw) {
  WindowCount c{0, 0, 0};
  int widest = 0, clo = W, chi = -1;
  for (int pw = 0; pw < PW; ++pw) {
    int low, span;
    bin_cells(g.start_w, pw, g.bin_w, g.grid_w, W, &low, &span);
    if (span > 0) { widest = max(widest, span); clo = min(clo, low); chi = max(chi, low + span - 1); }
  }
  for (int ph = 0; ph < PH; ++ph) {
    int low, span;
    bin_cells(g.start_h, ph, g.bin_h, g.grid_h, H, &low, &span);
    c.taps += span;
  }
  if (widest == 0 || c.taps == 0) return WindowCount{0, 0, 0};
  c.windows = (widest + kWindowCells - 1) / kWindowCells;
  c.tiles_x = chi / tw - clo / tw + 1;
  return c;
}

// Window items, step 1: counts[r] = windows of ROI r (-1: its grid has more than kMergedGrid
// points along an axis), work[r] = an upper bound of the work entries of its items.
__global__ void __launch_bounds__(256)
window_counts_kernel(const float* __restrict__ rois, int R, float scale, int PH, int PW, int S, int H, int W,
                     int tw, int* __restrict__ counts, long long* __restrict__ work) {
  for (long long r = blockIdx.x * 256ll + threadIdx.x; r < R; r += 256ll * gridDim.x) {
    const RoiGeom g = roi_geometry(rois + r * 5, scale, PH, PW, S);
    if (g.grid_h > kMergedGrid || g.grid_w > kMergedGrid || g.grid_h < 1 || g.grid_w < 1) {
      counts[r] = -1;
      work[r] = 0;
      continue;
    }
    const WindowCount c = count_windows(g, PH, PW, H, W, tw);
    counts[r] = c.windows;
    work[r] = static_cast<long long>(c.windows) * c.tiles_x * c.taps;
  }
}

// Step 2: offsets[r] = number of the first window item of ROI r, offsets[R] = their total
// (offsets may be the array of counts: every thread reads its share before any writes);
// info[0] = the total, info[1] = 1 if some ROI's grid is too large to merge (the caller
// then takes another path), info[2] = an upper bound of the work entries of all items
// (saturating at 2^30).  One workgroup of 1024 threads.
__global__ void __launch_bounds__(1024)
window_offsets_kernel(const int* __restrict__ counts, const long long* __restrict__ work, int R,
                      int* __restrict__ offsets, int* __restrict__ info) {
  __shared__ int part[1024];
  __shared__ long long entries[1024];
  __shared__ int too_big;
  const int t = threadIdx.x, share = (R + 1023) / 1024;
  const int first = min(R, t * share), last = min(R, first + share);
  if (t == 0) too_big = 0;
  __syncthreads();
  int sum = 0;
  long long all = 0;
  for (int r = first; r < last; ++r) {
    const int c = counts[r];
    if (c < 0) too_big = 1;
    sum += max(c, 0);
    all += work[r];
  }
  part[t] = sum;
  entries[t] = all;
  __syncthreads();
  if (t == 0) {   // exclusive prefix over the threads
    int run = 0;
    long long total = 0;
    for (int i = 0; i < 1024; ++i) { const int c = part[i]; part[i] = run; run += c; total += entries[i]; }
    offsets[R] = run;
    info[0] = run;
    info[1] = too_big;
    info[2] = static_cast<int>(min(total, 1ll << 30));
  }
  __syncthreads();
  int at = part[t];
  for (int r = first; r < last; ++r) {
    const int c = max(counts[r], 0);
    offsets[r] = at;
    at += c;
  }
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
  const int* window_offsets;   // merged weights: the first item of every ROI (null: one item per ROI)
};

__device__ __forceinline__ void build_lists_body(unsigned block, const ListsArgs& a) {
  const float* __restrict__ rois = a.rois;
  const int items = a.items, PH = a.PH, PW = a.PW, S = a.S_given, H = a.H, W = a.W;
  const float scale = a.scale;
  const long long num_images = a.num_images;
  const TileGrid tg = a.tg;
  const ListLayout ll = a.ll;
  TileBox* __restrict__ boxes = a.boxes;
  int* __restrict__ cursors = a.cursors;
  AxisUnit* __restrict__ lists = a.lists;
  // the two bump pointers of build_tile_work_kernel, which runs after this one
  if (block == 0 && threadIdx.x < 2) cursors[threadIdx.x] = 0;
  const int item = static_cast<int>((block * 256u + threadIdx.x) >> 6);
  if (item >= items) return;
  const int lane = threadIdx.x & 63;
  const int roi = item;
  const RoiGeom g = roi_geometry(rois + static_cast<long long>(roi) * 5, scale, PH, PW, S);
  // one row sample and one column sample per lane
  const int iy = lane % S, ix_of_lane = lane % S;
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
      // Each unit lands on up to two tile rows; the taps are ordered by row, and within a row
      // the high parts (of the units whose low row is the row above) come before the low parts,
      // each in lane order: sample order, since sample coordinates never decrease with the lane.
      // That also makes the lanes of a row contiguous among the live ones, so a tap's place
      // follows from counts alone: lane r < 16 holds the numbers of row r.
      int row0 = u.w0 != 0.0f ? u.pos : -1, row1 = u.w1 != 0.0f ? u.pos + 1 : -1;
      float w0 = u.w0, w1 = u.w1;
      if (S == 2) {
        // Samples less than a pixel apart share rows: the second sample of a pooled row hands
        // the parts that land on a row of the first one to it (one tap, the weights added up:
        // a tap is a load of a row of dy for the tile owner).
        const int next_row0 = __shfl_down(row0, 1), next_row1 = __shfl_down(row1, 1);
        const float next_w0 = __shfl_down(w0, 1), next_w1 = __shfl_down(w1, 1);
        const int first_row0 = __shfl_up(row0, 1), first_row1 = __shfl_up(row1, 1);
        if ((lane & 1) == 0) {
          if (next_row0 >= 0 && next_row0 == row0) w0 += next_w0;
          if (next_row0 >= 0 && next_row0 == row1) w1 += next_w0;
          if (next_row1 >= 0 && next_row1 == row1) w1 += next_w1;
        } else {
          if (row0 >= 0 && (row0 == first_row0 || row0 == first_row1)) row0 = -1;
          if (row1 >= 0 && row1 == first_row1) row1 = -1;
        }
      }
      const unsigned long long below = (1ull << lane) - 1ull;
      const int before0 = __popcll(__ballot(row0 >= 0) & below), before1 = __popcll(__ballot(row1 >= 0) & below);
      int n0 = 0, n1 = 0;   // low and high parts on row `lane`
#pragma unroll
      for (int r = 0; r < kTileRows; ++r) {
        const int c0 = __popcll(__ballot(row0 == r)), c1 = __popcll(__ballot(row1 == r));
        if (lane == r) { n0 = c0; n1 = c1; }
      }
      int upto0 = n0, upto1 = n1;   // inclusive sums over the rows up to this lane's
      for (int off = 1; off < kTileRows; off <<= 1) {
        const int a0 = __shfl_up(upto0, off), a1 = __shfl_up(upto1, off);
        if (lane >= off) { upto0 += a0; upto1 += a1; }
      }
      // row r starts at (low parts before r) + (high parts before r); its high parts come first
      const int low_before = __shfl(upto0 - n0, max(row1, 0));    // low parts on rows above row1
      const int high_upto = __shfl(upto1, max(row0, 0));          // high parts on rows up to and including row0
      if (row1 >= 0) table->taps[low_before + before1] = RowTap{ph, w1};
      if (row0 >= 0) table->taps[high_upto + before0] = RowTap{ph, w0};
      if (lane < kTileRows)
        table->index[lane] = static_cast<unsigned short>((upto0 - n0 + upto1 - n1) | ((n0 + n1) << 8));
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

// Merged weights.  Row taps of one (item, tile row): per tile row start | count << 16, then the
// taps by tile row and pooled row: at most one per pair, ListLayout::row_stride leaves room for all.
struct alignas(16) WindowRowTable {
  unsigned index[kTileRows];
  RowTap taps[kTileRows * 32];
};
// The cells of one window of one pooled column inside one tile column band.
//   header  cell | turns_log << 16: `cell` is the cell of w[0] in a tile row whose cell 0 is a
//           dummy to the left of the tile (so the tile's first column is cell 1); the window is
//           shifted so that all seven cells lie in the tile, cells it does not reach weigh zero.
//           turns_log: log2 of the smallest power-of-two distance (in pooled columns, at most 8)
//           at which the windows of this item never share a cell their owner touches (w[0..3]
//           are added together, and so are w[4..6]: a group is skipped if all of it is zero).
//   w       weight of cells cell .. cell + 6
struct alignas(32) ColWindow { int header; float w[kWindowCells]; };
static_assert(sizeof(ColWindow) == 32, "eight dwords: the tile owners load one per lane");

// One wavefront per window item (ROI, j): the row taps of every tile row the ROI
// touches -- the same for all windows of a ROI -- and window j of every pooled column.
__device__ __forceinline__ void build_window_lists_body(unsigned block, const ListsArgs& a) {
  const int items = a.items, R = a.R, PH = a.PH, PW = a.PW, H = a.H, W = a.W;
  const TileGrid tg = a.tg;
  const ListLayout ll = a.ll;
  if (block == 0 && threadIdx.x < 2) a.cursors[threadIdx.x] = 0;
  const int item = static_cast<int>((block * 256u + threadIdx.x) >> 6);
  if (item >= items) return;
  const int lane = threadIdx.x & 63;
  int roi;
  {   // the ROI whose items include this one
    int lo = 0, hi = R;
    while (hi - lo > 1) {
      const int mid = (lo + hi) / 2;
      if (a.window_offsets[mid] <= item) lo = mid; else hi = mid;
    }
    roi = lo;
  }
  const int j = item - a.window_offsets[roi];
  const RoiGeom g = roi_geometry(a.rois + static_cast<long long>(roi) * 5, a.scale, PH, PW, a.S_given);
  // lane p < 32: pooled row p and pooled column p
  int rlow = 0, rspan = 0, clow = 0, cspan = 0;
  if (lane < PH) bin_cells(g.start_h, lane, g.bin_h, g.grid_h, H, &rlow, &rspan);
  if (lane < PW) bin_cells(g.start_w, lane, g.bin_w, g.grid_w, W, &clow, &cspan);
  const int wlow_mine = clow + kWindowCells * j;                    // first cell of the window
  const int wn_mine = max(0, min(kWindowCells, cspan - kWindowCells * j));   // its cells
  int row_lo, row_hi, col_lo, col_hi;
  {
    int rlo = rspan > 0 ? rlow : H, rhi = rspan > 0 ? rlow + rspan - 1 : -1;
    int clo = wn_mine > 0 ? wlow_mine : W, chi = wn_mine > 0 ? wlow_mine + wn_mine - 1 : -1;
    for (int off = 32; off > 0; off >>= 1) {
      rlo = min(rlo, __shfl_xor(rlo, off)); rhi = max(rhi, __shfl_xor(rhi, off));
      clo = min(clo, __shfl_xor(clo, off)); chi = max(chi, __shfl_xor(chi, off));
    }
    const bool image_ok = g.batch >= 0 && g.batch < a.num_images;
    const bool any = image_ok && rlo <= rhi && clo <= chi;
    row_lo = any ? rlo : 0; row_hi = any ? rhi : -1;
    col_lo = any ? clo : 0; col_hi = any ? chi : -1;
    const int ty0 = row_lo / tg.th, ty1 = any ? row_hi / tg.th : -1;
    const int tx0 = col_lo / tg.tw, tx1 = any ? col_hi / tg.tw : -1;
    if (lane == 0) a.boxes[item] = TileBox{any ? g.batch : -1, ty0 | (ty1 << 16), tx0 | (tx1 << 16), roi};
    if (!any) return;
  }
  AxisUnit* const base = a.lists + static_cast<long long>(item) * ll.roi_stride;
  const float inv_count = 1.0f / g.count;
  {
    // row taps: lane = tile row * 4 + k; the lane takes the pooled rows k, k + 4, ...
    const int r = lane >> 2, k4 = lane & 3;
    for (int ty = row_lo / tg.th; ty <= row_hi / tg.th; ++ty) {
      const int row = ty * tg.th + r;
      WindowRowTable* const table = reinterpret_cast<WindowRowTable*>(base + ty * ll.row_stride);
      float w[8];
      int at[8];
      int mine = 0;   // taps of this lane's tile row so far
#pragma unroll
      for (int q = 0; q < 8; ++q) {
        w[q] = 0.0f; at[q] = 0;
        if (4 * q < PH) {   // (the same for every lane)
          const int ph = 4 * q + k4;
          if (ph < PH && row < H)
            w[q] = merged_weight(g.start_h, ph, g.bin_h, g.grid_h, H, row) * inv_count;
          const unsigned nib = static_cast<unsigned>(__ballot(w[q] != 0.0f) >> (4 * r)) & 15u;
          at[q] = mine + __popc(nib & ((1u << k4) - 1u));
          mine += __popc(nib);
        }
      }
      int start = 0;
      for (int q = 0; q < kTileRows; ++q) {
        const int t = __shfl(mine, 4 * q);
        if (q < r) start += t;
      }
#pragma unroll
      for (int q = 0; q < 8; ++q)
        if (w[q] != 0.0f) table->taps[start + at[q]] = RowTap{4 * q + k4, w[q]};
      if (k4 == 0) table->index[r] = static_cast<unsigned>(start) | (static_cast<unsigned>(mine) << 16);
    }
  }
  {
    // windows: lane = pooled column (of eight) * 8 + dword of its ColWindow
    const int sub = lane >> 3, slot = (lane & 7) - 1;   // slot -1: the header
    int* const cols = reinterpret_cast<int*>(base + static_cast<long long>(ll.ty) * ll.row_stride);
    for (int tx = col_lo / tg.tw; tx <= col_hi / tg.tw; ++tx) {
      for (int pw0 = 0; pw0 < ll.pw_padded; pw0 += 8) {
        const int pw = pw0 + sub;
        // (every lane takes part in the exchange: the lane asked may be one whose column does not exist)
        const int wlow = __shfl(wlow_mine, pw & 63), wn_any = __shfl(wn_mine, pw & 63);
        const int wn = pw < PW ? wn_any : 0;
        // local cell of the window's first cell, and of w[0] once the window lies inside the tile
        const int s0 = wlow - tx * tg.tw;
        const int b = max(0, min(s0, tg.tw - kWindowCells));
        const int cell = tx * tg.tw + b + slot;           // the cell this lane weighs
        const int c = cell - wlow;                        // its place in the window
        float w = 0.0f;
        if (slot >= 0 && c >= 0 && c < wn && b + slot < tg.tw && cell < W)
          w = merged_weight(g.start_w, pw, g.bin_w, g.grid_w, W, cell);
        // The cells the tile owner reads and writes for this window (local): w[0..3] if one of
        // them is not zero, w[4..6] likewise -- cells of weight zero among them included.
        const unsigned live = static_cast<unsigned>(__ballot(w != 0.0f) >> (8 * sub)) & 0xffu;
        const bool head = (live & 0x1eu) != 0, tail = (live & 0xe0u) != 0;
        const int lo = head ? b : tail ? b + 4 : tg.tw;
        const int hi = tail ? b + kWindowCells - 1 : head ? b + 3 : -1;
        // smallest power-of-two distance at which no two windows of these eight columns share a cell
        int lg = 0;
#pragma unroll
        for (int d = 1; d <= 4; d <<= 1) {
          const int lo_d = __shfl_down(lo, 8 * d), hi_d = __shfl_down(hi, 8 * d);
          const bool clash = sub + d < 8 && lo <= hi && lo_d <= hi_d && lo_d <= hi && lo <= hi_d;
          if (__ballot(clash) != 0) lg = __builtin_ctz(d) + 1;
        }
        const int out = slot < 0 ? ((b + 1) | (lg << 16)) : __float_as_int(w);
        cols[(static_cast<long long>(tx) * ll.col_stride + 2 * pw) * 4 + (lane & 7)] = out;
      }
    }
  }
}

__global__ void __launch_bounds__(256) build_lists_kernel(ListsArgs a) {
  if (a.window_offsets != nullptr) build_window_lists_body(blockIdx.x, a);
  else build_lists_body(blockIdx.x, a);
}


// One wavefront's share of a tile: the (ROI, pooled row, weight) taps that land
// on one tile row, in ROI order, so that the owner of that row streams through
// them without looking anything up.
struct alignas(16) WorkEntry {
  int roi;     // the list item (its column pairs are read from its lists)
  int ph;
  float wy;
  int flags;   // bit 0: continues the previous entry's item; bit 1: last entry of its item;
               // bits 2..: the ROI whose dy the entry reads (the item itself, or the ROI it is a window of)
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
// WIN: the items are windows of merged weights (WindowRowTable) rather than sample lists.
constexpr int kTileListCap = 4096;   // items of one tile that LDS holds (longer lists go through memory)

template <bool WIN>
__global__ void __launch_bounds__(kTileRows * 64)
build_tile_work_kernel(const TileBox* __restrict__ boxes, int R, int* __restrict__ tile_rois,
                       const AxisUnit* __restrict__ lists, TileGrid tg, ListLayout ll,
                       int* __restrict__ cursors, WorkRange* __restrict__ ranges,
                       WorkEntry* __restrict__ entries) {
  __shared__ int hits[kTileRows];
  __shared__ int row_total[kTileRows];
  __shared__ int list_base, tile_base;
  // the tile's items and the ROIs whose dy they read (<< 2, as the entries hold them), in item
  // order: in LDS, so that the wavefronts below need not wait for memory to see the list
  __shared__ int item_s[kTileListCap];
  __shared__ int owner_s[kTileListCap];
  const long long tile = blockIdx.x;
  const int lane = threadIdx.x & 63, row = threadIdx.x >> 6;
  const int image = static_cast<int>(tile / tg.per_image);
  const int t = static_cast<int>(tile % tg.per_image);
  const int ty = t / tg.tx, tx = t % tg.tx;

  // ---- the tile's item list ----
  const int share = ((R + kTileRows * 64 - 1) / (kTileRows * 64)) * 64;
  const int r_begin = row * share, r_end = min(R, r_begin + share);
  auto hit_of = [&](int r, int* owner) {
    if (r >= r_end) return false;
    const TileBox b = boxes[r];
    *owner = b.roi << 2;
    return b.batch == image && ty >= (b.ty & 0xffff) && ty <= (b.ty >> 16) && tx >= (b.tx & 0xffff) &&
           tx <= (b.tx >> 16);
  };
  // (what the first kKept chunks of 64 boxes of the wavefront's share gave is kept for the second
  // walk: with up to 4096 boxes in all that is every chunk, and the boxes are read once)
  constexpr int kKept = 4;
  bool kept_hit[kKept];
  int kept_owner[kKept];
  int mine = 0;
#pragma unroll
  for (int k = 0; k < kKept; ++k) {
    kept_owner[k] = 0;
    kept_hit[k] = hit_of(r_begin + 64 * k + lane, &kept_owner[k]);
    mine += __popcll(__ballot(kept_hit[k]));
  }
  for (int base = r_begin + 64 * kKept; base < r_end; base += 64) {
    int unused_owner = 0;
    mine += __popcll(__ballot(hit_of(base + lane, &unused_owner)));
  }
  if (lane == 0) hits[row] = mine;
  __syncthreads();
  int written = 0, count = 0;
  for (int r = 0; r < kTileRows; ++r) {
    if (r < row) written += hits[r];
    count += hits[r];
  }
  const bool in_lds = count <= kTileListCap;   // (the same for the whole workgroup)
  if (!in_lds) {
    if (threadIdx.x == 0) list_base = atomicAdd(cursors, count);
    __syncthreads();
  }
  int* const long_list = tile_rois + (in_lds ? 0 : list_base);
  auto put = [&](int base, bool hit, int owner) {
    const unsigned long long mask = __ballot(hit);
    if (hit) {
      const int at = written + __popcll(mask & ((1ull << lane) - 1ull));
      if (in_lds) { item_s[at] = base + lane; owner_s[at] = owner; }
      else long_list[at] = base + lane;
    }
    written += __popcll(mask);
    mine -= __popcll(mask);
  };
#pragma unroll
  for (int k = 0; k < kKept; ++k)
    if (mine > 0) put(r_begin + 64 * k, kept_hit[k], kept_owner[k]);
  for (int base = r_begin + 64 * kKept; base < r_end && mine > 0; base += 64) {
    int owner = 0;
    const bool hit = hit_of(base + lane, &owner);
    put(base, hit, owner);
  }
  __syncthreads();   // the list is complete and visible to the whole workgroup
  auto item_at = [&](int i) { return in_lds ? item_s[i] : long_list[i]; };
  auto owner_at = [&](int i, int item) { return in_lds ? owner_s[i] : boxes[item].roi << 2; };

  // ---- the work lists of the sixteen rows ----
  // taps of list item `roi` on this wavefront's tile row: where they start, how many
  auto taps_of = [&](int roi, const RowTap** taps) {
    const AxisUnit* const table = lists + static_cast<long long>(roi) * ll.roi_stride +
                                  static_cast<long long>(ty) * ll.row_stride;
    if (WIN) {
      const WindowRowTable* const tb = reinterpret_cast<const WindowRowTable*>(table);
      const unsigned idx = tb->index[row];
      *taps = tb->taps + (idx & 0xffffu);
      return static_cast<int>(idx >> 16);
    }
    const RowTapTable* const tb = reinterpret_cast<const RowTapTable*>(table);
    const unsigned idx = tb->index[row];
    *taps = tb->taps + (idx & 0xffu);
    return static_cast<int>(idx >> 8);
  };
  // (what the first 64 items gave is kept for the second walk: most tiles have no more)
  int total = 0, first_c = 0, first_item = 0;
  const RowTap* first_taps = nullptr;
  for (int base = 0; base < count; base += 64) {
    int c = 0, item = 0;
    const RowTap* taps = nullptr;
    if (base + lane < count) {
      item = item_at(base + lane);
      c = taps_of(item, &taps);
    }
    if (base == 0) { first_c = c; first_item = item; first_taps = taps; }
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
  for (int base = 0; base < count; base += 64) {
    int c = first_c, roi = first_item, owner = 0;
    const RowTap* taps = first_taps;
    if (base > 0) {
      c = 0; roi = 0; taps = nullptr;
      if (base + lane < count) {
        roi = item_at(base + lane);
        c = taps_of(roi, &taps);
      }
    }
    if (base + lane < count) owner = owner_at(base + lane, roi);
    int incl = c;
    for (int off = 1; off < 64; off <<= 1) {
      const int up = __shfl_up(incl, off);
      if (lane >= off) incl += up;
    }
    WorkEntry* dst = entries + out + incl - c;
    // (four taps at a time: their loads go out together instead of one after the other)
    for (int q0 = 0; q0 < c; q0 += 4) {
      RowTap four[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) four[k] = taps[min(q0 + k, c - 1)];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const int q = q0 + k;
        if (q < c) dst[q] = WorkEntry{roi, four[k].ph, four[k].wy, (q > 0 ? 1 : 0) | (q == c - 1 ? 2 : 0) | owner};
      }
    }
    out += __shfl(incl, 63);
  }
  // padding: taps of weight zero that continue the last ROI and never end it
  if (lane < reserved - total) {
    const int item = item_at(count - 1);
    entries[out + lane] = WorkEntry{item, 0, 0.0f, 1 | owner_at(count - 1, item)};
  }
}

}  // namespace roialign
