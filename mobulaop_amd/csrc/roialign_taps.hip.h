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
//   col list  of (roi, tx): PW*2 units, slot = pw*2 + ix
// Only fixed sampling grids with S <= 2 use this path.
// Sample coordinates come from roialign_geometry.h (reference operation order).
#pragma once
#include "roialign_tiles.hip.h"

namespace roialign {

// `bin` is the pooled row/column; `pos` the local position of the low corner.
struct alignas(16) AxisUnit { int bin; int pos; float w0, w1; };

// Bit 16 of `bin` of the first column unit of a pooled column: the cells of
// its two units overlap.  Bit 17: this pooled column's cells overlap the next
// pooled column's.
// Bits 18..20 of `bin` of slot 0 of a column list: log2 of the smallest power
// of two s such that units k and k+s of the list never share a cell.  Units
// k, k+s, k+2s, ... can then be processed together (loads before stores).
constexpr int kPairOverlaps = 1 << 16;
constexpr int kNextOverlaps = 1 << 17;
constexpr int kStrideShift = 18;
constexpr int kStrideMask = 7;

constexpr int kRowSlots = 32;   // PH * S <= 32 sample rows per ROI
constexpr int kMaxListPW = 16;  // PW <= 16, S <= 2
constexpr int kTileRows = 16;   // rows of a tile (fixed by the row-tap index)

struct RowTap { int ph; float wy; };
// Row taps of one (roi, tile row): 32-byte index + up to 2*kRowSlots taps.
struct alignas(16) RowTapTable {
  unsigned short index[kTileRows];   // start | count << 8, per tile row
  RowTap taps[2 * kRowSlots];
};
constexpr int kRowTableUnits = sizeof(RowTapTable) / 16;   // in 16-byte units

struct ListLayout {
  int ty, tx;            // tiles per image
  int row_stride;        // 16-byte units per (roi, ty) row-tap table
  int col_stride;        // units per (roi, tx) column list = 2 * PW
  long long roi_stride;  // units per ROI: ty*row_stride + tx*col_stride
};

inline ListLayout make_list_layout(const TileGrid& tg, int PW) {
  ListLayout l;
  l.ty = tg.ty; l.tx = tg.tx;
  l.row_stride = kRowTableUnits;
  l.col_stride = 2 * PW;
  l.roi_stride = static_cast<long long>(l.ty) * l.row_stride + static_cast<long long>(l.tx) * l.col_stride;
  return l;
}

inline bool lists_supported(int PH, int PW, int S) {
  return S >= 1 && S <= 2 && PH * S <= kRowSlots && PW <= kMaxListPW;
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
__global__ void __launch_bounds__(256)
build_lists_kernel(const RoiRec* __restrict__ recs, int R, int PH, int PW, int S, int H, int W,
                   TileGrid tg, ListLayout ll, AxisUnit* __restrict__ lists) {
  const int roi = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
  if (roi >= R) return;
  const int lane = threadIdx.x & 63;
  const RoiRec rec = recs[roi];
  if (rec.row_lo > rec.row_hi) return;
  AxisUnit* const base = lists + static_cast<long long>(roi) * ll.roi_stride;
  const float inv_count = 1.0f / rec.count;
  {
    const int ph = lane / S, iy = lane - ph * S;
    AxisSample a = axis_sample(sample_coord(rec.start_h, ph, rec.bin_h, iy, S), H);
    a.valid = a.valid && lane < PH * S;
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
    const int pw = lane / S, ix = lane - pw * S;
    const bool real = lane < PW * S;
    AxisSample a = axis_sample(sample_coord(rec.start_w, pw, rec.bin_w, ix, S), W);
    a.valid = a.valid && real;
    AxisUnit* const cols = base + static_cast<long long>(ll.ty) * ll.row_stride;
    for (int tx = rec.col_lo / tg.tw; tx <= rec.col_hi / tg.tw; ++tx) {
      AxisUnit u = clip_unit(pw, a, tx * tg.tw, tg.tw, 1.0f);
      const bool live = u.w0 != 0.0f || u.w1 != 0.0f;
      // neighbours: the other unit of this pooled column, the units of the next one
      const int pos_next = __shfl_down(u.pos, 1), pos_next2 = __shfl_down(u.pos, 2);
      const bool live_next = __shfl_down(live ? 1 : 0, 1) != 0;
      const bool live_next2 = __shfl_down(live ? 1 : 0, 2) != 0;
      auto near = [](int p, int q) { return p - q >= -1 && p - q <= 1; };
      if (S == 2) {
        // lane = 2*pw + ix.  Flags live in the ix == 0 unit.
        const bool pair = live && live_next && near(u.pos, pos_next);
        // this column's units vs the next column's two units
        const int pos_next3 = __shfl_down(u.pos, 3);
        const bool live_next3 = __shfl_down(live ? 1 : 0, 3) != 0;
        bool next = false;
        if (ix == 0) {
          next = (live && live_next2 && near(u.pos, pos_next2)) ||
                 (live && live_next3 && near(u.pos, pos_next3)) ||
                 (live_next && live_next2 && near(pos_next, pos_next2)) ||
                 (live_next && live_next3 && near(pos_next, pos_next3));
          if (pair) u.bin |= kPairOverlaps;
          if (next) u.bin |= kNextOverlaps;
        }
        {
          // smallest power-of-two stride at which no two live units share a cell
          int lg = 0;
#pragma unroll
          for (int d = 1; d <= 16; d <<= 1) {
            const int pos_d = __shfl_down(u.pos, d);
            const bool live_d = __shfl_down(live ? 1 : 0, d) != 0;
            const bool clash = live && live_d && lane + d < PW * S && near(u.pos, pos_d);
            if (__ballot(clash) != 0) lg = (d == 16) ? 5 : __builtin_ctz(d) + 1;
          }
          if (lane == 0) u.bin |= lg << kStrideShift;
        }
        if (real) cols[tx * ll.col_stride + lane] = u;
      } else {
        // S == 1: slot 2*pw holds the unit, slot 2*pw + 1 is dead
        const bool next = live && live_next && near(u.pos, pos_next);
        if (next) u.bin |= kNextOverlaps;
        {
          int lg = 0;
#pragma unroll
          for (int d = 1; d <= 16; d <<= 1) {
            const int pos_d = __shfl_down(u.pos, d);
            const bool live_d = __shfl_down(live ? 1 : 0, d) != 0;
            const bool clash = live && live_d && lane + d < PW && near(u.pos, pos_d);
            // slots are 2 apart for S == 1
            if (__ballot(clash) != 0) lg = (d == 16) ? 5 : __builtin_ctz(d) + 2;
          }
          if (lane == 0) u.bin |= min(lg, 5) << kStrideShift;
        }
        if (real) {
          cols[tx * ll.col_stride + 2 * lane] = u;
          cols[tx * ll.col_stride + 2 * lane + 1] = AxisUnit{pw, tg.tw, 0.0f, 0.0f};
        }
      }
    }
  }
}


// One wavefront's share of a tile: the (ROI, pooled row, weight) taps that land
// on one tile row, in ROI order, so that the owner of that row streams through
// them without looking anything up.
struct alignas(16) WorkEntry {
  int roi;
  int ph;
  float wy;
  int flags;   // bit 0: continues the previous entry's ROI; bit 1: last entry of its ROI
};
struct WorkRange { int begin; int count; };

// One workgroup per tile, one wavefront per tile row: lane j looks at ROI j of
// the tile's list, takes its taps for this row from the row-tap table, and all
// lanes append theirs in list order.  Space for the tile's sixteen lists comes
// from one bump-pointer allocation per tile (*cursor).
__global__ void __launch_bounds__(kTileRows * 64)
build_worklists_kernel(const int* __restrict__ tile_offset, const int* __restrict__ tile_rois,
                       const AxisUnit* __restrict__ lists, TileGrid tg, ListLayout ll,
                       int* __restrict__ cursor, WorkRange* __restrict__ ranges,
                       WorkEntry* __restrict__ entries) {
  __shared__ int row_total[kTileRows];
  __shared__ int tile_base;
  const long long tile = blockIdx.x;
  const int lane = threadIdx.x & 63, row = threadIdx.x >> 6;
  const int ty = static_cast<int>(tile % tg.per_image) / tg.tx;
  const int begin = tile_offset[tile], end = tile_offset[tile + 1];
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
  if (lane == 0) row_total[row] = total;
  __syncthreads();
  if (threadIdx.x == 0) {
    int sum = 0;
    for (int r = 0; r < kTileRows; ++r) sum += row_total[r];
    tile_base = sum > 0 ? atomicAdd(cursor, sum) : 0;
  }
  __syncthreads();
  int out = tile_base;
  for (int r = 0; r < row; ++r) out += row_total[r];
  if (lane == 0) ranges[tile * kTileRows + row] = WorkRange{out, total};
  for (int base = begin; base < end; base += 64) {
    int c = 0, roi = 0;
    const RowTap* taps = nullptr;
    if (base + lane < end) {
      roi = tile_rois[base + lane];
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
      dst[q] = WorkEntry{roi, taps[q].ph, taps[q].wy, (q > 0 ? 1 : 0) | (q == c - 1 ? 2 : 0)};
    out += __shfl(incl, 63);
  }
}

}  // namespace roialign
