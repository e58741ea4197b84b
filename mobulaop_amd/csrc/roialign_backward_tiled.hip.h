// Tiled ROIAlign backward: every (tile, channel block) of dx is owned by one
// workgroup, accumulated in LDS and written to memory exactly once -- no global
// atomics and no separate zero-fill pass.
//
// LDS layout: acc[c][1 + row*34 + col], channel stride odd, so the 64 lanes of
// a wavefront (one channel each) always hit 64 different banks; weights and
// pixel positions are the same for all lanes.  Each row has a dummy cell on
// either side (columns -1 and 32), which lets every column unit be a two-cell
// read-modify-write even at the tile border and gives dead units (weights 0,
// position 32) somewhere harmless to go.
// LDS float atomics are not used (they run at a few lanes per clock on this
// part): each of the sixteen wavefronts owns one tile row instead, and there
// is no barrier between the initial clear and the final store -- every
// wavefront walks the tile's ROI list on its own.
//
// Everything uniform stays off the vector ALU, which is what bounds the inner
// loop: the column units of a ROI come through scalar loads (they are written
// once per (ROI, tile column) by the pre-pass, see roialign_taps.hip.h), loop
// control and liveness tests run on scalar registers.  Per (row tap, pooled
// column) the vector work is one multiply plus, per unit, one address add and
// two fused multiply-adds around a two-cell LDS read/write.
//
// dy is read straight from memory, one channel per lane: the PW floats of one
// pooled row are contiguous (28 bytes for PW = 7), the other rows of the same
// 64-channel block are fetched by the wavefronts that own the rows they land
// on, so the lines are reused out of L1/L2 while the ROI is being processed.
//
// Arithmetic per cell: dx += (dy * (wy / count)) * wx, against the reference's
// (dy * (wy*wx)) / count (opzoo/ROIAlign/ROIAlign.cpp:143-157): same samples
// and weights, rounding differs in the last bits.
#pragma once
#include "roialign_taps.hip.h"

namespace roialign {

struct BwdTile {
  static constexpr int TH = 16, TW = 32, CH = 64;
  static constexpr int NW = TH;                  // one wavefront per tile row
  static constexpr int NT = NW * 64;
  static constexpr int RS = TW + 2;              // row stride: dummy cell, 32 columns, dummy cell
  static constexpr int CS = TH * RS + 1;         // channel stride, odd
  static constexpr int PWB = 8;                  // pooled columns per dy register block
  static constexpr int UB = 4;                   // pooled columns per unit block (8 units)
  static constexpr int G = 4;                    // work entries per group
  static_assert(CS % 2 == 1 && TH == kTileRows, "layout");
};

// Host-side gate: the tiled backward kernel takes fixed sampling grids with
// S <= 2 whose lists fit the pre-pass layout.
inline bool backward_tiled_supports(int PH, int PW, int S) {
  return lists_supported(PH, PW, S) && PW <= BwdTile::PWB;
}

typedef float float4u __attribute__((ext_vector_type(4), aligned(4)));
typedef float float2u __attribute__((ext_vector_type(2), aligned(4)));

// The eight (PW real, rest zero) dy values of one pooled row for this lane's channel.
__device__ __forceinline__ void load_dy_row(const float* __restrict__ p, float (&d)[8]) {
  const float4 a = *reinterpret_cast<const float4*>(p);
  const float4 b = *reinterpret_cast<const float4*>(p + 4);
  d[0] = a.x; d[1] = a.y; d[2] = a.z; d[3] = a.w; d[4] = b.x; d[5] = b.y; d[6] = b.z; d[7] = b.w;
}

// Eight column units (four pooled columns) held in scalar registers: two
// 64-byte scalar loads instead of one small load per field.
typedef int int16v __attribute__((ext_vector_type(16)));
struct UnitBlock {
  int16v lo, hi;
  __device__ __forceinline__ int pos(int k) const { return k < 4 ? lo[4 * (k & 3) + 1] : hi[4 * (k & 3) + 1]; }
  __device__ __forceinline__ float w0(int k) const {
    return __int_as_float(k < 4 ? lo[4 * (k & 3) + 2] : hi[4 * (k & 3) + 2]);
  }
  __device__ __forceinline__ float w1(int k) const {
    return __int_as_float(k < 4 ? lo[4 * (k & 3) + 3] : hi[4 * (k & 3) + 3]);
  }
};

// Eight column units fetched with broadcast LDS reads (same address in every
// lane): the fields are uniform but live in vector registers.
struct LdsUnitBlock {
  AxisUnit u[8];
  __device__ __forceinline__ int pos(int k) const { return u[k].pos; }
  __device__ __forceinline__ float w0(int k) const { return u[k].w0; }
  __device__ __forceinline__ float w1(int k) const { return u[k].w1; }
};

__device__ __forceinline__ LdsUnitBlock load_unit_block_lds(const AxisUnit* u) {
  LdsUnitBlock b;
#pragma unroll
  for (int k = 0; k < 8; ++k) b.u[k] = u[k];
  return b;
}

__device__ __forceinline__ UnitBlock load_unit_block(const AxisUnit* __restrict__ u) {
  const int16v* p = reinterpret_cast<const int16v*>(u);
  UnitBlock b;
  b.lo = p[0];
  b.hi = p[1];
  return b;
}

// row[pos] += g*w0, row[pos+1] += g*w1 for the units of a block; unit k belongs
// to pooled column k/2 of the block and uses g[G0 + k/2].  Only the first NV
// pooled columns of the block exist (the rest of the 128 bytes belongs to
// whatever follows the list).  Units k, k+ST, k+2*ST, ... never share a cell
// (or are dead and sit on dummy cells), so each such group issues all its
// loads before its first store -- one LDS round trip per group.  LDS accesses
// of a wavefront complete in program order, so the next group sees the stores.
template <int G0, int NV, int ST, typename Block>
__device__ __forceinline__ void add_block_n(float* row, const float (&g)[8], const Block& u) {
#pragma unroll
  for (int p = 0; p < ST && p < 2 * NV; ++p) {
    float x[8], y[8];
#pragma unroll
    for (int k = p; k < 2 * NV; k += ST) { x[k] = row[u.pos(k)]; y[k] = row[u.pos(k) + 1]; }
#pragma unroll
    for (int k = p; k < 2 * NV; k += ST) {
      row[u.pos(k)] = fmaf(g[G0 + (k >> 1)], u.w0(k), x[k]);
      row[u.pos(k) + 1] = fmaf(g[G0 + (k >> 1)], u.w1(k), y[k]);
    }
  }
}

template <int G0, int NV, typename Block>
__device__ __forceinline__ void add_block_s(float* row, const float (&g)[8], const Block& u, int lg) {
  switch (lg) {
    case 0: add_block_n<G0, NV, 1>(row, g, u); break;
    case 1: add_block_n<G0, NV, 2>(row, g, u); break;
    case 2: add_block_n<G0, NV, 4>(row, g, u); break;
    default: add_block_n<G0, NV, 8>(row, g, u); break;
  }
}

template <int G0, typename Block>
__device__ __forceinline__ void add_block(float* row, const float (&g)[8], const Block& u,
                                          int nv, int lg) {
  switch (nv) {
    case 4: add_block_s<G0, 4>(row, g, u, lg); break;
    case 3: add_block_s<G0, 3>(row, g, u, lg); break;
    case 2: add_block_s<G0, 2>(row, g, u, lg); break;
    default: add_block_s<G0, 1>(row, g, u, lg); break;
  }
}

// dy[r][c][ph][pw] -> dyt[r][ph][c][8] (pw padded to 8 with zeros, requires
// PW <= 8): the form in which one lane per channel can fetch the PW values of
// a pooled row with two 16-byte loads while the wavefront reads one
// contiguous 2 KB segment.  One workgroup per (ROI, 64 channels): the 64*PH*PW
// input words are contiguous, and so are the 64*8 output words of each pooled
// row.
__global__ void __launch_bounds__(256)
transpose_dy_kernel(const float* __restrict__ dy, float* __restrict__ dyt, int C, int PH, int PW,
                    int cblocks) {
  extern __shared__ float tbuf[];   // [64][PH*PW]
  const int r = blockIdx.x / cblocks, cb = blockIdx.x % cblocks;
  const int c0 = cb * 64, nch = min(64, C - c0);
  const int bins = PH * PW;
  const float* src = dy + (static_cast<size_t>(r) * C + c0) * bins;
  const int n_in = nch * bins;
  if ((reinterpret_cast<size_t>(src) & 15) == 0) {
    for (int i = threadIdx.x * 4; i < n_in; i += 1024) {
      if (i + 3 < n_in) {
        const float4 v = *reinterpret_cast<const float4*>(src + i);
        tbuf[i] = v.x; tbuf[i + 1] = v.y; tbuf[i + 2] = v.z; tbuf[i + 3] = v.w;
      } else {
        for (int k = i; k < n_in; ++k) tbuf[k] = src[k];
      }
    }
  } else {
    for (int i = threadIdx.x; i < n_in; i += 256) tbuf[i] = src[i];
  }
  __syncthreads();
  // one float4 per thread and step: element e = ((ph * 64) + c) * 8 + k0, k0 in {0, 4}
  for (int q = threadIdx.x; q < PH * 64 * 2; q += 256) {
    const int k0 = (q & 1) * 4, c = (q >> 1) & 63, ph = q >> 7;
    if (c >= nch) continue;
    const float* in = tbuf + c * bins + ph * PW;
    float4 v;
    v.x = k0 + 0 < PW ? in[k0 + 0] : 0.0f;
    v.y = k0 + 1 < PW ? in[k0 + 1] : 0.0f;
    v.z = k0 + 2 < PW ? in[k0 + 2] : 0.0f;
    v.w = k0 + 3 < PW ? in[k0 + 3] : 0.0f;
    *reinterpret_cast<float4*>(dyt + ((static_cast<size_t>(r) * PH + ph) * C + c0 + c) * 8 + k0) = v;
  }
}

__global__ void __launch_bounds__(BwdTile::NT)
backward_tiled_kernel(const float* __restrict__ dyt, float* __restrict__ dx,
                      const int* __restrict__ tile_offset, const WorkRange* __restrict__ ranges,
                      const WorkEntry* __restrict__ entries, const AxisUnit* __restrict__ lists,
                      TileGrid tg, ListLayout ll, int C, int H, int W, int PH, int PW, int cblocks,
                      long long num_jobs, int assign) {
  using K = BwdTile;
  __shared__ float acc[K::CH * K::CS];
  __shared__ AxisUnit ubuf[K::NW][K::G * 16];   // per wavefront: the column lists of one group

  // XCD-aware job order: consecutive workgroup ids go round-robin to the 8
  // XCDs, so give each XCD a contiguous run of logical jobs (neighbouring
  // tiles of one image and channel block share dy blocks through that XCD's L2).
  const long long per_xcd = gridDim.x / 8;
  const long long job = static_cast<long long>(blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
  if (job >= num_jobs) return;
  const int t_in_img = static_cast<int>(job % tg.per_image);
  const int cb = static_cast<int>((job / tg.per_image) % cblocks);
  const int n = static_cast<int>(job / (static_cast<long long>(tg.per_image) * cblocks));
  const long long tile = static_cast<long long>(n) * tg.per_image + t_in_img;
  const int ty = t_in_img / tg.tx, tx = t_in_img % tg.tx;
  const int r0 = ty * K::TH, q0 = tx * K::TW;
  const int c0 = cb * K::CH;
  const int nch = min(K::CH, C - c0);
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // = the tile row this wavefront owns
  const int rows = min(K::TH, H - r0), cols = min(K::TW, W - q0);
  float* const plane0 = dx + (static_cast<size_t>(n) * C + c0) * H * W;

  const int list_begin = tile_offset[tile], list_end = tile_offset[tile + 1];
  if (list_begin == list_end) {
    if (assign) {
      for (int i = tid; i < nch * K::TH * K::TW; i += K::NT) {
        const int col = i % K::TW, row = (i / K::TW) % K::TH, c = i / (K::TW * K::TH);
        if (row < rows && col < cols)
          plane0[static_cast<size_t>(c) * H * W + static_cast<size_t>(r0 + row) * W + q0 + col] = 0.0f;
      }
    }
    return;
  }

  for (int i = tid; i < K::CH * K::CS; i += K::NT) acc[i] = 0.0f;
  __syncthreads();

  const int ch = min(lane, nch - 1);                 // lanes past the last channel shadow it
  float* const row = acc + ch * K::CS + 1 + wave * K::RS;
  const float* const dy_lane = dyt + static_cast<size_t>(c0 + ch) * 8;   // dyt[r][ph][c][8]
  const size_t roi_dy_stride = static_cast<size_t>(PH) * C * 8, ph_dy_stride = static_cast<size_t>(C) * 8;
  const AxisUnit* const col_lists =
      lists + static_cast<long long>(ll.ty) * ll.row_stride + static_cast<long long>(tx) * ll.col_stride;

  // Each wavefront streams through the work list of its tile row: entries
  // (ROI, pooled row, weight) in ROI order, four at a time.  Software pipeline:
  //   entries of group k+2   scalar load in flight
  //   group k+1              dy rows (two 16-byte loads per entry and lane) and the
  //                          four column lists (one 16-byte load per lane) in flight
  //   group k                fold the taps of a ROI into g[pw]; at its last entry
  //                          walk the ROI's column units (staged through this
  //                          wavefront's private LDS slot and read back as broadcasts)
  if (wave < rows) {
    const WorkRange wr = ranges[tile * kTileRows + wave];
    const int n = wr.count;
    const int16v* const wl = reinterpret_cast<const int16v*>(entries + wr.begin);
    AxisUnit* const my_units = ubuf[wave];
    const int lane_list = lane >> 4, lane_unit = lane & 15;

    auto issue = [&](const int16v& e, int e0, float (&d)[K::G][8], AxisUnit& uv) {
      int my_roi = e[0];
#pragma unroll
      for (int j = 0; j < K::G; ++j) {
        if (e0 + j < n) load_dy_row(dy_lane + e[4 * j] * roi_dy_stride + e[4 * j + 1] * ph_dy_stride, d[j]);
        my_roi = (lane_list == j && e0 + j < n) ? e[4 * j] : my_roi;
      }
      uv = col_lists[static_cast<long long>(my_roi) * ll.roi_stride + lane_unit];
    };
    float g[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    auto process = [&](const int16v& e, int e0, const float (&d)[K::G][8], const AxisUnit& uv) {
      my_units[lane] = uv;
#pragma unroll
      for (int j = 0; j < K::G; ++j) {
        if (e0 + j < n) {
          const float wy = __int_as_float(e[4 * j + 2]);
          const int fl = e[4 * j + 3];
          if ((fl & 1) == 0) {
#pragma unroll
            for (int k = 0; k < 8; ++k) g[k] = d[j][k] * wy;
          } else {
#pragma unroll
            for (int k = 0; k < 8; ++k) g[k] = fmaf(d[j][k], wy, g[k]);
          }
          if ((fl & 2) != 0 && lane < nch) {
            const AxisUnit* const ul = my_units + 16 * j;
            const LdsUnitBlock ub_a = load_unit_block_lds(ul);
            const int lg = (__builtin_amdgcn_readfirstlane(ub_a.u[0].bin) >> kStrideShift) & kStrideMask;
            add_block<0>(row, g, ub_a, min(PW, K::UB), lg);
            if (PW > K::UB) add_block<4>(row, g, load_unit_block_lds(ul + 8), PW - K::UB, lg);
          }
        }
      }
    };

    if (n > 0) {
      int16v e_cur = wl[0], e_nx = wl[1], e_n2;
      float d_a[K::G][8], d_b[K::G][8];
      AxisUnit uv_a, uv_b;
      issue(e_cur, 0, d_a, uv_a);
      for (int e0 = 0; e0 < n; e0 += 2 * K::G) {
        // group at e0 lives in set a, group at e0 + G in set b
        e_n2 = wl[(e0 >> 2) + 2];
        if (e0 + K::G < n) issue(e_nx, e0 + K::G, d_b, uv_b);
        process(e_cur, e0, d_a, uv_a);
        e_cur = e_nx; e_nx = e_n2;
        if (e0 + K::G < n) {
          e_n2 = wl[(e0 >> 2) + 3];
          if (e0 + 2 * K::G < n) issue(e_nx, e0 + 2 * K::G, d_a, uv_a);
          process(e_cur, e0 + K::G, d_b, uv_b);
          e_cur = e_nx; e_nx = e_n2;
        }
      }
    }
  }
  __syncthreads();

  // Owner writes its tile: two 32-pixel rows per wavefront access.
  for (int i = tid; i < nch * K::TH * K::TW; i += K::NT) {
    const int col = i % K::TW, row_i = (i / K::TW) % K::TH, c = i / (K::TW * K::TH);
    if (row_i < rows && col < cols) {
      float* p = plane0 + static_cast<size_t>(c) * H * W + static_cast<size_t>(r0 + row_i) * W + q0 + col;
      const float v = acc[c * K::CS + 1 + row_i * K::RS + col];
      *p = assign ? v : *p + v;
    }
  }
}

}  // namespace roialign
