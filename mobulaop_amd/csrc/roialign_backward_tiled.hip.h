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
  static constexpr int UB = 4;                   // pooled columns per scalar unit block (8 units)
  static_assert(CS % 2 == 1, "channel stride must be odd");
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
template <int G0, int NV, int ST>
__device__ __forceinline__ void add_block_n(float* row, const float (&g)[8], const UnitBlock& u) {
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

template <int G0, int NV>
__device__ __forceinline__ void add_block_s(float* row, const float (&g)[8], const UnitBlock& u, int lg) {
  switch (lg) {
    case 0: add_block_n<G0, NV, 1>(row, g, u); break;
    case 1: add_block_n<G0, NV, 2>(row, g, u); break;
    case 2: add_block_n<G0, NV, 4>(row, g, u); break;
    default: add_block_n<G0, NV, 8>(row, g, u); break;
  }
}

template <int G0>
__device__ __forceinline__ void add_block(float* row, const float (&g)[8], const UnitBlock& u,
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
// contiguous 2 KB segment.  One workgroup per (ROI, 64 channels).
__global__ void __launch_bounds__(256)
transpose_dy_kernel(const float* __restrict__ dy, float* __restrict__ dyt, int C, int PH, int PW,
                    int cblocks) {
  __shared__ float buf[64 * 65];
  const int r = blockIdx.x / cblocks, cb = blockIdx.x % cblocks;
  const int c0 = cb * 64, nch = min(64, C - c0);
  const int bins = PH * PW;
  const float* src = dy + (static_cast<size_t>(r) * C + c0) * bins;
  float* dst = dyt + static_cast<size_t>(r) * PH * C * 8;
  for (int b0 = 0; b0 < bins; b0 += 64) {
    const int nb = min(64, bins - b0);
    __syncthreads();
    for (int i = threadIdx.x; i < nch * nb; i += 256) {
      const int c = i / nb, b = i - c * nb;
      buf[c * 65 + b] = src[static_cast<size_t>(c) * bins + b0 + b];
    }
    __syncthreads();
    // bins [b0, b0+nb) of every channel -> rows ph = bin / PW, slot k = bin % PW
    for (int i = threadIdx.x; i < nch * nb; i += 256) {
      const int b = i / nch, c = i - b * nch;
      const int bin = b0 + b, ph = bin / PW, k = bin - ph * PW;
      dst[(static_cast<size_t>(ph) * C + c0 + c) * 8 + k] = buf[c * 65 + b];
    }
  }
  // zero the padding slots
  for (int i = threadIdx.x; i < PH * nch * (8 - PW); i += 256) {
    const int k = PW + i % (8 - PW), c = (i / (8 - PW)) % nch, ph = i / ((8 - PW) * nch);
    dst[(static_cast<size_t>(ph) * C + c0 + c) * 8 + k] = 0.0f;
  }
}

__global__ void __launch_bounds__(BwdTile::NT)
backward_tiled_kernel(const float* __restrict__ dyt, float* __restrict__ dx,
                      const int* __restrict__ tile_offset, const int* __restrict__ tile_rois,
                      const AxisUnit* __restrict__ lists, TileGrid tg, ListLayout ll, int C, int H,
                      int W, int PH, int PW, int cblocks, long long num_jobs, int assign) {
  using K = BwdTile;
  __shared__ float acc[K::CH * K::CS];

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
  const AxisUnit* const row_lists = lists + static_cast<long long>(ty) * ll.row_stride;
  const AxisUnit* const col_lists =
      lists + static_cast<long long>(ll.ty) * ll.row_stride + static_cast<long long>(tx) * ll.col_stride;
  const AxisUnit kDead = AxisUnit{0, -4, 0.0f, 0.0f};

  // Software pipeline over the tile's ROI list, per wavefront:
  //   stage 1 (ROI it+2): fetch row unit `lane` of its row list
  //   stage 2 (ROI it+1): which sample rows land on my tile row?  fetch the dy
  //                       row of the first of them
  //   stage 3 (ROI it)  : fold all taps into g[pw], walk the column units
  auto fetch_ru = [&](int it) -> AxisUnit {
    if (it >= list_end || lane >= kRowSlots) return kDead;
    return row_lists[static_cast<long long>(tile_rois[it]) * ll.roi_stride + lane];
  };
  auto mine_of = [&](const AxisUnit& ru) -> float {
    return ru.pos == wave ? ru.w0 : ru.pos + 1 == wave ? ru.w1 : 0.0f;
  };
  if (wave < rows) {
    int roi_cur = tile_rois[list_begin];
    int roi_nx = list_begin + 1 < list_end ? tile_rois[list_begin + 1] : roi_cur;
    AxisUnit ru_cur = fetch_ru(list_begin), ru_nx = fetch_ru(list_begin + 1);
    float w_cur = mine_of(ru_cur);
    unsigned long long taps_cur = __ballot(w_cur != 0.0f);
    float d_cur[8];
    {
      const int ph0 = __builtin_amdgcn_readlane(ru_cur.bin, taps_cur ? __builtin_ctzll(taps_cur) : 0);
      load_dy_row(dy_lane + roi_cur * roi_dy_stride + ph0 * ph_dy_stride, d_cur);
    }
    for (int it = list_begin; it < list_end; ++it) {
      // stage 1
      const int roi_n2 = it + 2 < list_end ? tile_rois[it + 2] : roi_nx;
      const AxisUnit ru_n2 =
          (it + 2 < list_end && lane < kRowSlots)
              ? row_lists[static_cast<long long>(roi_n2) * ll.roi_stride + lane] : kDead;
      // stage 2
      const float w_nx = mine_of(ru_nx);
      const unsigned long long taps_nx = __ballot(w_nx != 0.0f);
      float d_nx[8];
      if (taps_nx != 0) {
        const int ph0 = __builtin_amdgcn_readlane(ru_nx.bin, __builtin_ctzll(taps_nx));
        load_dy_row(dy_lane + roi_nx * roi_dy_stride + ph0 * ph_dy_stride, d_nx);
      }
      // stage 3
      if (taps_cur != 0) {
        const AxisUnit* const cl = col_lists + static_cast<long long>(roi_cur) * ll.roi_stride;
        const float* const dy_roi = dy_lane + roi_cur * roi_dy_stride;
        const UnitBlock ub0 = load_unit_block(cl);
        const int lg = (ub0.lo[0] >> kStrideShift) & kStrideMask;
        for (int pwb = 0; pwb < PW; pwb += K::PWB) {
          const int nb = min(K::PWB, PW - pwb);
          const UnitBlock ub_a = pwb == 0 ? ub0 : load_unit_block(cl + 2 * pwb);
          float g[8];
          unsigned long long taps = taps_cur;
          bool first = true;
          while (taps != 0) {
            const int i = __builtin_ctzll(taps);
            taps &= taps - 1;
            const int ph = __builtin_amdgcn_readlane(ru_cur.bin, i);
            const float wy = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(w_cur), i));
            float d[8];
            if (first && pwb == 0) {
#pragma unroll
              for (int k = 0; k < 8; ++k) d[k] = d_cur[k];
            } else {
              load_dy_row(dy_roi + ph * ph_dy_stride, d);
            }
#pragma unroll
            for (int k = 0; k < 8; ++k) g[k] = first ? d[k] * wy : fmaf(d[k], wy, g[k]);
            first = false;
          }
#ifdef LAB_NO_ADD
          if (g[0] == 12345.f && g[3] == 3.f && g[6] == 1.f) row[ub_a.pos(0)] = g[1] + g[2] + g[4] + g[5] + g[7];
          continue;
#endif
          if (lane < nch) {
            add_block<0>(row, g, ub_a, min(nb, K::UB), lg);
            if (nb > K::UB) add_block<4>(row, g, load_unit_block(cl + 2 * (pwb + K::UB)), nb - K::UB, lg);
          }
        }
      }
      // rotate
      ru_cur = ru_nx; ru_nx = ru_n2; w_cur = w_nx; taps_cur = taps_nx;
      roi_cur = roi_nx; roi_nx = roi_n2;
#pragma unroll
      for (int k = 0; k < 8; ++k) d_cur[k] = d_nx[k];
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
