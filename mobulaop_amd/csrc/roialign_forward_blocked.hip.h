// Forward ROIAlign over a channel-blocked copy of the feature map.
//
// The map is first rewritten from NCHW to [N][C/CB][H][W][CB] with CB = 32
// channels for fp32 and 64 for fp16: the channels of a block at one pixel are
// one 128-byte line.  A wavefront then computes one (ROI, channel block): its
// 64 lanes are 8 pooled columns x 8 groups of 16 bytes of channels, so a single
// 16-byte load per lane fetches one bilinear corner of eight bins (1 KB),
// sixteen such loads are in flight per lane, and every lane sums its own bin:
// no cross-lane traffic.  Row corners are the same for the
// whole wavefront and live in scalar registers; a map row that several samples
// of a pooled column touch (samples less than a pixel apart, within a bin or in
// neighbouring bins) is fetched once and its weighted column sum reused.
// Channel block b is only ever read by XCD b % 8 and ROIs are visited in
// spatial order, so what one L2 has to hold is a 128-byte-per-pixel slice of
// the neighbourhood the XCD is currently working in.
#pragma once
#include <type_traits>

#include "roialign_geometry.h"

namespace roialign {

struct FwdBlocked {
  static constexpr int NW = 4;         // independent wavefronts per workgroup
  static constexpr int MAXT = 16;      // column samples held in LDS (two for each of 8 pooled columns)
  static constexpr int ROWT = 64;      // row samples held in LDS at a time
  static constexpr int PWB = 8;        // pooled columns per step (one per group of 8 lanes)
  static constexpr int CELL = 32;      // side of the sorting cells in pixels
  static constexpr int MAXCELLS = 8192;
};

// Per element type: channels per lane (16 bytes), channels per block of the
// blocked layout (8 lanes: 128 bytes per pixel), staged outputs per wavefront
// (8704 bytes: with the sample tables 39.9 KB per workgroup of four, four workgroups
// to a CU, which the registers allow anyway; 14 x 14 pooled maps go in four passes).
template <typename T>
struct BlockOf {
  static constexpr int CPL = 16 / sizeof(T);
  static constexpr int CB = 8 * CPL;
  static constexpr int STAGE = 8704 / sizeof(T);
  // the same for the gather of larger sampling grids (one wavefront per workgroup: with 6400 bytes
  // the registers, not LDS, bound the wavefronts of a CU)
  static constexpr int STAGE_MERGED = 6400 / sizeof(T);
};

// Pooled rows staged per pass, 0 if the shape is not taken by this path.
template <typename T>
inline int blocked_rows_per_pass(int C, long long H, long long W, int PH, int PW, bool merged) {
  using B = BlockOf<T>;
  const int stage = merged ? B::STAGE_MERGED : B::STAGE;
  if (C % B::CPL != 0 || PW < 1 || B::CB * PW > stage) return 0;
  if (H * W * 128 >= (1ll << 31)) return 0;
  return min(PH, stage / (B::CB * PW));
}

struct OrderArgs { const float* rois; int* order; int R; float scale; int H, W; long long num_images; };

template <int NT, int MAXC>
__device__ __forceinline__ void roi_order_body(int* hist, int* wave_sum, int* carry, const float* __restrict__ rois,
                                               int R, float scale, int H, int W, long long num_images,
                                               int* __restrict__ order);

// out[n][cb][p][CB] = in[n][cb*CB + k][p]; channels past C are written as zero.
// With oa.order set the launch has one more column of workgroups, the first of which sorts the
// ROIs (roi_order_body with the cells that fit the tile's LDS) while the others copy: the
// ordering of a few thousand ROIs then costs nothing beside a copy that takes several times as long.
template <typename T, bool VEC>
__global__ void __launch_bounds__(256)
transpose_to_blocked_kernel(const T* __restrict__ in, T* __restrict__ out, int C, int P, OrderArgs oa) {
  constexpr int CB = BlockOf<T>::CB;
  struct alignas(4 * sizeof(T)) V4 { T v[4]; };
  __shared__ T tile[CB][65];
  int bx = blockIdx.x;
  if (oa.order != nullptr) {
    if (bx == 0) {
      if (blockIdx.y == 0 && blockIdx.z == 0) {
        constexpr int WORDS = static_cast<int>(sizeof(tile) / 4), MAXC = WORDS - 24;
        int* const words = reinterpret_cast<int*>(&tile[0][0]);
        roi_order_body<256, MAXC>(words, words + MAXC + 1, words + MAXC + 20, oa.rois, oa.R, oa.scale, oa.H, oa.W,
                                  oa.num_images, oa.order);
      }
      return;
    }
    --bx;
  }
  const int n = blockIdx.z, cb = blockIdx.y, cblk = gridDim.y;
  const int p0 = bx * 64, c0 = cb * CB;
  const T* src = in + static_cast<size_t>(n) * C * P;
  T* dst = out + (static_cast<size_t>(n) * cblk + cb) * P * CB;
  if (VEC) {
    const int q = threadIdx.x & 15, r = threadIdx.x >> 4;   // 16 quads of pixels, 16 channels per pass
#pragma unroll
    for (int k = 0; k < CB / 16; ++k) {
      const int c = c0 + r + 16 * k, p = p0 + 4 * q;
      V4 v;
#pragma unroll
      for (int i = 0; i < 4; ++i) v.v[i] = from_float<T>(0.0f);
      if (c < C && p < P) {   // the map is read once here: no need to keep it in the caches
        if constexpr (sizeof(T) == 4) {
          typedef float f32x4 __attribute__((ext_vector_type(4)));
          const f32x4 raw = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(src + static_cast<size_t>(c) * P + p));
          v = __builtin_bit_cast(V4, raw);
        } else {
          typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
          const u32x2 raw = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(src + static_cast<size_t>(c) * P + p));
          v = __builtin_bit_cast(V4, raw);
        }
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) tile[r + 16 * k][4 * q + i] = v.v[i];
    }
  } else {
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
#pragma unroll
    for (int k = 0; k < CB / 4; ++k) {
      const int c = c0 + ty + 4 * k, p = p0 + tx;
      tile[ty + 4 * k][tx] = (c < C && p < P) ? src[static_cast<size_t>(c) * P + p] : from_float<T>(0.0f);
    }
  }
  __syncthreads();
  constexpr int QP = CB / 4, PP = 256 / QP;   // channel quads per pixel, pixels per pass
  const int cq = threadIdx.x % QP, pr = threadIdx.x / QP;
#pragma unroll
  for (int k = 0; k < 64 / PP; ++k) {
    const int pl = pr + PP * k;
    if (p0 + pl < P) {
      V4 v;
#pragma unroll
      for (int i = 0; i < 4; ++i) v.v[i] = tile[4 * cq + i][pl];
      *reinterpret_cast<V4*>(dst + static_cast<size_t>(p0 + pl) * CB + 4 * cq) = v;
    }
  }
}

// order[] = ROI indices sorted by (image, 32x32-pixel cell of the box centre,
// rows of cells walked in alternating direction): consecutive wavefronts then
// read neighbouring parts of the map.  One workgroup; counting sort with the
// histogram in LDS.  ROIs that name no image sort last.
// (the body: NT threads of one workgroup, at most MAXC cells; hist holds MAXC + 1 counters)
template <int NT, int MAXC>
__device__ __forceinline__ void roi_order_body(int* hist, int* wave_sum, int* carry, const float* __restrict__ rois,
                                               int R, float scale, int H, int W, long long num_images,
                                               int* __restrict__ order) {
  using K = FwdBlocked;
  int cell = K::CELL;
  long long cy = (H + cell - 1) / cell, cx = (W + cell - 1) / cell;
  while (cy * cx * num_images > MAXC && cell < (1 << 20)) {
    cell *= 2;
    cy = (H + cell - 1) / cell; cx = (W + cell - 1) / cell;
  }
  const int cells = cy * cx * num_images > MAXC ? 1 : static_cast<int>(cy * cx * num_images);
  auto key_of = [&](int r) {
    const float* q = rois + static_cast<long long>(r) * 5;
    const int b = static_cast<int>(q[0]);
    if (b < 0 || b >= num_images) return cells;
    if (cells == 1) return 0;
    const float mx = 0.5f * (q[1] + q[3]) * scale, my = 0.5f * (q[2] + q[4]) * scale;
    const int ix = min(max(static_cast<int>(mx), 0), W - 1) / cell;
    const int iy = min(max(static_cast<int>(my), 0), H - 1) / cell;
    const int sx = (iy & 1) ? static_cast<int>(cx) - 1 - ix : ix;
    return static_cast<int>((b * cy + iy) * cx + sx);
  };
  for (int i = threadIdx.x; i <= cells; i += NT) hist[i] = 0;
  if (threadIdx.x == 0) *carry = 0;
  __syncthreads();
  for (int r = threadIdx.x; r < R; r += NT) atomicAdd(&hist[key_of(r)], 1);
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int base = 0; base <= cells; base += NT) {
    const int i = base + threadIdx.x;
    const int v = i <= cells ? hist[i] : 0;
    int incl = v;
    for (int off = 1; off < 64; off <<= 1) {
      const int up = __shfl_up(incl, off);
      if (lane >= off) incl += up;
    }
    if (lane == 63) wave_sum[wave] = incl;
    __syncthreads();
    int before = *carry;
    for (int w = 0; w < wave; ++w) before += wave_sum[w];
    if (i <= cells) hist[i] = before + incl - v;
    __syncthreads();
    if (threadIdx.x == NT - 1) *carry = before + incl;
    __syncthreads();
  }
  for (int r = threadIdx.x; r < R; r += NT) order[atomicAdd(&hist[key_of(r)], 1)] = r;
}

__global__ void __launch_bounds__(1024)
roi_order_kernel(const float* __restrict__ rois, int R, float scale, int H, int W,
                 long long num_images, int* __restrict__ order) {
  __shared__ int hist[FwdBlocked::MAXCELLS + 1];
  __shared__ int wave_sum[16];
  __shared__ int carry;
  roi_order_body<1024, FwdBlocked::MAXCELLS>(hist, wave_sum, &carry, rois, R, scale, H, W, num_images, order);
}

// A row sample: byte offsets of its low and high row in a channel block's
// plane (lo negative: the sample lies outside the map) and their weights.
struct alignas(16) RowEntry { int lo, hi; float wl, wh; };
// A column sample, likewise, with the offsets in bytes along a row.
struct alignas(16) ColEntry { int lo, hi; float wl, wh; };

// Sixteen bytes of consecutive channels as they lie in a lane's registers: four
// fp32 or eight 16-bit values (kept packed; an element is widened where it is used).
template <typename T> struct LaneData;
template <> struct LaneData<float> { typedef float type __attribute__((ext_vector_type(4))); };
template <> struct LaneData<__half> { typedef _Float16 type __attribute__((ext_vector_type(8))); };
template <> struct LaneData<bfloat16> { typedef __bf16 type __attribute__((ext_vector_type(8))); };

// The sixteen bytes at byte offset lane_off + row_off of a raw buffer; lane
// offsets outside the buffer read as zero without an access.
template <typename T>
__device__ __forceinline__ typename LaneData<T>::type buffer_load_lane(__amdgpu_buffer_rsrc_t rsrc, int lane_off,
                                                                       int row_off) {
  typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
  const u32x4 raw = __builtin_amdgcn_raw_buffer_load_b128(rsrc, lane_off, row_off, 0);
  return __builtin_bit_cast(typename LaneData<T>::type, raw);
}

// Number of workgroups for R ROIs and cblk channel blocks (see the job decode
// at the top of forward_blocked_kernel).
// (nw: wavefronts per workgroup of the kernel that is launched)
inline long long blocked_grid(long long R, int cblk, int nw = FwdBlocked::NW) {
  long long per_xcd;
  if (cblk >= 8) per_xcd = R * ((cblk + 7) / 8);
  else per_xcd = (R + (8 / cblk) - 1) / (8 / cblk);
  return 8 * ((per_xcd + nw - 1) / nw);
}

// The same for channels-last maps (see the job decode).
inline long long blocked_grid_nhwc(long long R, int cblk, int nw = FwdBlocked::NW) {
  return 8 * (((R + 7) / 8 * cblk + nw - 1) / nw);
}

template <typename T, bool NHWC>
__global__ void __launch_bounds__(FwdBlocked::NW * 64, 4)
forward_blocked_kernel(const T* __restrict__ xt, const float* __restrict__ rois,
                       const int* __restrict__ order, T* __restrict__ y, float scale, int C, int H,
                       int W, int PH, int PW, int S, long long num_images, int cblk,
                       int rows_per_pass, int R) {
  using K = FwdBlocked;
  constexpr int CPL = BlockOf<T>::CPL, CB = BlockOf<T>::CB, STAGE = BlockOf<T>::STAGE;
  typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
  constexpr int CWIN = K::MAXT / K::PWB;   // column samples per pooled column held at a time
  __shared__ RowEntry rows_s[K::NW][K::ROWT];
  __shared__ ColEntry cols_s[K::NW][K::MAXT];
  __shared__ __attribute__((aligned(16))) T stage_s[K::NW][STAGE];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  auto uni_i = [](int v) { return __builtin_amdgcn_readfirstlane(v); };
  auto uni_f = [](float v) { return __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(v))); };
  // Job decode.  Workgroups are dealt to the 8 XCDs round-robin, so blockIdx % 8
  // names the XCD: it takes the channel blocks b with b % 8 == xcd and walks
  // the sorted ROIs; with fewer than 8 blocks the ROIs of a block are split
  // into 8 / cblk contiguous ranges instead.
  const int xcd = blockIdx.x & 7;
  const long long wi = static_cast<long long>(blockIdx.x >> 3) * K::NW + wave;
  long long slot;
  int cb;
  if (NHWC) {
    // the caller's map: an XCD takes an eighth of the (spatially sorted) ROIs
    // (channel block by channel block: what the XCD's L2 has to hold at a time is one
    // 128-byte slice of the pixels its ROIs cover)
    const long long range = (R + 7) / 8;
    cb = static_cast<int>(wi / range);
    if (cb >= cblk) return;
    slot = xcd * range + (wi - cb * range);
  } else if (cblk >= 8) {
    const int nx = (cblk - xcd + 7) >> 3;
    slot = wi / nx;
    cb = xcd + 8 * static_cast<int>(wi % nx);
  } else {
    const int parts = 8 / cblk;
    cb = xcd % cblk;
    const int part = xcd / cblk;
    const long long range = (R + parts - 1) / parts;
    if (part >= parts || wi >= range) return;
    slot = part * range + wi;
  }
  if (slot >= R) return;
  const int roi = uni_i(order != nullptr ? order[slot] : static_cast<int>(slot));   // no order: as listed
  const int c0 = cb * CB, nch = min(CB, C - c0);
  const int grp = lane >> 3, quad = lane & 7;   // pooled column within a step, channel quad
  const bool quad_on = CPL * quad < nch;
  const RoiGeom g = roi_geometry(rois + static_cast<long long>(roi) * 5, scale, PH, PW, S);
  const int bins = PH * PW;
  const int batch = uni_i(g.batch);
  const bool image_ok = batch >= 0 && batch < num_images;
  const int gh = uni_i(g.grid_h), gw = uni_i(g.grid_w);
  const float count = uni_f(g.count);
  // count is a power of two for the usual sampling ratios: multiply by its exact reciprocal
  const bool pow2 = (gh & (gh - 1)) == 0 && (gw & (gw - 1)) == 0;
  const float inv_count = 1.0f / count;
  RowEntry* const rows = rows_s[wave];
  ColEntry* const cols = cols_s[wave];
  T* const stage = stage_s[wave];
  // NHWC: the caller's [N][H][W][C] map is read where it lies, a pixel's channels C * sizeof(T) apart
  const int px_bytes = (NHWC ? C : CB) * static_cast<int>(sizeof(T)), row_bytes = W * px_bytes;
  const int lane_off = quad * 16;
  constexpr int kDead = static_cast<int>(0x80000000u);

  // The (image, channel block) plane as a raw buffer: a load whose lane offset
  // is kDead falls outside it and returns zero.
  const size_t image_no = static_cast<size_t>(image_ok ? batch : 0);
  const char* const plane_ptr = reinterpret_cast<const char*>(xt) +
      (NHWC ? image_no * H * row_bytes + static_cast<size_t>(cb) * 128 : (image_no * cblk + cb) * H * row_bytes);
  const __amdgpu_buffer_rsrc_t plane = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<char*>(plane_ptr), 0, H * row_bytes - (NHWC ? cb * 128 : 0), 0x00020000);

  // LDS holds a window of the row samples (flat index ph * gh + iy) and, for the
  // current block of 8 pooled columns, a window of CWIN column samples each.
  // Both are refilled by the whole wavefront when a step leaves the window;
  // with the usual grids one fill per ROI covers everything.
  int row_s0 = 0, row_s1 = 0;
  auto need_rows = [&](int s, int n) {
    if (s < row_s0 || s + n > row_s1) {
      row_s0 = s;
      row_s1 = min(s + K::ROWT, PH * gh);
      for (int i = lane; i < row_s1 - row_s0; i += 64) {
        const int f = row_s0 + i, ph = f / gh, iy = f - ph * gh;
        const AxisSample a = axis_sample(sample_coord(g.start_h, ph, g.bin_h, iy, gh), H);
        rows[i] = RowEntry{a.valid ? a.low * row_bytes : -1, a.high * row_bytes, a.h, a.l};
      }
    }
  };
  int col_pwb = -1, col_x0 = 0, col_x1 = 0;
  auto need_cols = [&](int pwb, int ix, int n) {
    if (pwb != col_pwb || ix < col_x0 || ix + n > col_x1) {
      col_pwb = pwb; col_x0 = ix; col_x1 = min(ix + CWIN, gw);
      for (int i = lane; i < K::MAXT; i += 64) {
        const int pw = pwb + i / CWIN, x = col_x0 + i % CWIN;
        if (pw < PW && x < col_x1) {
          const AxisSample a = axis_sample(sample_coord(g.start_w, pw, g.bin_w, x, gw), W);
          cols[i] = ColEntry{a.valid ? a.low * px_bytes : -1, a.high * px_bytes, a.h, a.l};
        }
      }
    }
  };

  for (int ph0 = 0; ph0 < PH; ph0 += rows_per_pass) {
    const int rp = min(rows_per_pass, PH - ph0), seg = rp * PW;
    for (int pwb = 0; pwb < PW; pwb += K::PWB) {
      const int pw = pwb + grp;
      const bool bin_on = pw < PW && quad_on;
      // Column corners of this lane's pooled column (samples 0 and 1: the grid is at most
      // 2 x 2 here).  A corner that does not exist (outside the map, past the grid, no bin
      // for this lane) or that repeats an earlier one is not loaded.
      int coff[4];
      float cw[4];
      if (image_ok) {
        need_cols(pwb, 0, gw);
#pragma unroll
        for (int a = 0; a < 2; ++a) {
          const ColEntry e = cols[grp * CWIN + min(a, gw - 1) - col_x0];
          const bool ok = e.lo >= 0 && a < gw && bin_on;
          coff[2 * a] = ok ? e.lo + lane_off : kDead;
          coff[2 * a + 1] = ok ? e.hi + lane_off : kDead;
          cw[2 * a] = ok ? e.wl : 0.0f;
          cw[2 * a + 1] = ok ? e.wh : 0.0f;
        }
        const bool both = coff[0] != kDead && coff[2] != kDead;
        const bool same = both && coff[2] == coff[0];
        const bool next = both && !same && coff[2] == coff[1];
        cw[0] += same ? cw[2] : 0.0f;
        cw[1] += same ? cw[3] : (next ? cw[2] : 0.0f);
        if (same || next) { coff[2] = coff[3]; cw[2] = cw[3]; coff[3] = kDead; cw[3] = 0.0f; }
        if (same) { coff[2] = kDead; cw[2] = 0.0f; }
      }
      // how many of the four corner slots any lane uses: boxes whose samples are at most a
      // pixel apart need three (two when both samples of every bin share their pixels)
      const int ncol = !image_ok ? 2 : __ballot(coff[3] != kDead) != 0 ? 4 : __ballot(coff[2] != kDead) != 0 ? 3 : 2;
      // A map row's contribution to this lane's pooled column, t(row) = sum over the column
      // corners of weight x value, is the same for every sample that touches the row: samples
      // less than a pixel apart share rows, within a bin and from one bin to the next (rows
      // only go up), so t of the two rows of the last sample is carried along and a row is
      // fetched once per pooled column however many samples use it.
      // (With eight channels per lane the carried sums would not fit the registers that four
      // wavefronts per SIMD leave: 16-bit maps share rows within a pooled row only.)
      constexpr bool CARRY = CPL <= 4;
      int carry_off[2] = {kDead, kDead};   // (no row has this offset)
      float carry[2][CPL];
#pragma unroll
      for (int i = 0; i < CPL; ++i) carry[0][i] = carry[1][i] = 0.0f;
      auto pooled_rows = [&](auto corner_slots) {
        constexpr int NC = decltype(corner_slots)::value;
#pragma nounroll
        for (int ph = ph0; ph < ph0 + rp; ++ph) {
          float acc[CPL];
#pragma unroll
          for (int i = 0; i < CPL; ++i) acc[i] = 0.0f;
          if (image_ok) {
            // Row corners of samples 0 and 1: the same for every lane, so they sit in scalar
            // registers and steer uniform branches.
            need_rows(ph * gh, gh);
            int roff[4];
            float rw[4];
            int from[4];   // -1: no such corner; 0: loaded; 5, 6: the carried rows; 7: the sample's other row
            {
              int known[2] = {carry_off[0], carry_off[1]};   // the carried rows by the time of each sample
#pragma unroll
              for (int a = 0; a < 2; ++a) {
                const RowEntry e = rows[ph * gh + min(a, gh - 1) - row_s0];
                const int lo = uni_i(e.lo), hi = uni_i(e.hi);
                roff[2 * a] = lo; roff[2 * a + 1] = hi;
                rw[2 * a] = uni_f(e.wl); rw[2 * a + 1] = uni_f(e.wh);
                if (lo >= 0 && a < gh) {
                  from[2 * a] = lo == known[0] ? 5 : lo == known[1] ? 6 : 0;
                  from[2 * a + 1] = hi == lo ? 7 : hi == known[0] ? 5 : hi == known[1] ? 6 : 0;
                  known[0] = lo; known[1] = hi;
                } else {
                  from[2 * a] = from[2 * a + 1] = -1;
                }
              }
            }
            // up to sixteen corners: four rows (scalar) x four columns (per lane)
            typename LaneData<T>::type v[4][NC];
#pragma unroll
            for (int r = 0; r < 4; ++r)
              if (from[r] == 0) {
#pragma unroll
                for (int c = 0; c < NC; ++c) v[r][c] = buffer_load_lane<T>(plane, coff[c], roff[r]);
              }
            if constexpr (CARRY) {
#pragma unroll
              for (int a = 0; a < 2; ++a) {
                if (from[2 * a] < 0) continue;
                float t[2][CPL];
#pragma unroll
                for (int k = 0; k < 2; ++k) {
                  const int r = 2 * a + k;
                  if (from[r] == 0) {
#pragma unroll
                    for (int i = 0; i < CPL; ++i) {
                      float u = cw[0] * static_cast<float>(v[r][0][i]);
#pragma unroll
                      for (int c = 1; c < NC; ++c) u = fmaf(cw[c], static_cast<float>(v[r][c][i]), u);
                      t[k][i] = u;
                    }
                  } else if (from[r] == 5) {
#pragma unroll
                    for (int i = 0; i < CPL; ++i) t[k][i] = carry[0][i];
                  } else if (from[r] == 6) {
#pragma unroll
                    for (int i = 0; i < CPL; ++i) t[k][i] = carry[1][i];
                  } else {
#pragma unroll
                    for (int i = 0; i < CPL; ++i) t[k][i] = t[0][i];
                  }
#pragma unroll
                  for (int i = 0; i < CPL; ++i) acc[i] = fmaf(rw[r], t[k][i], acc[i]);
                }
                carry_off[0] = roff[2 * a]; carry_off[1] = roff[2 * a + 1];
#pragma unroll
                for (int i = 0; i < CPL; ++i) { carry[0][i] = t[0][i]; carry[1][i] = t[1][i]; }
              }
            } else {
              // a repeated row's weight goes to the corner that fetched the row
              if (from[1] == 7) rw[0] += rw[1];
              if (from[3] == 7) rw[2] += rw[3];
#pragma unroll
              for (int r = 2; r < 4; ++r) {
                if (from[r] == 5) rw[0] += rw[r];
                if (from[r] == 6) rw[1] += rw[r];
              }
#pragma unroll
              for (int r = 0; r < 4; ++r)
                if (from[r] == 0) {
#pragma unroll
                  for (int i = 0; i < CPL; ++i) {
                    float u = cw[0] * static_cast<float>(v[r][0][i]);
#pragma unroll
                    for (int c = 1; c < NC; ++c) u = fmaf(cw[c], static_cast<float>(v[r][c][i]), u);
                    acc[i] = fmaf(rw[r], u, acc[i]);
                  }
                }
            }
          }
          if (pow2) {
#pragma unroll
            for (int i = 0; i < CPL; ++i) acc[i] *= inv_count;
          } else {
            asm volatile("" ::: "memory");   // keeps the division out of the common path
#pragma unroll
            for (int i = 0; i < CPL; ++i) acc[i] /= count;
          }
          if (NHWC) {
            // y[roi][ph][pw][C]: the lane's channels of its bin are 16 contiguous bytes
            if (bin_on) {
              T out[CPL];
#pragma unroll
              for (int i = 0; i < CPL; ++i) out[i] = from_float<T>(acc[i]);
              T* const dst = y + ((static_cast<size_t>(roi) * PH + ph) * PW + pw) * C + c0 + CPL * quad;
              *reinterpret_cast<u32x4*>(dst) = *reinterpret_cast<const u32x4*>(out);
            }
          } else if (bin_on) {
#pragma unroll
            for (int i = 0; i < CPL; ++i)
              stage[(CPL * quad + i) * seg + (ph - ph0) * PW + pw] = from_float<T>(acc[i]);
          }
        }
      };
      if (ncol == 4) pooled_rows(std::integral_constant<int, 4>());
      else if (ncol == 3) pooled_rows(std::integral_constant<int, 3>());
      else pooled_rows(std::integral_constant<int, 2>());
    }
    if (NHWC) continue;
    // the wavefront's outputs of this pass leave LDS in the order of y
    // (the lane number through an empty asm: the addresses below are then formed here, not
    // ahead of the gather, where they would take registers the gather needs)
    int lane_now = lane;
    asm volatile("" : "+v"(lane_now));
    if (rp == PH) {
      const int total = nch * seg;
      T* const dst = y + (static_cast<size_t>(roi) * C + c0) * bins;
      constexpr int per = 16 / sizeof(T);
      if (reinterpret_cast<size_t>(dst) % 16 == 0) {
        const int nvec = total / per;
        for (int i = lane_now; i < nvec; i += 64)
          __builtin_nontemporal_store(reinterpret_cast<const u32x4*>(stage)[i], reinterpret_cast<u32x4*>(dst) + i);
        for (int i = nvec * per + lane_now; i < total; i += 64) dst[i] = stage[i];
      } else {
        for (int i = lane_now; i < total; i += 64) dst[i] = stage[i];
      }
    } else {
      // some pooled rows of every channel: seg contiguous elements per channel, the lanes cover
      // as many channels at a time as fit (one division per pass, none per element)
      const int chans = max(1, 64 / seg), cl = lane_now / seg, j0 = lane_now - cl * seg;
      if (seg <= 64) {
        if (cl < chans) {
          // (the same base for every lane: scalar registers; 32-bit offsets per lane)
          T* const base = y + (static_cast<size_t>(roi) * C + c0) * bins + ph0 * PW;
          int to = cl * bins + j0, from = cl * seg + j0;
#pragma nounroll
          for (int c = cl; c < nch; c += chans, to += chans * bins, from += chans * seg) base[to] = stage[from];
        }
      } else {
        for (int c = 0; c < nch; ++c)
          for (int j = lane_now; j < seg; j += 64)
            y[(static_cast<size_t>(roi) * C + c0 + c) * bins + ph0 * PW + j] = stage[c * seg + j];
      }
    }
  }
}

}  // namespace roialign
