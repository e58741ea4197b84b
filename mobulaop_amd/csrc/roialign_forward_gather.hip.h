// ROIAlign forward as a channel-last gather.
//
// Step 1 (transpose_to_channel_last_kernel): the NCHW feature map is copied
// once to [N][H][W][C].  Step 2 (forward_gather_kernel): one workgroup per
// (ROI, block of 64 channels), one wavefront per pooled row, one channel per
// lane.  With channels innermost the four corners of a bilinear sample are
// four 256-byte coalesced loads, and everything that depends only on the ROI
// -- sample positions, corner weights, validity -- is the same for all 64
// lanes: the column samples are computed once per workgroup into LDS, row
// samples once per wavefront, and the addresses are built on the scalar unit.
//
// Arithmetic per sample: hy*(hx*v1 + lx*v2) + ly*(hx*v3 + lx*v4), summed over
// the grid and divided by the sample count, against the reference's
// w1*v1 + w2*v2 + w3*v3 + w4*v4 with wk = products of the same four weights
// (opzoo/ROIAlign/bilinear.h:46-58, ROIAlign.cpp:56-74): same samples and
// weights (coordinates come from roialign_geometry.h), rounding differs in the
// last bits.  Invalid samples (outside [-1, size] on either axis) are skipped.
#pragma once
#include <type_traits>
#include "roialign_geometry.h"

namespace roialign {

// out[n][p][c] = in[n][c][p], p = pixel index; 64x64 tiles through LDS.  With
// VEC the tile is moved with 16-byte (fp32) / 8-byte (fp16) accesses on both
// sides; it needs P % 4 == 0, C % 4 == 0 and aligned base pointers.
template <typename T, bool VEC>
__global__ void __launch_bounds__(256)
transpose_to_channel_last_kernel(const T* __restrict__ in, T* __restrict__ out, int C, int P) {
  __shared__ T tile[64][65];
  const int n = blockIdx.z;
  const int p0 = blockIdx.x * 64, c0 = blockIdx.y * 64;
  const T* src = in + static_cast<size_t>(n) * C * P;
  T* dst = out + static_cast<size_t>(n) * C * P;
  if (VEC) {
    struct alignas(4 * sizeof(T)) V4 { T v[4]; };
    const int q = threadIdx.x & 15, r = threadIdx.x >> 4;   // 16 quads per row, 16 rows per pass
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int c = c0 + r + 16 * k, p = p0 + 4 * q;
      if (c < C && p < P) {
        const V4 v = *reinterpret_cast<const V4*>(src + static_cast<size_t>(c) * P + p);
#pragma unroll
        for (int i = 0; i < 4; ++i) tile[r + 16 * k][4 * q + i] = v.v[i];
      }
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int p = p0 + r + 16 * k, c = c0 + 4 * q;
      if (c < C && p < P) {
        V4 v;
#pragma unroll
        for (int i = 0; i < 4; ++i) v.v[i] = tile[4 * q + i][r + 16 * k];
        *reinterpret_cast<V4*>(dst + static_cast<size_t>(p) * C + c) = v;
      }
    }
  } else {
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      const int c = c0 + ty + 4 * k, p = p0 + tx;
      if (c < C && p < P) tile[ty + 4 * k][tx] = src[static_cast<size_t>(c) * P + p];
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      const int p = p0 + ty + 4 * k, c = c0 + tx;
      if (c < C && p < P) dst[static_cast<size_t>(p) * C + c] = tile[tx][ty + 4 * k];
    }
  }
}

struct FwdGather {
  static constexpr int CH = 64;      // channels per workgroup (one per lane)
  static constexpr int NW = 8;       // wavefronts: pooled rows in flight
  static constexpr int NT = NW * 64;
  static constexpr int MAXC = 512;   // column samples held in LDS
  static constexpr int PWB = 8;      // pooled columns per register block
};

// One column sample: element offsets (x * C) of its two corners, their weights;
// hx == lx == 0 marks a sample that contributes nothing.
struct alignas(16) ColSample { int lo, hi; float hx, lx; };

template <typename T>
__global__ void __launch_bounds__(FwdGather::NT)
forward_gather_kernel(const T* __restrict__ xt, const float* __restrict__ rois, T* __restrict__ y,
                      float scale, int C, int H, int W, int PH, int PW, int S, long long num_images,
                      int cblocks) {
  using K = FwdGather;
  __shared__ ColSample cols[K::MAXC];
  const int roi = blockIdx.x / cblocks, cb = blockIdx.x % cblocks;
  const int c0 = cb * K::CH;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const bool lane_on = c0 + lane < C;
  const int ch = lane_on ? c0 + lane : C - 1;
  const RoiGeom g = roi_geometry(rois + static_cast<long long>(roi) * 5, scale, PH, PW, S);
  const int bins = PH * PW;
  T* const y_lane = y + (static_cast<size_t>(roi) * C + ch) * bins;
  const bool image_ok = g.batch >= 0 && g.batch < num_images;
  const int n_cols = PW * g.grid_w;
  const bool cols_in_lds = n_cols <= K::MAXC;

  if (image_ok && cols_in_lds) {
    for (int s = tid; s < n_cols; s += K::NT) {
      const int pw = s / g.grid_w;
      const AxisSample a = axis_sample(sample_coord(g.start_w, pw, g.bin_w, s - pw * g.grid_w, g.grid_w), W);
      cols[s] = ColSample{a.low * C, a.high * C, a.valid ? a.h : 0.0f, a.valid ? a.l : 0.0f};
    }
  }
  __syncthreads();

  const T* const img = xt + static_cast<size_t>(image_ok ? g.batch : 0) * H * W * C + ch;
  for (int ph = wave; ph < PH; ph += K::NW) {
    for (int pwb = 0; pwb < PW; pwb += K::PWB) {
      float acc[K::PWB];
#pragma unroll
      for (int k = 0; k < K::PWB; ++k) acc[k] = 0.0f;
      if (image_ok) {
        for (int iy = 0; iy < g.grid_h; ++iy) {
          const AxisSample ry = axis_sample(sample_coord(g.start_h, ph, g.bin_h, iy, g.grid_h), H);
          if (!__builtin_amdgcn_readfirstlane(ry.valid ? 1 : 0)) continue;
          const float hy = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(ry.h)));
          const float ly = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(ry.l)));
          const T* const row_lo = img + static_cast<size_t>(__builtin_amdgcn_readfirstlane(ry.low)) * W * C;
          const T* const row_hi = img + static_cast<size_t>(__builtin_amdgcn_readfirstlane(ry.high)) * W * C;
#pragma unroll
          for (int k = 0; k < K::PWB; ++k) {
            const int pw = pwb + k;
            if (pw >= PW) break;
            float part = 0.0f;
            for (int ix = 0; ix < g.grid_w; ++ix) {
              ColSample cs;
              if (cols_in_lds) {
                cs = cols[pw * g.grid_w + ix];
              } else {
                const AxisSample a = axis_sample(sample_coord(g.start_w, pw, g.bin_w, ix, g.grid_w), W);
                cs = ColSample{a.low * C, a.high * C, a.valid ? a.h : 0.0f, a.valid ? a.l : 0.0f};
              }
              const float hx = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(cs.hx)));
              const float lx = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(cs.lx)));
              if (((__float_as_int(hx) | __float_as_int(lx)) << 1) == 0) continue;
              const int lo = __builtin_amdgcn_readfirstlane(cs.lo), hi = __builtin_amdgcn_readfirstlane(cs.hi);
              const float v1 = to_float(row_lo[lo]), v2 = to_float(row_lo[hi]);
              const float v3 = to_float(row_hi[lo]), v4 = to_float(row_hi[hi]);
              part = fmaf(hy, fmaf(hx, v1, lx * v2), part);
              part = fmaf(ly, fmaf(hx, v3, lx * v4), part);
            }
            acc[k] += part;
          }
        }
      }
      if (lane_on) {
#pragma unroll
        for (int k = 0; k < K::PWB; ++k)
          if (pwb + k < PW) y_lane[ph * PW + pwb + k] = from_float<T>(acc[k] / g.count);
      }
    }
  }
}


// ---------------------------------------------------------------------------
// Wide variant of the gather: a lane carries four consecutive channels, so one
// wavefront moves 256 channels of a pixel per load (1 KB for fp32) and sixteen
// such loads are in flight per wavefront.  Results of a workgroup are staged in
// LDS in the layout of y and leave as contiguous 16-byte stores.
// ---------------------------------------------------------------------------
struct FwdGather4 {
  static constexpr int CW = 256;        // channels per workgroup
  static constexpr int MAXW = 8;        // wavefronts per workgroup (tasks in flight)
  static constexpr int MAXS = 512;      // row / column samples held in LDS
  static constexpr int PWB = 8;         // pooled columns per task
  static constexpr int STAGE = 14336;   // staged outputs per pass (elements)
  static constexpr int CELL = 32;       // side of the sorting cells in pixels
  static constexpr int MAXCELLS = 8192;
};

// Pooled rows per pass of forward_gather4_kernel, 0 if the shape does not fit.
inline int gather4_rows_per_pass(int C, int PH, int PW) {
  if (C % 4 != 0 || PW < 1 || FwdGather4::CW * PW > FwdGather4::STAGE) return 0;
  return min(PH, FwdGather4::STAGE / (FwdGather4::CW * PW));
}

// order[] = ROI indices sorted by (image, 32x32-pixel cell of the box centre):
// consecutive workgroups then read neighbouring parts of the map, which is what
// keeps their corner reads in the L2 of the XCD they run on.  One workgroup;
// counting sort with the histogram in LDS.  ROIs of no image sort last.
__global__ void __launch_bounds__(1024)
roi_order_kernel(const float* __restrict__ rois, int R, float scale, int H, int W,
                 long long num_images, int* __restrict__ order) {
  using K = FwdGather4;
  __shared__ int hist[K::MAXCELLS + 1];
  __shared__ int wave_sum[16];
  __shared__ int carry;
  int cell = K::CELL;
  long long cy = (H + cell - 1) / cell, cx = (W + cell - 1) / cell;
  while (cy * cx * num_images > K::MAXCELLS && cell < (1 << 20)) {
    cell *= 2;
    cy = (H + cell - 1) / cell; cx = (W + cell - 1) / cell;
  }
  const int cells = cy * cx * num_images > K::MAXCELLS ? 1 : static_cast<int>(cy * cx * num_images);
  auto key_of = [&](int r) {
    const float* q = rois + static_cast<long long>(r) * 5;
    const int b = static_cast<int>(q[0]);
    if (b < 0 || b >= num_images) return cells;
    if (cells == 1) return 0;
    const float mx = 0.5f * (q[1] + q[3]) * scale, my = 0.5f * (q[2] + q[4]) * scale;
    const int ix = min(max(static_cast<int>(mx), 0), W - 1) / cell;
    const int iy = min(max(static_cast<int>(my), 0), H - 1) / cell;
    // serpentine rows: the end of one row of cells is next to the start of the following one
    const int sx = (iy & 1) ? static_cast<int>(cx) - 1 - ix : ix;
    return static_cast<int>((b * cy + iy) * cx + sx);
  };
  for (int i = threadIdx.x; i <= cells; i += 1024) hist[i] = 0;
  if (threadIdx.x == 0) carry = 0;
  __syncthreads();
  for (int r = threadIdx.x; r < R; r += 1024) atomicAdd(&hist[key_of(r)], 1);
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int base = 0; base <= cells; base += 1024) {
    const int i = base + threadIdx.x;
    const int v = i <= cells ? hist[i] : 0;
    int incl = v;
    for (int off = 1; off < 64; off <<= 1) {
      const int up = __shfl_up(incl, off);
      if (lane >= off) incl += up;
    }
    if (lane == 63) wave_sum[wave] = incl;
    __syncthreads();
    int before = carry;
    for (int w = 0; w < wave; ++w) before += wave_sum[w];
    if (i <= cells) hist[i] = before + incl - v;
    __syncthreads();
    if (threadIdx.x == 1023) carry = before + incl;
    __syncthreads();
  }
  for (int r = threadIdx.x; r < R; r += 1024) order[atomicAdd(&hist[key_of(r)], 1)] = r;
}

// One row sample: element offsets (y * W * C) of its two rows and their weights.
struct alignas(16) RowSample { int lo, hi; float hy, ly; };

template <typename T>
__global__ void __launch_bounds__(FwdGather4::MAXW * 64, 4)
forward_gather4_kernel(const T* __restrict__ xt, const float* __restrict__ rois,
                       const int* __restrict__ order, T* __restrict__ y, float scale, int C, int H,
                       int W, int PH, int PW, int S, long long num_images, int cblocks,
                       int rows_per_pass, long long num_jobs) {
  using K = FwdGather4;
  struct alignas(4 * sizeof(T)) V4 { T v[4]; };
  typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
  __shared__ ColSample cols[K::MAXS];
  __shared__ RowSample rows[K::MAXS];
  __shared__ __attribute__((aligned(16))) T stage[K::STAGE];

  // consecutive jobs go to one XCD (workgroups are dealt to the 8 XCDs round-robin)
  const long long per_xcd = gridDim.x / 8;
  const long long job = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
  if (job >= num_jobs) return;
  const int slot = static_cast<int>(job / cblocks), cb = static_cast<int>(job % cblocks);
  const int roi = order[slot];
  const int c0 = cb * K::CW, nch = min(K::CW, C - c0);
  const int tid = threadIdx.x, lane = tid & 63, nt = blockDim.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), nw = nt >> 6;
  const bool lane_on = 4 * lane < nch;
  const RoiGeom g = roi_geometry(rois + static_cast<long long>(roi) * 5, scale, PH, PW, S);
  const int bins = PH * PW;
  const bool image_ok = g.batch >= 0 && g.batch < num_images;
  const int n_cols = PW * g.grid_w, n_rows = PH * g.grid_h;
  const bool cols_in_lds = n_cols <= K::MAXS, rows_in_lds = n_rows <= K::MAXS;
  const int row_pitch = W * C;

  auto col_sample = [&](int pw, int ix) {
    const AxisSample a = axis_sample(sample_coord(g.start_w, pw, g.bin_w, ix, g.grid_w), W);
    return ColSample{a.low * C, a.high * C, a.h, a.l};
  };
  auto row_sample = [&](int ph, int iy) {
    const AxisSample a = axis_sample(sample_coord(g.start_h, ph, g.bin_h, iy, g.grid_h), H);
    return RowSample{a.low * row_pitch, a.high * row_pitch, a.h, a.l};
  };
  if (image_ok) {
    if (cols_in_lds)
      for (int s = tid; s < n_cols; s += nt) cols[s] = col_sample(s / g.grid_w, s % g.grid_w);
    if (rows_in_lds)
      for (int s = tid; s < n_rows; s += nt) rows[s] = row_sample(s / g.grid_h, s % g.grid_h);
  }
  __syncthreads();

  const T* const img = xt + static_cast<size_t>(image_ok ? g.batch : 0) * H * row_pitch + c0 + 4 * lane;
  const int pwblocks = (PW + K::PWB - 1) / K::PWB;
  auto uni_i = [](int v) { return __builtin_amdgcn_readfirstlane(v); };
  auto uni_f = [](float v) { return __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(v))); };

  for (int ph0 = 0; ph0 < PH; ph0 += rows_per_pass) {
    const int rp = min(rows_per_pass, PH - ph0), seg = rp * PW;
    for (int task = wave; task < rp * pwblocks; task += nw) {
      const int ph = ph0 + task / pwblocks, pwb = (task % pwblocks) * K::PWB;
      float acc[K::PWB][4];
#pragma unroll
      for (int k = 0; k < K::PWB; ++k)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[k][j] = 0.0f;
      if (image_ok && lane_on) {
        // NY x NX samples of one bin at a time: 4 * NY * NX independent loads
        auto block = [&](float (&a)[4], int pw, int iy, int ix, auto ny_tag, auto nx_tag) {
          constexpr int NY = decltype(ny_tag)::value, NX = decltype(nx_tag)::value;
          RowSample rs[NY];
          ColSample cs[NX];
#pragma unroll
          for (int i = 0; i < NY; ++i) {
            const RowSample t = rows_in_lds ? rows[ph * g.grid_h + iy + i] : row_sample(ph, iy + i);
            rs[i] = RowSample{uni_i(t.lo), uni_i(t.hi), uni_f(t.hy), uni_f(t.ly)};
          }
#pragma unroll
          for (int i = 0; i < NX; ++i) {
            const ColSample t = cols_in_lds ? cols[pw * g.grid_w + ix + i] : col_sample(pw, ix + i);
            cs[i] = ColSample{uni_i(t.lo), uni_i(t.hi), uni_f(t.hx), uni_f(t.lx)};
          }
          V4 v[NY][NX][4];
#pragma unroll
          for (int i = 0; i < NY; ++i)
#pragma unroll
            for (int j = 0; j < NX; ++j) {
              v[i][j][0] = *reinterpret_cast<const V4*>(img + rs[i].lo + cs[j].lo);
              v[i][j][1] = *reinterpret_cast<const V4*>(img + rs[i].lo + cs[j].hi);
              v[i][j][2] = *reinterpret_cast<const V4*>(img + rs[i].hi + cs[j].lo);
              v[i][j][3] = *reinterpret_cast<const V4*>(img + rs[i].hi + cs[j].hi);
            }
#pragma unroll
          for (int i = 0; i < NY; ++i)
#pragma unroll
            for (int j = 0; j < NX; ++j) {
              // a sample outside the map contributes nothing whatever the data holds
              const bool live = ((__float_as_int(rs[i].hy) | __float_as_int(rs[i].ly)) << 1) != 0 &&
                                ((__float_as_int(cs[j].hx) | __float_as_int(cs[j].lx)) << 1) != 0;
#pragma unroll
              for (int q = 0; q < 4; ++q) {
                const float top = fmaf(cs[j].hx, to_float(v[i][j][0].v[q]), cs[j].lx * to_float(v[i][j][1].v[q]));
                const float bot = fmaf(cs[j].hx, to_float(v[i][j][2].v[q]), cs[j].lx * to_float(v[i][j][3].v[q]));
                const float val = fmaf(rs[i].ly, bot, rs[i].hy * top);
                a[q] += live ? val : 0.0f;
              }
            }
        };
        using One = std::integral_constant<int, 1>;
        using Two = std::integral_constant<int, 2>;
#pragma unroll
        for (int k = 0; k < K::PWB; ++k) {
          const int pw = pwb + k;
          if (pw >= PW) break;
          int iy = 0;
          for (; iy + 1 < g.grid_h; iy += 2) {
            int ix = 0;
            for (; ix + 1 < g.grid_w; ix += 2) block(acc[k], pw, iy, ix, Two{}, Two{});
            if (ix < g.grid_w) block(acc[k], pw, iy, ix, Two{}, One{});
          }
          if (iy < g.grid_h) {
            int ix = 0;
            for (; ix + 1 < g.grid_w; ix += 2) block(acc[k], pw, iy, ix, One{}, Two{});
            if (ix < g.grid_w) block(acc[k], pw, iy, ix, One{}, One{});
          }
        }
      }
      if (lane_on) {
#pragma unroll
        for (int k = 0; k < K::PWB; ++k)
          if (pwb + k < PW) {
#pragma unroll
            for (int j = 0; j < 4; ++j)
              stage[(4 * lane + j) * seg + (ph - ph0) * PW + pwb + k] = from_float<T>(acc[k][j] / g.count);
          }
      }
    }
    __syncthreads();
    if (rp == PH) {
      // the workgroup's outputs are one contiguous piece of y
      T* const dst = y + (static_cast<size_t>(roi) * C + c0) * bins;
      const int total = nch * bins;
      constexpr int per = 16 / sizeof(T);
      if (reinterpret_cast<size_t>(dst) % 16 == 0) {
        const int nvec = total / per;
        for (int i = tid; i < nvec; i += nt)
          __builtin_nontemporal_store(reinterpret_cast<const u32x4*>(stage)[i], reinterpret_cast<u32x4*>(dst) + i);
        for (int i = nvec * per + tid; i < total; i += nt) dst[i] = stage[i];
      } else {
        for (int i = tid; i < total; i += nt) dst[i] = stage[i];
      }
    } else {
      for (int i = tid; i < nch * seg; i += nt) {
        const int c = i / seg, j = i - c * seg;
        y[(static_cast<size_t>(roi) * C + c0 + c) * bins + ph0 * PW + j] = stage[i];
      }
    }
    if (ph0 + rows_per_pass < PH) __syncthreads();
  }
}

}  // namespace roialign
