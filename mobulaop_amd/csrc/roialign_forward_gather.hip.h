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

}  // namespace roialign
