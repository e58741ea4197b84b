// Straightforward ROIAlign kernels: one thread per output element, every
// expression in the reference's order (opzoo/ROIAlign/ROIAlign.cpp:17-75,
// 84-160).  They are the library's correctness anchor on the GPU (bit-close to
// the reference arithmetic, including the order of the four-term weighted sum)
// and the fallback for shapes the tiled kernels do not take.
#pragma once
#include "roialign_geometry.h"

namespace roialign {

template <typename T>
__global__ void __launch_bounds__(256)
forward_naive_kernel(long long n_out, const T* __restrict__ x, float scale, int C, int H, int W,
                     int PH, int PW, int S, const float* __restrict__ rois, T* __restrict__ y,
                     long long num_images) {
  const long long stride = static_cast<long long>(gridDim.x) * blockDim.x;
  const int bins = PH * PW;
  for (long long idx = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x; idx < n_out;
       idx += stride) {
    const int pw = static_cast<int>(idx % PW);
    const int ph = static_cast<int>((idx / PW) % PH);
    const int c = static_cast<int>((idx / bins) % C);
    const long long r = idx / (static_cast<long long>(bins) * C);
    const RoiGeom g = roi_geometry(rois + r * 5, scale, PH, PW, S);
    float acc = 0.0f;
    if (g.batch >= 0 && g.batch < num_images) {
      const T* plane = x + (static_cast<long long>(g.batch) * C + c) * H * W;
      int y0, y1, x0, x1;   // samples outside add nothing
      valid_sample_range(g.start_h, ph, g.bin_h, g.grid_h, H, &y0, &y1);
      valid_sample_range(g.start_w, pw, g.bin_w, g.grid_w, W, &x0, &x1);
      for (int iy = y0; iy < y1; ++iy) {
        const AxisSample sy = axis_sample(sample_coord(g.start_h, ph, g.bin_h, iy, g.grid_h), H);
        for (int ix = x0; ix < x1; ++ix) {
          const AxisSample sx = axis_sample(sample_coord(g.start_w, pw, g.bin_w, ix, g.grid_w), W);
          float val = 0.0f;
          if (sy.valid && sx.valid) {
            const float v1 = to_float(plane[sy.low * W + sx.low]);
            const float v2 = to_float(plane[sy.low * W + sx.high]);
            const float v3 = to_float(plane[sy.high * W + sx.low]);
            const float v4 = to_float(plane[sy.high * W + sx.high]);
            const float w1 = sy.h * sx.h, w2 = sy.h * sx.l, w3 = sy.l * sx.h, w4 = sy.l * sx.l;
            val = w1 * v1 + w2 * v2 + w3 * v3 + w4 * v4;
          }
          acc += val;
        }
      }
    }
    y[idx] = from_float<T>(acc / g.count);
  }
}

// The boxes forward_merged_kernel leaves out: those whose sampling grid has more
// than kSearchedGrid points per bin along an axis.  One wavefront per ROI (it
// returns at once for every other box); its lanes share out the ROI's outputs
// and visit only the samples that can be valid.  NHWC: map [N][H][W][C] and
// pooled tensor [R][PH][PW][C].
template <typename T, bool NHWC>
__global__ void __launch_bounds__(64)
forward_large_grid_kernel(const T* __restrict__ x, float scale, int C, int H, int W, int PH, int PW, int S,
                          const float* __restrict__ rois, T* __restrict__ y, long long num_images) {
  const long long r = blockIdx.x;
  const RoiGeom g = roi_geometry(rois + r * 5, scale, PH, PW, S);
  if (g.grid_h <= kSearchedGrid && g.grid_w <= kSearchedGrid) return;
  const bool image_ok = g.batch >= 0 && g.batch < num_images;
  const int bins = PH * PW;
  for (int o = threadIdx.x; o < C * bins; o += 64) {
    // consecutive lanes take consecutive addresses of y in either layout
    const int c = NHWC ? o % C : o / bins, bin = NHWC ? o / C : o % bins;
    const int ph = bin / PW, pw = bin - ph * PW;
    float acc = 0.0f;
    if (image_ok) {
      int y0, y1, x0, x1;
      valid_sample_range(g.start_h, ph, g.bin_h, g.grid_h, H, &y0, &y1);
      valid_sample_range(g.start_w, pw, g.bin_w, g.grid_w, W, &x0, &x1);
      const long long image = static_cast<long long>(g.batch) * C * H * W;
      auto at = [&](int row, int col) {
        return to_float(x[NHWC ? image + (static_cast<long long>(row) * W + col) * C + c
                               : image + (static_cast<long long>(c) * H + row) * W + col]);
      };
      for (int iy = y0; iy < y1; ++iy) {
        const AxisSample sy = axis_sample(sample_coord(g.start_h, ph, g.bin_h, iy, g.grid_h), H);
        for (int ix = x0; ix < x1; ++ix) {
          const AxisSample sx = axis_sample(sample_coord(g.start_w, pw, g.bin_w, ix, g.grid_w), W);
          if (!(sy.valid && sx.valid)) continue;
          const float w1 = sy.h * sx.h, w2 = sy.h * sx.l, w3 = sy.l * sx.h, w4 = sy.l * sx.l;
          acc += w1 * at(sy.low, sx.low) + w2 * at(sy.low, sx.high) + w3 * at(sy.high, sx.low) +
                 w4 * at(sy.high, sx.high);
        }
      }
    }
    y[r * C * bins + o] = from_float<T>(acc / g.count);
  }
}

// TI: element type of dy; the sums go into an fp32 map.
template <typename TI>
__global__ void __launch_bounds__(256)
backward_naive_kernel(long long n_out, const TI* __restrict__ dy, float scale, int C, int H,
                      int W, int PH, int PW, int S, float* __restrict__ dx,
                      const float* __restrict__ rois, long long num_images) {
  const long long stride = static_cast<long long>(gridDim.x) * blockDim.x;
  const int bins = PH * PW;
  for (long long idx = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x; idx < n_out;
       idx += stride) {
    const int pw = static_cast<int>(idx % PW);
    const int ph = static_cast<int>((idx / PW) % PH);
    const int c = static_cast<int>((idx / bins) % C);
    const long long r = idx / (static_cast<long long>(bins) * C);
    const RoiGeom g = roi_geometry(rois + r * 5, scale, PH, PW, S);
    if (g.batch < 0 || g.batch >= num_images) continue;
    float* plane = dx + (static_cast<long long>(g.batch) * C + c) * H * W;
    const float top = to_float(dy[idx]);
    int y0, y1, x0, x1;   // samples outside add nothing
    valid_sample_range(g.start_h, ph, g.bin_h, g.grid_h, H, &y0, &y1);
    valid_sample_range(g.start_w, pw, g.bin_w, g.grid_w, W, &x0, &x1);
    for (int iy = y0; iy < y1; ++iy) {
      const AxisSample sy = axis_sample(sample_coord(g.start_h, ph, g.bin_h, iy, g.grid_h), H);
      if (!sy.valid) continue;
      for (int ix = x0; ix < x1; ++ix) {
        const AxisSample sx = axis_sample(sample_coord(g.start_w, pw, g.bin_w, ix, g.grid_w), W);
        if (!sx.valid) continue;
        const float w1 = sy.h * sx.h, w2 = sy.h * sx.l, w3 = sy.l * sx.h, w4 = sy.l * sx.l;
        atomicAdd(plane + sy.low * W + sx.low, top * w1 / g.count);
        atomicAdd(plane + sy.low * W + sx.high, top * w2 / g.count);
        atomicAdd(plane + sy.high * W + sx.low, top * w3 / g.count);
        atomicAdd(plane + sy.high * W + sx.high, top * w4 / g.count);
      }
    }
  }
}

// max(batch index)+1 over all ROIs, for callers that did not say how many
// images the feature map holds.
template <typename B>
__global__ void max_batch_kernel(const B* __restrict__ rois, int R, int* __restrict__ out) {
  int m = 0;
  for (int r = blockIdx.x * blockDim.x + threadIdx.x; r < R; r += gridDim.x * blockDim.x)
{
    const B b = rois[static_cast<long long>(r) * 5];   // (an index that is negative, huge or not a number names no image)
    if (b >= static_cast<B>(0) && b < static_cast<B>(2147483520.0)) m = max(m, static_cast<int>(b) + 1);
  }
  for (int off = 32; off > 0; off >>= 1) m = max(m, __shfl_xor(m, off));
  if ((threadIdx.x & 63) == 0) atomicMax(out, m);
}

// Clears n 32-bit words.  Used instead of a memset so that a caller may capture
// the launches of a call into a graph and replay them.
__global__ void __launch_bounds__(256)
zero_words_kernel(unsigned* __restrict__ p, long long n) {
  const long long stride = static_cast<long long>(gridDim.x) * blockDim.x;
  for (long long i = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += stride) p[i] = 0u;
}

// out[i] = in[i] (widened), and the way back, for the 16-bit detour of the
// straightforward backward kernel.
template <typename T>
__global__ void __launch_bounds__(256)
widen_kernel(const T* __restrict__ in, float* __restrict__ out, long long n) {
  const long long stride = static_cast<long long>(gridDim.x) * blockDim.x;
  for (long long i = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += stride)
    out[i] = to_float(in[i]);
}
template <typename T>
__global__ void __launch_bounds__(256)
narrow_kernel(const float* __restrict__ in, T* __restrict__ out, long long n) {
  const long long stride = static_cast<long long>(gridDim.x) * blockDim.x;
  for (long long i = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += stride)
    out[i] = from_float<T>(in[i]);
}

}  // namespace roialign
