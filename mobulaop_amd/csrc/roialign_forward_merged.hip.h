// Forward ROIAlign for sampling grids of more than 2 x 2 points per bin
// (sampling_ratio <= 0: ceil(bin size) points per axis; or a ratio above 2).
//
// Same blocked layout of the map, same wavefront-per-(ROI, channel block) job
// and lane roles as forward_blocked_kernel.  What differs is how a bin's
// samples are fetched.  The sum over a bin's gh x gw sample points of four
// weighted corners each is separable,
//     sum_iy sum_ix sum_corners = sum_r wy[r] * (sum_c wx[c] * x[r][c]),
// with wy[r] the total weight the bin's row samples put on map row r and
// wx[c] likewise for columns.  With an adaptive grid neighbouring samples are
// at most one pixel apart, so they share corners: gh samples touch about
// gh + 1 rows, not 2 * gh.  The kernel therefore turns every pooled row's
// samples into a merged list of (row offset, weight) and every pooled column's
// into (column offset, weight), and loads each pixel of the bin once:
// (gh + 1) * (gw + 1) loads instead of 4 * gh * gw.
// Weights of one map row are added in sample order, so results do not depend
// on scheduling; they differ from the per-sample order of the reference by
// rounding only.
#pragma once
#include <type_traits>

#include "roialign_forward_blocked.hip.h"

namespace roialign {

struct FwdMerged {
  static constexpr int LCAP = 24;   // entries per merged list
  static constexpr int WS = 11;     // samples merged per list at a time: at most 2 * WS entries
  static constexpr int RPH = 8;     // pooled rows whose lists are held at a time
  // One wavefront per workgroup: the wavefronts are independent, and a slot is refilled as soon
  // as its wavefront ends instead of when the slowest of four does (boxes differ a lot in work
  // with adaptive grids: cfg4 0.79 -> 0.65 ms).
  static constexpr int NW = 1;
};

// One map row (or column) of a merged list: byte offset and total weight.
struct alignas(8) MergedEntry { int off; float w; };

// Lane-local: merges samples i0 .. i0 + n - 1 of pooled index p along one axis
// into out[]; returns the number of entries.  Sample positions do not decrease
// with i, so a new sample's low corner can only be one of the last two entries
// or a new one, and its high corner only the last entry or a new one.
__device__ __forceinline__ int merge_axis_samples(MergedEntry* out, float start, int p, float bin, int i0,
                                                  int n, int grid, int size, int stride) {
  MergedEntry a{-1, 0.0f}, b{-1, 0.0f};   // second-to-last and last entry, not yet stored
  int count = 0;
  for (int i = i0; i < i0 + n; ++i) {
    const AxisSample s = axis_sample(sample_coord(start, p, bin, i, grid), size);
    if (!s.valid) continue;
    const int lo = s.low * stride, hi = s.high * stride;
    const float wl = s.low == s.high ? s.h + s.l : s.h;
    if (b.off == lo) {
      b.w += wl;
    } else if (a.off == lo) {
      a.w += wl;
    } else {
      if (a.off >= 0) out[count++] = a;
      a = b;
      b = MergedEntry{lo, wl};
    }
    if (s.low != s.high) {
      if (b.off == hi) {
        b.w += s.l;
      } else {
        if (a.off >= 0) out[count++] = a;
        a = b;
        b = MergedEntry{hi, s.l};
      }
    }
  }
  if (a.off >= 0) out[count++] = a;
  if (b.off >= 0) out[count++] = b;
  return count;
}

template <typename T, bool NHWC>
__global__ void __launch_bounds__(FwdMerged::NW * 64, 4)
forward_merged_kernel(const T* __restrict__ xt, const float* __restrict__ rois,
                      const int* __restrict__ order, T* __restrict__ y, float scale, int C, int H,
                      int W, int PH, int PW, int S, long long num_images, int cblk,
                      int rows_per_pass, int R) {
  using K = FwdBlocked;
  using M = FwdMerged;
  constexpr int CPL = BlockOf<T>::CPL, CB = BlockOf<T>::CB, STAGE = BlockOf<T>::STAGE_MERGED;
  typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
  __shared__ MergedEntry rowm_s[M::NW][M::RPH][M::LCAP];
  __shared__ MergedEntry colm_s[M::NW][K::PWB][M::LCAP];
  __shared__ int rown_s[M::NW][M::RPH];
  __shared__ int coln_s[M::NW][K::PWB];
  __shared__ __attribute__((aligned(16))) T stage_s[M::NW][STAGE];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  auto uni_i = [](int v) { return __builtin_amdgcn_readfirstlane(v); };
  auto uni_f = [](float v) { return __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(v))); };
  // job decode: as in forward_blocked_kernel
  const int xcd = blockIdx.x & 7;
  const long long wi = static_cast<long long>(blockIdx.x >> 3) * M::NW + wave;
  long long slot;
  int cb;
  if (NHWC) {
    // the caller's map: an XCD takes an eighth of the (spatially sorted) ROIs, channel
    // block by channel block
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
  const int grp = lane >> 3, quad = lane & 7;
  const bool quad_on = CPL * quad < nch;
  const RoiGeom g = roi_geometry(rois + static_cast<long long>(roi) * 5, scale, PH, PW, S);
  const int bins = PH * PW;
  const int batch = uni_i(g.batch);
  const bool image_ok = batch >= 0 && batch < num_images;
  const int gh = uni_i(g.grid_h), gw = uni_i(g.grid_w);
  // A box far larger than the map (or infinite) has up to 2^31 sample points per
  // bin, nearly all outside the map: forward_large_grid_kernel does those boxes.
  if (gh > kSearchedGrid || gw > kSearchedGrid) return;
  const float inv_count = 1.0f / uni_f(g.count);
  MergedEntry (*const rowm)[M::LCAP] = rowm_s[wave];
  MergedEntry (*const colm)[M::LCAP] = colm_s[wave];
  int* const rown = rown_s[wave];
  int* const coln = coln_s[wave];
  T* const stage = stage_s[wave];
  // NHWC: the caller's [N][H][W][C] map is read where it lies, a pixel's channels C * sizeof(T) apart
  const int px_bytes = (NHWC ? C : CB) * static_cast<int>(sizeof(T)), row_bytes = W * px_bytes;
  const int lane_off = quad * 16;
  constexpr int kDead = static_cast<int>(0x80000000u);

  const size_t image_no = static_cast<size_t>(image_ok ? batch : 0);
  const char* const plane_ptr = reinterpret_cast<const char*>(xt) +
      (NHWC ? image_no * H * row_bytes + static_cast<size_t>(cb) * 128 : (image_no * cblk + cb) * H * row_bytes);
  const __amdgpu_buffer_rsrc_t plane = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<char*>(plane_ptr), 0, H * row_bytes - (NHWC ? cb * 128 : 0), 0x00020000);

  // Lists held in LDS: rows of pooled rows row_p0 .. row_p0 + RPH - 1 for the
  // sample window starting at row_i0 (lane l builds the list of pooled row
  // row_p0 + l), columns of the pooled columns col_p0 .. col_p0 + 7 for the
  // window starting at col_i0.  With grids of up to WS points one build per
  // ROI (and block of pooled rows / columns) covers everything.
  int row_p0 = -1, row_i0 = -1;
  auto need_rows = [&](int ph, int i0) {
    if (i0 != row_i0 || ph < row_p0 || ph >= row_p0 + M::RPH) {
      row_p0 = ph; row_i0 = i0;
      if (lane < M::RPH && ph + lane < PH)
        rown[lane] = merge_axis_samples(rowm[lane], g.start_h, ph + lane, g.bin_h, i0, min(M::WS, gh - i0),
                                        gh, H, row_bytes);
    }
  };
  int col_p0 = -1, col_i0 = -1, col_max = 0;
  auto need_cols = [&](int pwb, int i0) {
    if (pwb != col_p0 || i0 != col_i0) {
      col_p0 = pwb; col_i0 = i0;
      int n = 0;
      if (lane < K::PWB && pwb + lane < PW) {
        n = merge_axis_samples(colm[lane], g.start_w, pwb + lane, g.bin_w, i0, min(M::WS, gw - i0), gw, W,
                               px_bytes);
        coln[lane] = n;
      } else if (lane < K::PWB) {
        coln[lane] = 0;
      }
      for (int off = 4; off > 0; off >>= 1) n = max(n, __shfl_xor(n, off));
      col_max = uni_i(n);
    }
  };

  for (int ph0 = 0; ph0 < PH; ph0 += rows_per_pass) {
    const int rp = min(rows_per_pass, PH - ph0), seg = rp * PW;
    for (int pwb = 0; pwb < PW; pwb += K::PWB) {
      const int pw = pwb + grp;
      const bool bin_on = pw < PW && quad_on;
#pragma nounroll
      for (int ph = ph0; ph < ph0 + rp; ++ph) {
        float acc[CPL];
#pragma unroll
        for (int i = 0; i < CPL; ++i) acc[i] = 0.0f;
        if (image_ok) {
#pragma nounroll
          for (int iyw = 0; iyw < gh; iyw += M::WS) {
            need_rows(ph, iyw);
            const int nr = uni_i(rown[ph - row_p0]);
            const MergedEntry* const rlist = rowm[ph - row_p0];
#pragma nounroll
            for (int ixw = 0; ixw < gw; ixw += M::WS) {
              need_cols(pwb, ixw);
              const int nc = bin_on ? coln[grp] : 0;
              const MergedEntry* const clist = colm[grp];
              // blocks of four map rows (scalar) x four or two map columns (per lane): the columns
              // of a block are decoded once for all its rows; a last block of at most two columns
              // is not padded to four
              auto block = [&](const int (&roff)[4], const float (&rw)[4], const bool (&rlive)[4], const int (&coff)[4],
                               const float (&cw)[4], auto width) {
                constexpr int NC = decltype(width)::value;
                typename LaneData<T>::type v[4][NC];
#pragma unroll
                for (int r = 0; r < 4; ++r)
                  if (rlive[r]) {
#pragma unroll
                    for (int c = 0; c < NC; ++c) v[r][c] = buffer_load_lane<T>(plane, coff[c], roff[r]);
                  }
#pragma unroll
                for (int r = 0; r < 4; ++r)
                  if (rlive[r]) {
                    if constexpr (CPL > NC) {
                      // more channels than columns per lane: the weight of a pixel first, then one
                      // multiply-add per pixel and channel
                      float w[NC];
#pragma unroll
                      for (int c = 0; c < NC; ++c) w[c] = rw[r] * cw[c];
#pragma unroll
                      for (int i = 0; i < CPL; ++i) {
#pragma unroll
                        for (int c = 0; c < NC; ++c) acc[i] = fmaf(w[c], static_cast<float>(v[r][c][i]), acc[i]);
                      }
                    } else {
#pragma unroll
                      for (int i = 0; i < CPL; ++i) {
                        float t = cw[0] * static_cast<float>(v[r][0][i]);
#pragma unroll
                        for (int c = 1; c < NC; ++c) t = fmaf(cw[c], static_cast<float>(v[r][c][i]), t);
                        acc[i] = fmaf(rw[r], t, acc[i]);
                      }
                    }
                  }
              };
#pragma nounroll
              for (int cc = 0; cc < col_max; cc += 4) {
                int coff[4];
                float cw[4];
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                  const MergedEntry e = clist[min(cc + k, M::LCAP - 1)];
                  const bool ok = cc + k < nc;
                  coff[k] = ok ? e.off + lane_off : kDead;
                  cw[k] = ok ? e.w : 0.0f;
                }
                const bool narrow = col_max - cc <= 2;   // (the same for every lane)
#pragma nounroll
                for (int r0 = 0; r0 < nr; r0 += 4) {
                  int roff[4];
                  float rw[4];
                  bool rlive[4];
#pragma unroll
                  for (int k = 0; k < 4; ++k) {
                    const MergedEntry e = rlist[min(r0 + k, nr - 1)];
                    roff[k] = uni_i(e.off); rw[k] = uni_f(e.w);
                    rlive[k] = r0 + k < nr;
                  }
                  if (narrow) block(roff, rw, rlive, coff, cw, std::integral_constant<int, 2>());
                  else block(roff, rw, rlive, coff, cw, std::integral_constant<int, 4>());
                }
              }
            }
          }
        }
        // (the reference divides by the number of samples; multiplying by its reciprocal
        // differs in the last bit only where that number is no power of two)
#pragma unroll
        for (int i = 0; i < CPL; ++i) acc[i] *= inv_count;
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
    }
    if (NHWC) continue;
    // the wavefront's outputs of this pass leave LDS in the order of y
    if (rp == PH) {
      const int total = nch * seg;
      T* const dst = y + (static_cast<size_t>(roi) * C + c0) * bins;
      constexpr int per = 16 / sizeof(T);
      if (reinterpret_cast<size_t>(dst) % 16 == 0) {
        const int nvec = total / per;
        for (int i = lane; i < nvec; i += 64)
          __builtin_nontemporal_store(reinterpret_cast<const u32x4*>(stage)[i], reinterpret_cast<u32x4*>(dst) + i);
        for (int i = nvec * per + lane; i < total; i += 64) dst[i] = stage[i];
      } else {
        for (int i = lane; i < total; i += 64) dst[i] = stage[i];
      }
    } else {
      // some pooled rows of every channel: seg contiguous elements per channel, the lanes cover
      // as many channels at a time as fit (one division per pass, none per element)
      const int chans = max(1, 64 / seg), cl = lane / seg, j0 = lane - cl * seg;
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
          for (int j = lane; j < seg; j += 64)
            y[(static_cast<size_t>(roi) * C + c0 + c) * bins + ph0 * PW + j] = stage[c * seg + j];
      }
    }
  }
}

}  // namespace roialign
