// The two gathered products of the convolution (forward, data gradient) with
// bf16 operands in memory.
//
// conv_igemm.hip.h rounds fp32 operands to bf16 on their way into LDS; that mode
// is bound by fetching the fp32 operands (sixteen 4-byte loads per lane and K
// step) and converting them, not by the matrix cores.  Here a pre-pass writes
// bf16 copies laid out so that one K step of a tile is contiguous memory:
//   * the gathered tensor (x for the forward, dy for the data gradient) as
//     [image][channel block][pixel][32 channels], channels padded with zeros to
//     a multiple of 32: the 32 channels of a K step at one pixel are 64
//     contiguous bytes, and neighbouring pixels follow;
//   * the weights as [K step][row][32 channels] (rows and channels padded with
//     zeros): the rows of a tile in one K step are one contiguous run.
// (With rows of a K step a large power-of-two stride apart -- [row][K] weights,
// [pixel][channel] activations -- all rows of a step fall into four of an L2's
// sixteen channels, and the product runs at the pace of those four.)
//
// K runs in steps of 32 channels, the taps of a channel block one after the other
// (step = block * taps + tap): the taps of a block read the same 64-byte pieces of
// the same pixels, so after the first tap a step's gathered operand comes from
// the L1 and L2 caches.  A workgroup owns a tile of 256 x 256: eight wavefronts
// of 128 x 64 (4 x 2 accumulators of v_mfma_f32_32x32x16_bf16, 128 accumulator
// registers, two wavefronts to a SIMD so that one multiplies while the other
// waits; one workgroup per CU), or 128 x 256 with four such wavefronts for
// products of at most 128 rows.  A tile this large needs 64 bytes from memory
// per matrix instruction, half of what 128 x 128 tiles need.
//
// Operands go from memory straight into LDS (buffer loads with the LDS flag,
// 16 bytes per lane: one instruction moves sixteen 64-byte rows), three stages
// deep: while step s is multiplied, step s + 1 has landed or is landing and
// step s + 2 is requested.  No register staging, no LDS store instructions.
// A column in the padding loads from beyond the buffer, which writes zeros.
// LDS rows are 64 bytes with no padding; the four 16-byte chunks of row r sit
// in slots chunk ^ ((r >> 2) & 3), which puts the 16-byte fragment reads of
// sixteen neighbouring rows on all 64 banks, each once.
//
// Split operands (fp32-like results at the matrix cores' bf16 rate): every fp32
// value as two bf16, its head (the value rounded to bf16) and its tail (what the
// head leaves, rounded to bf16), 16 significant bits together.  The pre-passes
// write both in one pass over the fp32 tensor, the tails as a second set of
// planes, and a product walks its K steps three times: head x head, head x tail,
// tail x head (tail x tail is below fp32's own rounding).
//
// Replaces, like conv_igemm.hip.h, the per-image im2col + matrix product of
// opzoo/Convolution/Convolution.py:17-57.
#pragma once
#include "conv_igemm.hip.h"

namespace conv {

struct TileB16 {
  static constexpr int BN = 256, BK = 32, STAGES = 3;
};

typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

// The bf16 a copy holds of v: its head (v rounded to bf16, part 0) or its tail (what the head
// leaves, rounded to bf16, part 1): head + tail carry sixteen significant bits of v.
__device__ __forceinline__ unsigned short bf16_part(float v, int part) {
  const unsigned head = pack_bf16(v, 0.0f) & 0xffffu;
  if (part == 0) return static_cast<unsigned short>(head);
  return static_cast<unsigned short>(pack_bf16(v - __uint_as_float(head << 16), 0.0f));
}
// heads (part 0) or tails (part 1) of two values, packed like pack_bf16
__device__ __forceinline__ unsigned pack_bf16_parts(float lo, float hi, int part) {
  return static_cast<unsigned>(bf16_part(lo, part)) | (static_cast<unsigned>(bf16_part(hi, part)) << 16);
}

// dst[n][c / 32][p][c % 32] = bf16(src[n][c][p]) for c < C, zero for C <= c < Cpad.  One
// workgroup: 64 pixels x 64 channels (two channel blocks) through LDS.  VEC: P is a multiple
// of four and src 16-byte aligned, a lane reads four pixels at a time.  The source is read
// once: its loads leave the caches to the copy that is about to be read.
// tail != 0: a second copy, `tail` halves after the first, holds the tails of the values (what
// their bf16 heads leave).
template <bool VEC>
__global__ void __launch_bounds__(256)
to_blocked_bf16_kernel(const float* __restrict__ src, unsigned short* __restrict__ dst, int C, int Cpad, int P,
                       size_t tail) {
  typedef float f32x4 __attribute__((ext_vector_type(4)));
  __shared__ float tile[64][65];
  const int n = blockIdx.z, c0 = blockIdx.y * 64, p0 = blockIdx.x * 64;
  const float* in = src + static_cast<size_t>(n) * C * P;
  if (VEC) {
    const int q = threadIdx.x & 15, r = threadIdx.x >> 4;   // 16 quads of pixels, 16 channels per pass
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int c = c0 + r + 16 * k, p = p0 + 4 * q;
      f32x4 v = {0.0f, 0.0f, 0.0f, 0.0f};
      if (c < C && p < P)
        v = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(in + static_cast<size_t>(c) * P + p));
#pragma unroll
      for (int i = 0; i < 4; ++i) tile[r + 16 * k][4 * q + i] = v[i];
    }
  } else {
    const int px = threadIdx.x & 63, cr = threadIdx.x >> 6;
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      const int c = c0 + cr + 4 * k, p = p0 + px;
      tile[cr + 4 * k][px] = (c < C && p < P) ? in[static_cast<size_t>(c) * P + p] : 0.0f;
    }
  }
  __syncthreads();
  // a thread: one pixel, 8 channels (16 bytes); four threads cover a pixel of one channel block
  const int cq = threadIdx.x & 3, pl = (threadIdx.x >> 2) & 63;
#pragma unroll
  for (int k = 0; k < 2; ++k) {   // the two channel blocks
    const int p = p0 + pl, cl = 32 * k + 8 * cq, c = c0 + cl;
    if (p < P && c < Cpad) {
      u32x4 v;
#pragma unroll
      for (int j = 0; j < 4; ++j) v[j] = pack_bf16(tile[cl + 2 * j][pl], tile[cl + 2 * j + 1][pl]);
      unsigned short* const to = dst + ((static_cast<size_t>(n) * (Cpad / 32) + c / 32) * P + p) * 32 + 8 * cq;
      *reinterpret_cast<u32x4*>(to) = v;
      if (tail != 0) {
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = pack_bf16_parts(tile[cl + 2 * j][pl], tile[cl + 2 * j + 1][pl], 1);
        *reinterpret_cast<u32x4*>(to + tail) = v;
      }
    }
  }
}

// out[(c / 32) * taps + tap][m][c % 32] = bf16(w[m * stride_m + c * stride_c + tap]) for m < M and
// c < C, else 0 (m < Mpad, c < Cpad).  tail != 0: three copies `tail` halves apart, heads, heads
// again and tails (what the bf16 heads leave): the weights of the three passes of a product with
// split operands, one after the other like the K steps that read them.
__global__ void __launch_bounds__(256)
arrange_weights_bf16_kernel(const float* __restrict__ w, unsigned short* __restrict__ out, int M, int Mpad,
                            int C, int Cpad, int taps, long long stride_m, long long stride_c, size_t tail) {
  const long long total = static_cast<long long>(Mpad) * taps * Cpad / 2;   // pairs of channels
  const long long i = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const int j = 2 * static_cast<int>(i % 16), m = static_cast<int>((i / 16) % Mpad);
  const int s = static_cast<int>(i / (16ll * Mpad));
  const int cb = s / taps, tap = s - cb * taps, c = cb * 32 + j;
  const float lo = (m < M && c < C) ? w[m * stride_m + c * stride_c + tap] : 0.0f;
  const float hi = (m < M && c + 1 < C) ? w[m * stride_m + (c + 1) * stride_c + tap] : 0.0f;
  reinterpret_cast<unsigned*>(out)[i] = pack_bf16(lo, hi);
  if (tail != 0) {
    reinterpret_cast<unsigned*>(out + tail)[i] = pack_bf16(lo, hi);
    reinterpret_cast<unsigned*>(out + 2 * tail)[i] = pack_bf16_parts(lo, hi, 1);
  }
}

__device__ __forceinline__ __amdgpu_buffer_rsrc_t buffer_of_bytes(const void* base, unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, static_cast<int>(bytes), 0x00020000);
}

// Row coordinate of a column that does not exist: fails every bounds test, whatever tap is added.
constexpr int kFarOutside = -(1 << 30);

// A K step as (filter row, filter column, channel block); wavefront-uniform, kept in scalar registers.
struct StepCursor { int kh, kw, cb, pass; };

// What the operand functors of igemm_tile_b16 have in common: the weights and the walk over K.
struct GatheredB16 {
  const unsigned short* __restrict__ wp;    // [K / 32][mpad][32]
  const unsigned short* __restrict__ src;   // [sets][images][cpad / 32][pixels][32]
  // K: what the tile loop runs over.  Plain bf16 operands: K = taps * cpad, one set of source
  // planes.  Split operands (source_tail != 0; two bf16 for every fp32, head and tail): K is three
  // times that, the steps three times over -- weight heads x source heads, weight heads x source
  // tails, weight tails x source heads -- with the weights of the three passes one after the other
  // in wp and the source's tails `source_tail` bytes after its heads.
  Geometry g; int M, Ncols, K, cpad, mpad, source_tail;
  __device__ int steps_of_a_pass() const { return g.KH * g.KW * (cpad / 32); }
  __device__ __amdgpu_buffer_rsrc_t a_buffer() const {
    return buffer_of_bytes(wp, static_cast<unsigned>(mpad) * static_cast<unsigned>(K) * 2u);
  }
  __device__ int a_offset(int m) const { return m * 64; }
  typedef StepCursor Cursor;
  __device__ StepCursor cursor(int s) const {
    const int pass = s / steps_of_a_pass(), s1 = s - pass * steps_of_a_pass();
    const int taps = g.KH * g.KW, cb = s1 / taps, tap = s1 - cb * taps, kh = tap / g.KW;
    return StepCursor{kh, tap - kh * g.KW, cb, pass};
  }
  __device__ void advance(StepCursor& c) const {
    if (++c.kw == g.KW) {
      c.kw = 0;
      if (++c.kh == g.KH) {
        c.kh = 0;
        if (++c.cb == cpad / 32) { c.cb = 0; ++c.pass; }
      }
    }
  }
  // byte offset of the set of source planes that the cursor's pass reads
  __device__ int source_set_bytes(const StepCursor& c) const { return c.pass == 1 ? source_tail : 0; }
  // the images from the one column n0 lies in, as a raw buffer
  __device__ __amdgpu_buffer_rsrc_t images_from(int first, size_t image_bytes) const {
    const size_t skip = static_cast<size_t>(first) * image_bytes;
    const size_t left = static_cast<size_t>(source_tail != 0 ? 2 : 1) * g.N * image_bytes - skip;
    return buffer_of_bytes(reinterpret_cast<const char*>(src) + skip,
                           static_cast<unsigned>(left < kRecordLimit ? left : kRecordLimit));
  }
};

// Operand functors of igemm_tile_b16:
//   Cursor cursor(s) / advance(cursor): the walk over the K steps;
//   Step step_at(cursor, s): what a K step adds to every row's and column's offset (uniform);
//   a_buffer() / a_offset(m): the left operand and the byte offset of row m in a K step;
//   b_buffer(n0): the gathered tensor from the first image of the tile on;
//   BCtx b_ctx(n, n0): what column n needs throughout;
//   b_offset(ctx, step, chunk): byte offset of the column's 16-byte chunk in that buffer (kDead: zeros);
//   Column column(n) / store(column, m, v): where results of column n go.

// y[img, d, oh, ow] = bias[d] + sum over (c, kh, kw) of W[d, c, kh, kw] * x[img, c, ih, iw]
struct ForwardOpsB16 : GatheredB16 {
  const float* __restrict__ bias; float* __restrict__ y;
  struct Step { int dh, dw, delta, a_delta; };
  struct BCtx { int anchor, ih0, iw0; };   // (a column past the last: ih0 far outside)
  struct Column { float* p; bool ok; };
  __device__ int plane_bytes() const { return g.H * g.W * 64; }
  __device__ Step step_at(const StepCursor& c, int s) const {
    const int dh = c.kh * g.dil_h, dw = c.kw * g.dil_w;
    return Step{dh, dw, c.cb * plane_bytes() + (dh * g.W + dw) * 64 + source_set_bytes(c), s * mpad * 64};
  }
  __device__ __amdgpu_buffer_rsrc_t b_buffer(int n0) const {
    return images_from(__builtin_amdgcn_readfirstlane(n0 / (g.OH * g.OW)), static_cast<size_t>(plane_bytes()) * (cpad / 32));
  }
  __device__ BCtx b_ctx(int n, int n0) const {
    BCtx c;
    const int ohw = g.OH * g.OW, first = n0 / ohw;
    const int img = n / ohw, r = n - img * ohw, oh = r / g.OW, ow = r - oh * g.OW;
    c.ih0 = n < Ncols ? oh * g.stride_h - g.pad_h : kFarOutside;
    c.iw0 = ow * g.stride_w - g.pad_w;
    c.anchor = (img - first) * plane_bytes() * (cpad / 32) + (c.ih0 * g.W + c.iw0) * 64;
    return c;
  }
  __device__ int b_offset(const BCtx& c, const Step& e, int chunk) const {
    const int ih = c.ih0 + e.dh, iw = c.iw0 + e.dw;
    const bool in = (static_cast<unsigned>(ih) < static_cast<unsigned>(g.H)) &
                    (static_cast<unsigned>(iw) < static_cast<unsigned>(g.W));
    return in ? c.anchor + e.delta + chunk * 16 : kDead;
  }
  __device__ Column column(int n) const {
    const int ohw = g.OH * g.OW, img = n / ohw, r = n - img * ohw;
    return Column{y + static_cast<size_t>(img) * g.D * ohw + r, n < Ncols};
  }
  __device__ void store(const Column& c, int m, float v) const {
    if (m < M && c.ok) c.p[static_cast<size_t>(m) * (g.OH * g.OW)] = bias != nullptr ? v + bias[m] : v;
  }
};

// dx[img, c, ih, iw] = sum over (d, kh, kw) of W[d, c, kh, kw] * dy[img, d, oh, ow]
// with oh * stride = ih + pad - kh * dil (and likewise for columns).
struct BackwardDataOpsB16 : GatheredB16 {
  float* __restrict__ dx; int accumulate;
  struct Step { int dh, dw, delta, a_delta; };
  struct BCtx { int anchor, ihp, iwp; };   // (a column past the last: ihp far outside)
  struct Column { float* p; bool ok; };
  __device__ bool unit_stride() const { return g.stride_h == 1 && g.stride_w == 1; }
  __device__ int plane_bytes() const { return g.OH * g.OW * 64; }
  __device__ Step step_at(const StepCursor& c, int s) const {
    const int dh = c.kh * g.dil_h, dw = c.kw * g.dil_w;
    // stride 1: the tap's offset from the anchor pixel (ih + pad, iw + pad) of dy
    return Step{dh, dw, c.cb * plane_bytes() - (unit_stride() ? (dh * g.OW + dw) * 64 : 0) + source_set_bytes(c),
                s * mpad * 64};
  }
  __device__ __amdgpu_buffer_rsrc_t b_buffer(int n0) const {
    return images_from(__builtin_amdgcn_readfirstlane(n0 / (g.H * g.W)), static_cast<size_t>(plane_bytes()) * (cpad / 32));
  }
  __device__ BCtx b_ctx(int n, int n0) const {
    BCtx c;
    const int hw = g.H * g.W, first = n0 / hw;
    const int img = n / hw, r = n - img * hw, ih = r / g.W, iw = r - ih * g.W;
    c.ihp = n < Ncols ? ih + g.pad_h : kFarOutside; c.iwp = iw + g.pad_w;
    // stride 1: byte offset of dy[img, block 0, ihp, iwp]; otherwise of dy[img, block 0, 0, 0]
    c.anchor = (img - first) * plane_bytes() * (cpad / 32) + (unit_stride() ? (c.ihp * g.OW + c.iwp) * 64 : 0);
    return c;
  }
  __device__ int b_offset(const BCtx& c, const Step& e, int chunk) const {
    const int th = c.ihp - e.dh, tw = c.iwp - e.dw;
    if (unit_stride()) {
      const bool in = (static_cast<unsigned>(th) < static_cast<unsigned>(g.OH)) &
                      (static_cast<unsigned>(tw) < static_cast<unsigned>(g.OW));
      return in ? c.anchor + e.delta + chunk * 16 : kDead;
    }
    const int oh = th / g.stride_h, ow = tw / g.stride_w;
    const bool in = (th >= 0) & (tw >= 0) & (oh * g.stride_h == th) & (ow * g.stride_w == tw) &
                    (oh < g.OH) & (ow < g.OW);
    return in ? c.anchor + e.delta + (oh * g.OW + ow) * 64 + chunk * 16 : kDead;
  }
  __device__ Column column(int n) const {
    const int hw = g.H * g.W, img = n / hw, r = n - img * hw;
    return Column{dx + static_cast<size_t>(img) * g.C * hw + r, n < Ncols};
  }
  __device__ void store(const Column& c, int m, float v) const {
    if (m >= M || !c.ok) return;
    float* p = c.p + static_cast<size_t>(m) * (g.H * g.W);
    *p = accumulate ? *p + v : v;
  }
};

// ---- the weight gradient as shifted plain products ---------------------------------------
//
// With unit strides, dW[d, c, kh, kw] = sum over images and output pixels of
// dy[d, oh, ow] * x[c, oh - pad + kh * dil, ow - pad + kw * dil].  On a common grid of
// Hg x Wg = (H + 2 pad_h) x (W + 2 pad_w) positions per plane -- x placed at (pad_h, pad_w),
// dy at (0, 0), zeros elsewhere -- this is, for every tap, a plain matrix product over the grid
// positions g of all images: dW_tap[d, c] = sum_g dyg[d, g] * xg[c, g + kh * dil_h * Wg + kw * dil_w].
// Where dyg is zero (outside the outputs, and in the tail that pads a plane to a multiple of
// 32 positions) it does not matter what the shifted read of xg finds, as long as it is finite:
// the next plane, or zeros beyond the buffer.  The positions are the K of the product, 32 to a
// step, contiguous in memory for every row (filter d) and column (channel c, tap): the same
// tile as for the gathered products applies, K cut into pieces that fill the device, the pieces
// summed in order afterwards.  Loads of four bytes and more need an even position: taps with
// an odd shift read a second copy of xg that is shifted by one position.
//
// Replaces the second im2col + product of opzoo/Convolution/Convolution.py:44-57.

// dst[plane][g] = bf16(src[plane][gh - off_h][gw - off_w]) for g = gh * Wg + gw < Hg * Wg with the
// source position inside H x W, zero elsewhere (g < Gp, a multiple of 8); shifted[plane][g] =
// dst[plane][g + 1] (shifted may be null).  A workgroup: `span` positions of a plane (a multiple of
// 8, at most kPaddedSpan; blockIdx.y counts the spans of a plane); neighbouring lanes read
// neighbouring positions, the bf16 values go through LDS and leave 16 bytes per lane.
constexpr int kPaddedSpan = 4096;
__global__ void __launch_bounds__(256)
to_padded_bf16_kernel(const float* __restrict__ src, unsigned short* __restrict__ dst,
                      unsigned short* __restrict__ shifted, int H, int W, int off_h, int off_w, int Hg, int Wg,
                      int Gp, int span, size_t tail) {
  // (tail != 0: the tails of the values as a second set of planes, `tail` halves after the heads)
  __shared__ __attribute__((aligned(16))) unsigned short vals_s[2][kPaddedSpan + 8];
  const int plane = blockIdx.x, base = blockIdx.y * span;
  const float* in = src + static_cast<size_t>(plane) * H * W;
  auto value_at = [&](int gh, int gw) {
    const int ih = gh - off_h, iw = gw - off_w;
    const bool inside = (gh < Hg) & (static_cast<unsigned>(ih) < static_cast<unsigned>(H)) &
                        (static_cast<unsigned>(iw) < static_cast<unsigned>(W));
    return inside ? __builtin_nontemporal_load(in + (inside ? ih * W + iw : 0)) : 0.0f;
  };
  const int step_h = 256 / Wg, step_w = 256 - step_h * Wg;   // 256 positions further on
  int g = base + threadIdx.x, gh = g / Wg, gw = g - gh * Wg;
  for (int j = threadIdx.x; j <= span; j += 256) {   // (position base + span: for the shifted copy)
    const float v = value_at(gh, gw);
    vals_s[0][j] = bf16_part(v, 0);
    if (tail != 0) vals_s[1][j] = bf16_part(v, 1);
    gh += step_h; gw += step_w;
    if (gw >= Wg) { gw -= Wg; ++gh; }
  }
  __syncthreads();
  for (int part = 0; part < (tail != 0 ? 2 : 1); ++part) {
    const unsigned short* const vals = vals_s[part];
    for (int j = 8 * threadIdx.x; j < span; j += 8 * 256) {
      const int g0 = base + j;
      if (g0 >= Gp) break;
      const u32x4 a = *reinterpret_cast<const u32x4*>(vals + j);
      const size_t at = static_cast<size_t>(plane) * Gp + g0 + part * tail;
      *reinterpret_cast<u32x4*>(dst + at) = a;
      if (shifted != nullptr) {
        const unsigned next = vals[j + 8];
        u32x4 b;
#pragma unroll
        for (int k = 0; k < 4; ++k) b[k] = (a[k] >> 16) | ((k < 3 ? a[k + 1] : next) << 16);
        *reinterpret_cast<u32x4*>(shifted + at) = b;
      }
    }
  }
}

// The same copy for planes whose rows are a multiple of four elements long and 16-byte aligned
// (VEC4 of the launcher): a workgroup takes `rows` whole grid rows (rows * Wg <= kPaddedSpan; the
// last span also the tail up to Gp), reads the source rows under them sixteen bytes per lane --
// they are one contiguous run -- and drops the values at their grid positions in LDS, which was
// zeroed first; LDS then leaves as above.  (With 4-byte loads the copy runs at 3.5 TB/s, with
// 16-byte loads as fast as the other layout copies.)
__global__ void __launch_bounds__(256)
to_padded_bf16_rows_kernel(const float* __restrict__ src, unsigned short* __restrict__ dst,
                           unsigned short* __restrict__ shifted, int H, int W, int off_h, int off_w, int Hg,
                           int Wg, int Gp, int rows, size_t tail) {
  typedef float f32x4 __attribute__((ext_vector_type(4)));
  __shared__ __attribute__((aligned(16))) unsigned short vals_s[2][kPaddedSpan + 8];
  const int plane = blockIdx.x, r0 = blockIdx.y * rows, r1 = min(r0 + rows, Hg);
  const bool last = (blockIdx.y + 1) * rows >= Hg;
  const int base = r0 * Wg, end = last ? Gp : r1 * Wg, count = end - base;   // (multiples of 8: the launcher sees to it)
  const int parts = tail != 0 ? 2 : 1;
  for (int part = 0; part < parts; ++part)
    for (int j = 4 * threadIdx.x; j < count + 8; j += 4 * 256) *reinterpret_cast<unsigned long long*>(vals_s[part] + j) = 0ull;
  __syncthreads();
  const float* in = src + static_cast<size_t>(plane) * H * W;
  const int ih0 = max(r0 - off_h, 0), ih1 = min(r1 - off_h, H);   // source rows under the span
  for (int i = ih0 * W + 4 * threadIdx.x; i < ih1 * W; i += 4 * 256) {
    const f32x4 v = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(in + i));
    const int ih = i / W, iw = i - ih * W;   // (four elements of one row: W is a multiple of four)
    const int at = (ih + off_h) * Wg + iw + off_w - base;
#pragma unroll
    for (int k = 0; k < 4; ++k) vals_s[0][at + k] = bf16_part(v[k], 0);
    if (tail != 0) {
#pragma unroll
      for (int k = 0; k < 4; ++k) vals_s[1][at + k] = bf16_part(v[k], 1);
    }
  }
  if (threadIdx.x == 0 && !last) {   // the position after the span, for the shifted copy
    const int ih = r1 - off_h, iw = -off_w;
    if (ih >= 0 && ih < H && iw >= 0 && iw < W) {
      vals_s[0][count] = bf16_part(in[ih * W + iw], 0);
      if (tail != 0) vals_s[1][count] = bf16_part(in[ih * W + iw], 1);
    }
  }
  __syncthreads();
  for (int part = 0; part < parts; ++part) {
    const unsigned short* const vals = vals_s[part];
    for (int j = 8 * threadIdx.x; j < count; j += 8 * 256) {
      const u32x4 a = *reinterpret_cast<const u32x4*>(vals + j);
      const size_t at = static_cast<size_t>(plane) * Gp + base + j + part * tail;
      *reinterpret_cast<u32x4*>(dst + at) = a;
      if (shifted != nullptr) {
        const unsigned next = vals[j + 8];
        u32x4 b;
#pragma unroll
        for (int k = 0; k < 4; ++k) b[k] = (a[k] >> 16) | ((k < 3 ? a[k + 1] : next) << 16);
        *reinterpret_cast<u32x4*>(shifted + at) = b;
      }
    }
  }
}

// Rows: filters d; columns: (tap, channel), tap-major; K: (image, grid position).
struct WeightGradOpsB16 {
  const unsigned short* __restrict__ dyg;   // [sets][N][D][Gp]
  const unsigned short* __restrict__ xg;    // [2][sets][N][C][Gp], the second copy shifted by one position
  float* __restrict__ dw;
  Geometry g; int M, Ncols, K, Gp, Wg, accumulate; unsigned copy_bytes;
  // split != 0: dyg and xg hold two sets of planes each, heads then tails of the operands (two
  // bf16 for every fp32), and K runs over the images three times: dy heads x x heads, dy heads x
  // x tails, dy tails x x heads
  int split;
  struct Cursor { int n, j, pass; };   // image, K step within the image, pass over the images
  struct Step { int delta, a_delta; };
  struct BCtx { int anchor; };   // (kDead for a column past the last)
  struct Column { float* p; bool ok; };
  __device__ __amdgpu_buffer_rsrc_t a_buffer() const {
    return buffer_of_bytes(dyg, static_cast<unsigned>(split ? 2 : 1) * g.N * g.D * Gp * 2u);
  }
  __device__ int a_offset(int m) const { return m * Gp * 2; }
  __device__ Cursor cursor(int s) const {
    const int per_image = Gp / TileB16::BK, n = s / per_image, pass = n / g.N;
    return Cursor{n - pass * g.N, s - n * per_image, pass};
  }
  __device__ void advance(Cursor& c) const {
    if (++c.j == Gp / TileB16::BK) {
      c.j = 0;
      if (++c.n == g.N) { c.n = 0; ++c.pass; }
    }
  }
  __device__ Step step_at(const Cursor& c, int) const {
    const int nx = c.n + (c.pass == 1 ? g.N : 0), ny = c.n + (c.pass == 2 ? g.N : 0);   // which set of planes
    return Step{(nx * g.C * Gp + c.j * TileB16::BK) * 2, (ny * g.D * Gp + c.j * TileB16::BK) * 2};
  }
  __device__ __amdgpu_buffer_rsrc_t b_buffer(int) const { return buffer_of_bytes(xg, 2u * copy_bytes); }
  __device__ BCtx b_ctx(int n, int) const {
    const int tap = n / g.C, c = n - tap * g.C, kh = tap / g.KW, kw = tap - kh * g.KW;
    const int shift = kh * g.dil_h * Wg + kw * g.dil_w, odd = shift & 1;
    return BCtx{n < Ncols ? static_cast<int>(odd * copy_bytes) + (c * Gp + shift - odd) * 2 : kDead};
  }
  // (kDead plus the offsets of a step stays beyond every buffer)
  __device__ int b_offset(const BCtx& c, const Step& e, int chunk) const { return c.anchor + e.delta + chunk * 16; }
  __device__ Column column(int n) const {
    const int tap = n / g.C, c = n - tap * g.C;
    return Column{dw + static_cast<size_t>(c) * (g.KH * g.KW) + tap, n < Ncols};
  }
  __device__ void store(const Column& c, int m, float v) const {
    if (m >= M || !c.ok) return;
    float* p = c.p + static_cast<size_t>(m) * g.C * (g.KH * g.KW);
    *p = accumulate ? *p + v : v;
  }
};

// s_waitcnt vmcnt(n), the other counters left alone (gfx9 encoding of the immediate)
template <int N>
__device__ __forceinline__ void wait_for_loads_but() {
  __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));
}

__host__ __device__ inline int k_steps_b16(int K) { return (K + TileB16::BK - 1) / TileB16::BK; }

// A tile of ROWS x COLS results and the WAVES wavefronts that share it, each NI x NJ fragments of
// 32 x 32.  A stage in LDS always has room for 256 columns.
template <int ROWS_, int COLS_, int WAVES_, int NI_>
struct ShapeB16 {
  static constexpr int ROWS = ROWS_, COLS = COLS_, WAVES = WAVES_, NI = NI_;
  static constexpr int WM = ROWS / (32 * NI), WN = WAVES / WM;   // wavefronts down and across the tile
  static constexpr int NJ = COLS / WN / 32;
  static_assert(WM * NI * 32 == ROWS && WN * NJ * 32 == COLS && COLS <= TileB16::BN, "the wavefronts cover the tile");
  static constexpr int STAGE_HALVES = (ROWS + TileB16::BN) * TileB16::BK;
};
typedef ShapeB16<256, 256, 8, 4> WideShapeB16;     // 2 x 4 wavefronts of 128 x 64: two to a SIMD
typedef ShapeB16<128, 256, 4, 4> LowShapeB16;      // 1 x 4 wavefronts of 128 x 64, for products of at most 128 rows

// C[M, Ncols] = A[M, K] x B[K, Ncols], the tile of shape S at (m0, n0) over the K steps
// s_begin .. s_end - 1 (s_begin < s_end).  piece == nullptr: results go through ops.store;
// otherwise into the dense ROWS x 256 piece.
template <typename Ops, typename S>
__device__ __forceinline__ void igemm_tile_b16(const Ops& ops, int m0, int n0, int s_begin, int s_end,
                                               float* __restrict__ piece) {
  using T = TileB16;
  constexpr int ROWS = S::ROWS, WAVES = S::WAVES, NI = S::NI, NJ = S::NJ, WN = S::WN;
  constexpr int A_LOADS = ROWS / 16 / WAVES, B_LOADS = T::BN / 16 / WAVES, LOADS = A_LOADS + B_LOADS;
  constexpr int STAGE = S::STAGE_HALVES;
  __shared__ __attribute__((aligned(1024))) unsigned short lds[T::STAGES * STAGE];
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = (wave / WN) * (32 * NI), wn = (wave % WN) * (32 * NJ);   // the wavefront's part of the tile

  // ---- loading: an instruction moves 16 rows x 64 bytes into LDS, lane l to byte 16 * l of them;
  // the lane's chunk of its row is the one that belongs in that slot
  const int l_row = lane >> 2, l_chunk = (lane & 3) ^ ((lane >> 4) & 3);
  const __amdgpu_buffer_rsrc_t a_buf = ops.a_buffer(), b_buf = ops.b_buffer(n0);
  const int a_off = ops.a_offset(m0 + 16 * A_LOADS * wave + l_row) + l_chunk * 16;
  typename Ops::BCtx bctx[B_LOADS];
#pragma unroll
  for (int k = 0; k < B_LOADS; ++k) {   // (columns of the stage past the tile's: none)
    const int column = 16 * (B_LOADS * wave + k) + l_row;
    bctx[k] = ops.b_ctx(column < S::COLS ? n0 + column : 0x7fffffff, n0);
  }

  // Requests for the next K step (one step after the other): request(k) is load k of the LOADS a
  // wavefront contributes, step_requested() closes the step.  Past the last step the loads are
  // aimed beyond the buffers and bring zeros into a stage nobody reads: the loop body stays free
  // of branches and every step leaves the same number of loads in flight.
  typename Ops::Cursor cur = ops.cursor(s_begin);
  int s_issue = s_begin, stage_issue = 0;
  auto request = [&](int k) {
    unsigned short* const base = lds + stage_issue * STAGE;
    const int dead = s_issue < s_end ? 0 : kDead;
    const typename Ops::Step e = ops.step_at(cur, s_issue);
    if (k < A_LOADS) {
      __builtin_amdgcn_raw_ptr_buffer_load_lds(a_buf, base + 16 * (A_LOADS * wave + k) * 32, 16, a_off | dead,
                                               (s_issue < s_end ? e.a_delta : 0) + k * ops.a_offset(16), 0, 0);
    } else {
      const int kb = k - A_LOADS;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(b_buf, base + (ROWS + 16 * (B_LOADS * wave + kb)) * 32, 16,
                                               ops.b_offset(bctx[kb], e, l_chunk) | dead, 0, 0, 0);
    }
  };
  auto step_requested = [&]() {
    ops.advance(cur);
    ++s_issue;
    stage_issue = stage_issue + 1 == T::STAGES ? 0 : stage_issue + 1;
  };

  float16v acc[NI][NJ];
#pragma unroll
  for (int i = 0; i < NI; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  // ---- reading: fragment = rows base + col, K chunk 2 * kc + half (8 halves of a row) ----
  const int half = lane >> 5, col = lane & 31, sw = (col >> 2) & 3;
  int rd_a[2], rd_b[2];   // in halves
#pragma unroll
  for (int kc = 0; kc < 2; ++kc) {
    const int slot = (2 * kc + half) ^ sw;
    rd_a[kc] = (wm + col) * 32 + slot * 8;
    rd_b[kc] = (ROWS + wn + col) * 32 + slot * 8;
  }
  bf16x8 fa[2][NI], fb[2][NJ];
  // fragment reads of a chunk in the order the products below first need them: a0 b0 b1 .. a1 a2 ..
  constexpr int READS = NI + NJ;
  auto read_fragment = [&](int stage, int kc, int k) {
    const unsigned short* const base = lds + stage * STAGE;
    if (k == 0 || k > NJ) {
      const int i = k == 0 ? 0 : k - NJ;
      fa[kc][i] = *reinterpret_cast<const bf16x8*>(base + rd_a[kc] + i * 32 * 32);
    } else {
      fb[kc][k - 1] = *reinterpret_cast<const bf16x8*>(base + rd_b[kc] + (k - 1) * 32 * 32);
    }
  };
  auto multiply = [&](int kc, int k) {   // product k of the 4 * NJ of a chunk
    const int i = k / NJ, j = k % NJ;
    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[kc][i], fb[kc][j], acc[i][j], 0, 0, 0);
  };

  // One K step: each of its 8 * NJ matrix instructions occupies the matrix pipeline for 32
  // cycles, and whatever else the step needs is issued in their shadow, spread evenly over them
  // (the scheduling barriers pin that order):
  //   first half:  products of chunk 0 of stage s | fragment reads of chunk 1
  //   wait for stage s + 1 (all loads but those of later stages), barrier
  //   second half: products of chunk 1 | requests for stage s + STAGES - 1 (its LDS was stage
  //                s - 1, read by everyone before the barrier) | fragment reads of chunk 0 of
  //                stage s + 1
  constexpr int SLOTS = NI * NJ, ITEMS = LOADS + READS;   // products of a half step; what the second half issues besides
#pragma unroll
  for (int k = 0; k < T::STAGES - 1; ++k) {
#pragma unroll
    for (int q = 0; q < LOADS; ++q) request(q);
    step_requested();
  }
  wait_for_loads_but<(T::STAGES - 2) * LOADS>();
  __syncthreads();
  int stage = 0;
#pragma unroll
  for (int k = 0; k < READS; ++k) read_fragment(0, 0, k);
  for (int s = s_begin; s < s_end; ++s) {
    const int next = stage + 1 == T::STAGES ? 0 : stage + 1;
#pragma unroll
    for (int k = 0; k < SLOTS; ++k) {
      multiply(0, k);
#pragma unroll
      for (int q = k * READS / SLOTS; q < (k + 1) * READS / SLOTS; ++q) read_fragment(stage, 1, q);
      __builtin_amdgcn_sched_barrier(0);
    }
    wait_for_loads_but<(T::STAGES - 3) * LOADS>();
    __syncthreads();
#pragma unroll
    for (int k = 0; k < SLOTS; ++k) {
      multiply(1, k);
#pragma unroll
      for (int q = k * ITEMS / SLOTS; q < (k + 1) * ITEMS / SLOTS; ++q) {
        if (q < LOADS) request(q);
        else read_fragment(next, 0, q - LOADS);
        if (q == LOADS - 1) step_requested();
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    stage = next;
  }
  wait_for_loads_but<0>();   // (the requests past the last step)

  // accumulator register v of a lane: row 8 * (v / 4) + 4 * (lane / 32) + v % 4, column lane % 32
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
    const int column = wn + j * 32 + col;
    if (piece != nullptr) {
#pragma unroll
      for (int i = 0; i < NI; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v)
          piece[(wm + i * 32 + 8 * (v >> 2) + 4 * half + (v & 3)) * T::BN + column] = acc[i][j][v];
    } else {
      const typename Ops::Column out = ops.column(n0 + column);
#pragma unroll
      for (int i = 0; i < NI; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v)
          ops.store(out, m0 + wm + i * 32 + 8 * (v >> 2) + 4 * half + (v & 3), acc[i][j][v]);
    }
  }
}

// The tiles of shape S of the columns from n_base on, in column-major order, whole tiles first,
// then the tiles cut along K (see igemm_kernel).
template <typename Ops, typename S>
__global__ void __launch_bounds__(64 * S::WAVES, 1)
igemm_b16_kernel(Ops ops, int row_tiles, int n_base, TileSplit split, float* __restrict__ piece_buffer) {
  const int whole_blocks = tile_blocks(split.whole);
  int t, s_begin = 0, s_end = k_steps_b16(ops.K);
  float* piece = nullptr;
  if (static_cast<int>(blockIdx.x) < whole_blocks) {
    t = tile_of_block(split.whole);
    if (t < 0) return;
  } else {
    const int q = blockIdx.x - whole_blocks;
    t = split.whole + q / split.pieces;
    s_begin = (q % split.pieces) * split.steps_per_piece;
    s_end = min(s_end, s_begin + split.steps_per_piece);
    piece = piece_buffer + static_cast<size_t>(q) * S::ROWS * TileB16::BN;
  }
  igemm_tile_b16<Ops, S>(ops, (t % row_tiles) * S::ROWS, n_base + (t / row_tiles) * S::COLS, s_begin, s_end, piece);
}

// Results of the split tiles: sum of their pieces, in piece order.
template <typename Ops, typename S>
__global__ void __launch_bounds__(256)
reduce_pieces_b16_kernel(Ops ops, int row_tiles, int n_base, TileSplit split, const float* __restrict__ piece_buffer) {
  constexpr int TILE = S::ROWS * TileB16::BN;
  const int local = blockIdx.x / (TILE / 256), e = (blockIdx.x % (TILE / 256)) * 256 + threadIdx.x;
  const int t = split.whole + local, column = e % TileB16::BN;
  if (column >= S::COLS) return;
  const float* p = piece_buffer + static_cast<size_t>(local) * split.pieces * TILE + e;
  float sum = 0.0f;
  for (int i = 0; i < split.pieces; ++i) sum += p[static_cast<size_t>(i) * TILE];
  ops.store(ops.column(n_base + (t / row_tiles) * S::COLS + column), (t % row_tiles) * S::ROWS + e / TileB16::BN, sum);
}

}  // namespace conv
