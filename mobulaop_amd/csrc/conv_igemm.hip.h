// 2-D convolution as implicit GEMM on the fp32 matrix cores of gfx950.
//
// The reference (opzoo/Convolution/Convolution.py:17-57) unfolds every image
// into a [C*KH*KW, OH*OW] column buffer with im2col and multiplies it with the
// reshaped weights, one image at a time; the backward pass does the transposed
// product plus col2im for dx and a second im2col for dW.  Here the column
// buffer never exists: the three products
//   y [D, N*OH*OW]  = W [D, C*KH*KW]      x col(x) [C*KH*KW, N*OH*OW]
//   dx[C, N*H*W]    = W'[C, D*KH*KW]      x col'(dy)[D*KH*KW, N*H*W]
//   dW[D, C*KH*KW]  = dy[D, N*OH*OW]      x col(x)'[N*OH*OW, C*KH*KW]
// are tiled GEMMs whose operand elements are fetched from the tensors where
// they lie (an operand functor maps a (row, k) or (k, column) index to an
// address or to zero in the padding) and staged through LDS.
//
// Tiling: a workgroup of four wavefronts owns a 128x128 tile of the result and
// walks K in steps of 16; each wavefront holds a 64x64 quarter as 2x2
// accumulators of v_mfma_f32_32x32x2_f32 (64 registers per lane), or, with
// operands rounded to bf16, of v_mfma_f32_32x32x16_bf16.  The next K step is
// fetched into registers while the current one is multiplied out of LDS (two
// LDS buffers, one barrier per step).
#pragma once
#include <hip/hip_runtime.h>

namespace conv {

typedef float float16v __attribute__((ext_vector_type(16)));

struct Geometry {
  int N, C, H, W;        // input
  int D, KH, KW;         // filters
  int OH, OW;            // output
  int pad_h, pad_w, stride_h, stride_w, dil_h, dil_w;
};

struct Tile {
  static constexpr int BM = 128, BN = 128, BK = 16;
  static constexpr int PITCH = BM + 32;   // consecutive k rows of a tile land 32 banks apart
  static constexpr int NT = 256;
};

// Offsets that a raw buffer load answers with zero: beyond every record count used here.
constexpr int kDead = static_cast<int>(0x80000000u);
constexpr unsigned kRecordLimit = 0x7fffffffu;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t buffer_of(const float* base, unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(base), 0, static_cast<int>(bytes), 0x00020000);
}
__device__ __forceinline__ float buffer_load1(__amdgpu_buffer_rsrc_t r, int voffset, int soffset) {
  return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, voffset, soffset, 0));
}

// ---- the two gathered products (forward, data gradient) ----------------------
// K runs tap-major: k = tap * Cpad + c with Cpad = channels rounded up to 16,
// so that a K step of 16 lies within one filter tap: the position of the tap
// and whether it falls into the padding is worked out once per step and lane,
// and the 16 channels are 16 loads from one address with scalar plane offsets.
// The left operand is a copy of the weights in that order, [Mpad][taps][Cpad],
// zero where a row or channel is padding (arrange_weights_kernel), so that its
// loads need no guards; the gathered operand re-reads the last real channel
// for padding channels (times zero).

// One K step of a gathered product.
struct GatherStep {
  int dh, dw;     // dilated tap position
  int delta;      // byte offset of the tap relative to the lane's anchor pixel
  int c0;         // first channel of the step
};

// steps[s] for s = tap * (Cpad / 16) + c0 / 16; sign = +1: taps walk forward over
// the source (forward pass), -1: backward (data gradient, source = dy).
__global__ void __launch_bounds__(256)
build_gather_steps_kernel(GatherStep* __restrict__ steps, int count, int per_tap, int KW, int dil_h,
                          int dil_w, int row, int sign) {
  const int s = blockIdx.x * blockDim.x + threadIdx.x;
  if (s >= count) return;
  const int tap = s / per_tap, kh = tap / KW, kw = tap - kh * KW;
  steps[s] = GatherStep{kh * dil_h, kw * dil_w, sign * (kh * dil_h * row + kw * dil_w) * 4,
                        (s - tap * per_tap) * 16};
}

// out[m][tap][c] = w[m * stride_m + c * stride_c + tap] for m < M and c < C, else 0
// (m < Mpad, c < Cpad).
__global__ void __launch_bounds__(256)
arrange_weights_kernel(const float* __restrict__ w, float* __restrict__ out, int M, int Mpad, int C,
                       int Cpad, int taps, long long stride_m, long long stride_c) {
  const long long total = static_cast<long long>(Mpad) * taps * Cpad;
  const long long i = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const int c = static_cast<int>(i % Cpad), tap = static_cast<int>((i / Cpad) % taps);
  const int m = static_cast<int>(i / (static_cast<long long>(Cpad) * taps));
  out[i] = (m < M && c < C) ? w[m * stride_m + c * stride_c + tap] : 0.0f;
}

// ---- operand functors -------------------------------------------------------
// Step load_step(s): what is the same for all lanes in K step s (scalar);
// fetch_a(m, step, s, ak, out): A[m][16 s + ak .. + 7]; BCtx b_ctx(n, n0): what
// column n needs throughout (n0 = first column of the tile);
// fetch_b(ctx, step, bk, out): B[16 s + bk .. + 7][n], bk the same for a
// wavefront; store(m, n, v).  Elements outside the operands are zero.

struct ForwardOps {
  const float* __restrict__ x; const float* __restrict__ wp; const float* __restrict__ bias;
  float* __restrict__ y; const GatherStep* __restrict__ steps;
  Geometry g; int M, Ncols, K;   // K = taps * Cpad
  typedef GatherStep Step;
  struct BCtx { __amdgpu_buffer_rsrc_t src; int anchor; int ih0, iw0; bool ok; };
  __device__ Step load_step(int s) const { return steps[s]; }
  __device__ Step next_step(const Step&, int s) const { return steps[s]; }
  __device__ void fetch_a(int m, const Step&, int s, int ak, float (&out)[8]) const {
    const float4* p = reinterpret_cast<const float4*>(wp + static_cast<size_t>(m) * K + s * Tile::BK + ak);
    const float4 lo = p[0], hi = p[1];
    out[0] = lo.x; out[1] = lo.y; out[2] = lo.z; out[3] = lo.w;
    out[4] = hi.x; out[5] = hi.y; out[6] = hi.z; out[7] = hi.w;
  }
  __device__ BCtx b_ctx(int n, int n0) const {
    BCtx c;
    c.ok = n < Ncols;
    const int ohw = g.OH * g.OW, image = g.C * g.H * g.W;
    const int first = __builtin_amdgcn_readfirstlane(n0 / ohw);
    const int img = n / ohw, r = n - img * ohw, oh = r / g.OW, ow = r - oh * g.OW;
    const size_t skip = static_cast<size_t>(first) * image;
    const size_t left = (static_cast<size_t>(g.N) * image - skip) * sizeof(float);
    c.src = buffer_of(x + skip, static_cast<unsigned>(left < kRecordLimit ? left : kRecordLimit));
    c.ih0 = oh * g.stride_h - g.pad_h;
    c.iw0 = ow * g.stride_w - g.pad_w;
    c.anchor = ((img - first) * image + c.ih0 * g.W + c.iw0) * 4;
    return c;
  }
  __device__ void fetch_b(const BCtx& c, const Step& e, int bk, float (&out)[8]) const {
    const int ih = c.ih0 + e.dh, iw = c.iw0 + e.dw;
    const bool in = c.ok && static_cast<unsigned>(ih) < static_cast<unsigned>(g.H) &&
                    static_cast<unsigned>(iw) < static_cast<unsigned>(g.W);
    const int at = in ? c.anchor + e.delta : kDead;
    const int plane = g.H * g.W * 4;
#pragma unroll
    for (int j = 0; j < 8; ++j)
      out[j] = buffer_load1(c.src, at, min(e.c0 + bk + j, g.C - 1) * plane);
  }
  __device__ void store(int m, int n, float v) const {
    if (m >= M || n >= Ncols) return;
    const int ohw = g.OH * g.OW, img = n / ohw, r = n - img * ohw;
    y[(static_cast<size_t>(img) * g.D + m) * ohw + r] = bias != nullptr ? v + bias[m] : v;
  }
};

// dx[img, c, ih, iw] = sum over (d, kh, kw) of W[d, c, kh, kw] * dy[img, d, oh, ow]
// with oh * stride = ih + pad - kh * dil (and likewise for columns).
struct BackwardDataOps {
  const float* __restrict__ dy; const float* __restrict__ wp; float* __restrict__ dx;
  const GatherStep* __restrict__ steps;
  Geometry g; int M, Ncols, K; int accumulate;
  typedef GatherStep Step;
  struct BCtx { __amdgpu_buffer_rsrc_t src; int anchor; int ihp, iwp; bool ok; };
  __device__ Step load_step(int s) const { return steps[s]; }
  __device__ Step next_step(const Step&, int s) const { return steps[s]; }
  __device__ void fetch_a(int m, const Step&, int s, int ak, float (&out)[8]) const {
    const float4* p = reinterpret_cast<const float4*>(wp + static_cast<size_t>(m) * K + s * Tile::BK + ak);
    const float4 lo = p[0], hi = p[1];
    out[0] = lo.x; out[1] = lo.y; out[2] = lo.z; out[3] = lo.w;
    out[4] = hi.x; out[5] = hi.y; out[6] = hi.z; out[7] = hi.w;
  }
  __device__ BCtx b_ctx(int n, int n0) const {
    BCtx c;
    c.ok = n < Ncols;
    const int hw = g.H * g.W, image = g.D * g.OH * g.OW;
    const int first = __builtin_amdgcn_readfirstlane(n0 / hw);
    const int img = n / hw, r = n - img * hw, ih = r / g.W, iw = r - ih * g.W;
    const size_t skip = static_cast<size_t>(first) * image;
    const size_t left = (static_cast<size_t>(g.N) * image - skip) * sizeof(float);
    c.src = buffer_of(dy + skip, static_cast<unsigned>(left < kRecordLimit ? left : kRecordLimit));
    c.ihp = ih + g.pad_h; c.iwp = iw + g.pad_w;
    // stride 1: byte offset of dy[img, 0, ihp, iwp]; otherwise of dy[img, 0, 0, 0]
    const bool unit = g.stride_h == 1 && g.stride_w == 1;
    c.anchor = ((img - first) * image + (unit ? c.ihp * g.OW + c.iwp : 0)) * 4;
    return c;
  }
  __device__ void fetch_b(const BCtx& c, const Step& e, int bk, float (&out)[8]) const {
    const int th = c.ihp - e.dh, tw = c.iwp - e.dw;
    int at;
    if (g.stride_h == 1 && g.stride_w == 1) {
      const bool in = c.ok && static_cast<unsigned>(th) < static_cast<unsigned>(g.OH) &&
                      static_cast<unsigned>(tw) < static_cast<unsigned>(g.OW);
      at = in ? c.anchor + e.delta : kDead;
    } else {
      const int oh = th / g.stride_h, ow = tw / g.stride_w;
      const bool in = c.ok && th >= 0 && tw >= 0 && oh * g.stride_h == th && ow * g.stride_w == tw &&
                      oh < g.OH && ow < g.OW;
      at = in ? c.anchor + (oh * g.OW + ow) * 4 : kDead;
    }
    const int plane = g.OH * g.OW * 4;
#pragma unroll
    for (int j = 0; j < 8; ++j)
      out[j] = buffer_load1(c.src, at, min(e.c0 + bk + j, g.D - 1) * plane);
  }
  __device__ void store(int m, int n, float v) const {
    if (m >= M || n >= Ncols) return;
    const int hw = g.H * g.W, img = n / hw, r = n - img * hw;
    float* p = dx + (static_cast<size_t>(img) * g.C + m) * hw + r;
    *p = accumulate ? *p + v : v;
  }
};

// Table entry for one column of the weight gradient, n = (c, kh, kw): element
// offset of the channel plane in x and the dilated tap position.
struct Tap { int off; short dh, dw; };

__global__ void __launch_bounds__(256)
build_taps_kernel(Tap* __restrict__ taps, int count, int KH, int KW, int plane, int dil_h, int dil_w) {
  const int k = blockIdx.x * blockDim.x + threadIdx.x;
  if (k >= count) return;
  const int kw = k % KW, kh = (k / KW) % KH, ch = k / (KW * KH);
  taps[k] = Tap{ch * plane, static_cast<short>(kh * dil_h), static_cast<short>(kw * dil_w)};
}

// xp[plane][pad_h + ih][pad_w + iw] = x[plane][ih][iw], zeros around: planes of (H + 2 pad_h) x
// (W + 2 pad_w), in which every tap of every output pixel is an element (no range tests).
__global__ void __launch_bounds__(256)
pad_planes_kernel(const float* __restrict__ x, float* __restrict__ xp, int H, int W, int pad_h, int pad_w,
                  int Hp, int Wp) {
  const float* in = x + static_cast<size_t>(blockIdx.x) * H * W;
  float* out = xp + static_cast<size_t>(blockIdx.x) * Hp * Wp;
  const int step_h = 256 / Wp, step_w = 256 - step_h * Wp;   // 256 elements further on
  int i = blockIdx.y * 2048 + threadIdx.x, ph = i / Wp, pw = i - ph * Wp;
  const int end = min((blockIdx.y + 1) * 2048, Hp * Wp);
  for (; i < end; i += 256) {
    const int ih = ph - pad_h, iw = pw - pad_w;
    const bool inside = static_cast<unsigned>(ih) < static_cast<unsigned>(H) &&
                        static_cast<unsigned>(iw) < static_cast<unsigned>(W);
    out[i] = inside ? __builtin_nontemporal_load(in + ih * W + iw) : 0.0f;
    ph += step_h; pw += step_w;
    if (pw >= Wp) { pw -= Wp; ++ph; }
  }
}

// partial[z][d, (c, kh, kw)] = sum over the k of slice z of dy[img, d, oh, ow] *
// x[img, c, ih, iw], k = (img, oh, ow) flattened; a slice is a range of k.
struct BackwardWeightOps {
  const float* __restrict__ dy; const float* __restrict__ x; float* __restrict__ partial;
  const Tap* __restrict__ taps;   // taps over x (over the planes of xp if that is set)
  // zero-padded copy of x (pad_planes_kernel) of Hp x Wp per plane, or null: the taps of eight
  // neighbouring output pixels are then two 16-byte loads, no range tests
  const float* __restrict__ xp; int Hp, Wp;
  Geometry g; int M, Ncols, K;   // K = length of this slice
  int k_begin;                   // first k of this slice
  // image, pixel (flat and as row / column) of the step's first k; k left in the slice
  struct Step { int img, r, left, oh, ow; };
  struct BCtx { int off; int dh, dw; bool ok; };
  __device__ Step load_step(int s) const {
    const int ohw = g.OH * g.OW, k = k_begin + s * Tile::BK, img = k / ohw, r = k - img * ohw, oh = r / g.OW;
    return Step{img, r, K - s * Tile::BK, oh, r - oh * g.OW};
  }
  // the step after e: sixteen pixels on, without the divisions
  __device__ Step next_step(const Step& e, int) const {
    Step n{e.img, e.r + Tile::BK, e.left - Tile::BK, e.oh, e.ow + Tile::BK};
    while (n.ow >= g.OW) { n.ow -= g.OW; ++n.oh; }
    while (n.oh >= g.OH) { n.oh -= g.OH; ++n.img; n.r -= g.OH * g.OW; }
    return n;
  }
  __device__ void fetch_a(int m, const Step& e, int, int ak, float (&out)[8]) const {
    const int ohw = g.OH * g.OW;
    int img = e.img, r = e.r + ak;
    while (r >= ohw) { r -= ohw; ++img; }   // (an output map of fewer than eight pixels: several images on)
    const size_t at = (static_cast<size_t>(img) * g.D + m) * ohw + r;
    if (m < M && ak + 8 <= e.left && r + 8 <= ohw && (at & 3) == 0) {
      const float4 lo = *reinterpret_cast<const float4*>(dy + at), hi = *reinterpret_cast<const float4*>(dy + at + 4);
      out[0] = lo.x; out[1] = lo.y; out[2] = lo.z; out[3] = lo.w;
      out[4] = hi.x; out[5] = hi.y; out[6] = hi.z; out[7] = hi.w;
      return;
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      out[j] = (m < M && ak + j < e.left) ? dy[(static_cast<size_t>(img) * g.D + m) * ohw + r] : 0.0f;
      if (++r == ohw) { r = 0; ++img; }
    }
  }
  __device__ BCtx b_ctx(int n, int) const {
    BCtx c;
    c.ok = n < Ncols;
    const Tap t = taps[c.ok ? n : 0];
    c.off = t.off; c.dh = t.dh; c.dw = t.dw;
    return c;
  }
  __device__ void fetch_b(const BCtx& c, const Step& e, int bk, float (&out)[8]) const {
    const int ohw = g.OH * g.OW, image = g.C * g.H * g.W;
    int img = e.img, r = e.r + bk, oh0 = e.oh, ow0 = e.ow + bk;   // scalar: the step and bk are uniform
    while (ow0 >= g.OW) { ow0 -= g.OW; ++oh0; }
    while (r >= ohw) { r -= ohw; oh0 -= g.OH; ++img; }
    if (xp != nullptr) {
      const int image_p = g.C * Hp * Wp;
      if (g.stride_w == 1 && ow0 + 8 <= g.OW && bk + 8 <= e.left) {
        // eight pixels of one output row: eight neighbouring elements of the padded plane
        typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
        const __amdgpu_buffer_rsrc_t src = buffer_of(xp + static_cast<size_t>(img) * image_p, image_p * 4u);
        const int at = c.ok ? (c.off + (oh0 * g.stride_h + c.dh) * Wp + ow0 + c.dw) * 4 : kDead;
        const u32x4 lo = __builtin_amdgcn_raw_buffer_load_b128(src, at, 0, 0);
        const u32x4 hi = __builtin_amdgcn_raw_buffer_load_b128(src, at, 16, 0);
#pragma unroll
        for (int j = 0; j < 4; ++j) { out[j] = __uint_as_float(lo[j]); out[4 + j] = __uint_as_float(hi[j]); }
        return;
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int oh = r / g.OW, ow = r - oh * g.OW;
        const bool in = c.ok && bk + j < e.left;
        out[j] = in ? xp[static_cast<size_t>(img) * image_p + c.off + (oh * g.stride_h + c.dh) * Wp +
                         ow * g.stride_w + c.dw] : 0.0f;
        if (++r == ohw) { r = 0; ++img; }
      }
      return;
    }
    if (g.stride_w == 1 && ow0 + 8 <= g.OW && bk + 8 <= e.left) {
      // eight pixels of one output row: one row check, loads from one address
      const __amdgpu_buffer_rsrc_t src = buffer_of(x + static_cast<size_t>(img) * image, image * 4u);
      const int ih = oh0 * g.stride_h - g.pad_h + c.dh, iw0 = ow0 - g.pad_w + c.dw;
      const bool row = c.ok && static_cast<unsigned>(ih) < static_cast<unsigned>(g.H);
      const int at = (c.off + ih * g.W + iw0) * 4;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const bool in = row && static_cast<unsigned>(iw0 + j) < static_cast<unsigned>(g.W);
        out[j] = buffer_load1(src, in ? at + 4 * j : kDead, 0);
      }
      return;
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int oh = r / g.OW, ow = r - oh * g.OW;
      const int ih = oh * g.stride_h - g.pad_h + c.dh, iw = ow * g.stride_w - g.pad_w + c.dw;
      const bool in = c.ok && bk + j < e.left && static_cast<unsigned>(ih) < static_cast<unsigned>(g.H) &&
                      static_cast<unsigned>(iw) < static_cast<unsigned>(g.W);
      out[j] = in ? x[static_cast<size_t>(img) * image + c.off + ih * g.W + iw] : 0.0f;
      if (++r == ohw) { r = 0; ++img; }
    }
  }
  __device__ void store(int m, int n, float v) const {
    if (m >= M || n >= Ncols) return;
    partial[static_cast<size_t>(m) * Ncols + n] = v;
  }
};

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

// two fp32 -> two bf16 in one word, round to nearest even (v_cvt_pk_bf16_f32)
__device__ __forceinline__ unsigned pack_bf16(float lo, float hi) {
  const f32x2 v = {lo, hi};
  return __builtin_bit_cast(unsigned, __builtin_convertvector(v, bf16x2));
}

// How the products are formed.
//   kFp32:   fp32 operands, v_mfma_f32_32x32x2_f32.
//   kBf16:   operands rounded to bf16 on their way into LDS, v_mfma_f32_32x32x16_bf16
//            with fp32 accumulation (relative error of a result about 2e-3).
//   kBf16x3: every operand split into a bf16 head and a bf16 tail (a = ah + al
//            to 16 significant bits); ah*bh + ah*bl + al*bh on the bf16 matrix
//            cores, fp32 accumulation: fp32-like results (about 1e-5) at three
//            bf16 products, which is still a sixth of the fp32 matrix-core time.
enum Compute { kFp32 = 0, kBf16 = 1, kBf16x3 = 2 };

// Workgroup id -> tile, for a launch of tile_blocks(count) workgroups.
// Consecutive workgroup ids go round the eight XCDs, each with an L2 of its
// own; tile t is handed to XCD t / ceil(count / 8), so that an XCD walks a
// contiguous range of tiles and the operand rows these share stay in its L2.
// Returns -1 for the padding workgroups.
__host__ __device__ inline int tile_blocks(int count) { return (count + 7) / 8 * 8; }
__device__ __forceinline__ int tile_of_block(int count) {
  const int per = (count + 7) / 8, t = (blockIdx.x & 7) * per + (blockIdx.x >> 3);
  return (blockIdx.x >> 3) < per && t < count ? t : -1;
}

// Where a tile's results go: through the operand functor, or (piece != nullptr:
// the tile covers part of K only) into a dense 128x128 piece buffer.
template <typename Ops>
struct StoreResult {
  const Ops& ops;
  float* piece;
  __device__ void operator()(int m, int n, int lm, int ln, float v) const {
    if (piece != nullptr) piece[lm * Tile::BN + ln] = v;
    else ops.store(m, n, v);
  }
};

// C[M, Ncols] = A[M, K] x B[K, Ncols], one 128x128 tile per workgroup, over the K
// steps s_begin .. s_end - 1; results go to store(m, n, row in tile, column in tile, value).
template <typename Ops, int MODE, typename Store>
__device__ __forceinline__ void igemm_tile(const Ops& ops, int m0, int n0, int s_begin, int s_end,
                                           const Store& store) {
  using T = Tile;
  constexpr bool BF16 = MODE != kFp32;
  constexpr int PARTS = MODE == kBf16x3 ? 2 : 1;   // head, tail
  // fp32: [k][row] so that the 32 lanes of a half read consecutive words;
  // bf16: [part][row][k] (pitch 24 halves = 48 bytes) so that a lane reads its eight k as 16 bytes
  constexpr int PK = 24;
  constexpr int PART_WORDS = T::BM * PK / 2;
  constexpr int LDS_WORDS = BF16 ? PARTS * PART_WORDS : T::BK * T::PITCH;
  __shared__ __attribute__((aligned(16))) float As[2][LDS_WORDS];
  __shared__ __attribute__((aligned(16))) float Bs[2][LDS_WORDS];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64;

  // staging roles: A: row a_m, eight consecutive k starting at a_k; B: column
  // b_n, eight consecutive k starting at b_k (the same for a wavefront)
  const int a_m = tid >> 1, a_k = (tid & 1) * 8;
  const int b_n = tid & 127, b_k = __builtin_amdgcn_readfirstlane(tid >> 7) * 8;
  const typename Ops::BCtx bctx = ops.b_ctx(n0 + b_n, n0);

  float16v acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  float ra[8], rb[8];
  typename Ops::Step step = ops.load_step(s_begin);
  auto fetch = [&](int s) {
    ops.fetch_a(m0 + a_m, step, s, a_k, ra);
    ops.fetch_b(bctx, step, b_k, rb);
  };
  auto stage = [&](int buf) {
    if (BF16) {
      typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
#pragma unroll
      for (int part = 0; part < PARTS; ++part) {
        u32x4 pa, pb;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          pa[j] = pack_bf16(ra[2 * j], ra[2 * j + 1]);
          pb[j] = pack_bf16(rb[2 * j], rb[2 * j + 1]);
        }
        *reinterpret_cast<u32x4*>(reinterpret_cast<unsigned short*>(As[buf] + part * PART_WORDS) + a_m * PK + a_k) = pa;
        *reinterpret_cast<u32x4*>(reinterpret_cast<unsigned short*>(Bs[buf] + part * PART_WORDS) + b_n * PK + b_k) = pb;
        if (part + 1 < PARTS) {
          // what the heads left over (exact in fp32)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            ra[2 * j] -= __uint_as_float(pa[j] << 16); ra[2 * j + 1] -= __uint_as_float(pa[j] & 0xffff0000u);
            rb[2 * j] -= __uint_as_float(pb[j] << 16); rb[2 * j + 1] -= __uint_as_float(pb[j] & 0xffff0000u);
          }
        }
      }
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) As[buf][(a_k + j) * T::PITCH + a_m] = ra[j];
#pragma unroll
      for (int j = 0; j < 8; ++j) Bs[buf][(b_k + j) * T::PITCH + b_n] = rb[j];
    }
  };

  const int steps = s_end;
  const int half = lane >> 5, col = lane & 31;
  fetch(s_begin);
  stage(0);
  __syncthreads();
  for (int s = s_begin; s < steps; ++s) {
    const int buf = (s - s_begin) & 1;
    if (s + 1 < steps) {
      step = ops.next_step(step, s + 1);
      fetch(s + 1);
    }
    if (BF16) {
      bf16x8 a[PARTS][2], b[PARTS][2];
#pragma unroll
      for (int part = 0; part < PARTS; ++part) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
          a[part][i] = *reinterpret_cast<const bf16x8*>(
              reinterpret_cast<const unsigned short*>(As[buf] + part * PART_WORDS) + (wm + i * 32 + col) * PK + half * 8);
#pragma unroll
        for (int j = 0; j < 2; ++j)
          b[part][j] = *reinterpret_cast<const bf16x8*>(
              reinterpret_cast<const unsigned short*>(Bs[buf] + part * PART_WORDS) + (wn + j * 32 + col) * PK + half * 8);
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          if (PARTS == 2) {   // small terms first
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[1][i], b[0][j], acc[i][j], 0, 0, 0);
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[0][i], b[1][j], acc[i][j], 0, 0, 0);
          }
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[0][i], b[0][j], acc[i][j], 0, 0, 0);
        }
    } else {
#pragma unroll
      for (int kk = 0; kk < T::BK; kk += 2) {
        float a[2], b[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) a[i] = As[buf][(kk + half) * T::PITCH + wm + i * 32 + col];
#pragma unroll
        for (int j = 0; j < 2; ++j) b[j] = Bs[buf][(kk + half) * T::PITCH + wn + j * 32 + col];
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int j = 0; j < 2; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], acc[i][j], 0, 0, 0);
      }
    }
    if (s + 1 < steps) stage(buf ^ 1);
    __syncthreads();
  }

  // accumulator register v of a lane: row 8 * (v / 4) + 4 * (lane / 32) + v % 4, column lane % 32
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int row = wm + i * 32 + 8 * (v >> 2) + 4 * half + (v & 3), column = wn + j * 32 + col;
        store(m0 + row, n0 + column, row, column, acc[i][j][v]);
      }
}

__host__ __device__ inline int k_steps(int K) { return (K + Tile::BK - 1) / Tile::BK; }

// How a launch covers `count` tiles: the first `whole` tiles by one workgroup
// each; each of the others by `pieces` workgroups that take `steps_per_piece`
// K steps apiece and leave their sums in a piece buffer (added up, in order,
// by reduce_pieces_kernel).  The split evens out the last round of a launch
// whose tile count is a little more than a multiple of what the device holds
// at a time, and fills the device when there are few tiles.
struct TileSplit {
  int whole, pieces, steps_per_piece;
};

// Tiles in column-major order: the row tiles of one column tile are neighbours
// and read the same gathered operand.
template <typename Ops, int MODE>
__global__ void __launch_bounds__(Tile::NT)
igemm_kernel(Ops ops, int row_tiles, TileSplit split, float* __restrict__ piece_buffer) {
  const int whole_blocks = tile_blocks(split.whole);
  int t, s_begin = 0, s_end = k_steps(ops.K);
  float* piece = nullptr;
  if (static_cast<int>(blockIdx.x) < whole_blocks) {
    t = tile_of_block(split.whole);
    if (t < 0) return;
  } else {
    const int q = blockIdx.x - whole_blocks;
    t = split.whole + q / split.pieces;
    s_begin = (q % split.pieces) * split.steps_per_piece;
    s_end = min(s_end, s_begin + split.steps_per_piece);
    piece = piece_buffer + static_cast<size_t>(q) * Tile::BM * Tile::BN;
  }
  igemm_tile<Ops, MODE>(ops, (t % row_tiles) * Tile::BM, (t / row_tiles) * Tile::BN, s_begin, s_end,
                        StoreResult<Ops>{ops, piece});
}

// Results of the split tiles: sum of their pieces, in piece order.
template <typename Ops>
__global__ void __launch_bounds__(256)
reduce_pieces_kernel(Ops ops, int row_tiles, TileSplit split, const float* __restrict__ piece_buffer) {
  constexpr int TILE = Tile::BM * Tile::BN;
  const int local = blockIdx.x / (TILE / 256), e = (blockIdx.x % (TILE / 256)) * 256 + threadIdx.x;
  const int t = split.whole + local;
  const float* p = piece_buffer + static_cast<size_t>(local) * split.pieces * TILE + e;
  float sum = 0.0f;
  for (int i = 0; i < split.pieces; ++i) sum += p[static_cast<size_t>(i) * TILE];
  ops.store((t % row_tiles) * Tile::BM + e / Tile::BN, (t / row_tiles) * Tile::BN + e % Tile::BN, sum);
}

// Slices of K times tiles, slice-major; every slice writes its own partial.
template <int MODE>
__global__ void __launch_bounds__(Tile::NT)
igemm_weight_kernel(BackwardWeightOps ops, int k_per_slice, int k_total, int row_tiles,
                    int tiles_per_slice, int count) {
  const int t = tile_of_block(count);
  if (t < 0) return;
  const int slice = t / tiles_per_slice, tile = t - slice * tiles_per_slice;
  ops.k_begin = slice * k_per_slice;
  ops.K = min(k_per_slice, k_total - ops.k_begin);
  ops.partial += static_cast<size_t>(slice) * ops.M * ops.Ncols;
  igemm_tile<BackwardWeightOps, MODE>(ops, (tile % row_tiles) * Tile::BM, (tile / row_tiles) * Tile::BN, 0,
                                      k_steps(ops.K), StoreResult<BackwardWeightOps>{ops, nullptr});
}

// out[i] (+)= sum over slices of partial[s][i]
__global__ void __launch_bounds__(256)
reduce_slices_kernel(const float* __restrict__ partial, float* __restrict__ out, long long count,
                     int slices, int accumulate) {
  const long long i = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= count) return;
  float s = 0.0f;
  for (int z = 0; z < slices; ++z) s += partial[static_cast<long long>(z) * count + i];
  out[i] = accumulate ? out[i] + s : s;
}

// db[d] (+)= sum over images and pixels of dy[img, d, :, :]; one workgroup per filter.
__global__ void __launch_bounds__(256)
bias_grad_kernel(const float* __restrict__ dy, float* __restrict__ db, int N, int D, int ohw, int accumulate) {
  __shared__ float part[256];
  const int d = blockIdx.x;
  float s = 0.0f;
  for (int img = 0; img < N; ++img) {
    const float* p = dy + (static_cast<size_t>(img) * D + d) * ohw;
    for (int i = threadIdx.x; i < ohw; i += 256) s += p[i];
  }
  part[threadIdx.x] = s;
  __syncthreads();
  for (int off = 128; off > 0; off >>= 1) {
    if (threadIdx.x < off) part[threadIdx.x] += part[threadIdx.x + off];
    __syncthreads();
  }
  if (threadIdx.x == 0) db[d] = accumulate ? db[d] + part[0] : part[0];
}

// The reference's unfold and fold (opzoo/Convolution/Convolution.cpp:13-90), one
// image per launch: kept for callers that use mobula.func.im2col / col2im directly.
__global__ void __launch_bounds__(256)
im2col_kernel(long long n, const float* __restrict__ im, int H, int W, int KH, int KW, int pad_h,
              int pad_w, int stride_h, int stride_w, int dil_h, int dil_w, int OH, int OW,
              float* __restrict__ col) {
  const long long stride = static_cast<long long>(gridDim.x) * blockDim.x;
  for (long long idx = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x; idx < n; idx += stride) {
    long long t = idx;
    const int ow = t % OW; t /= OW;
    const int oh = t % OH; t /= OH;
    const int kw = t % KW; t /= KW;
    const int kh = t % KH; t /= KH;
    const int c = static_cast<int>(t);
    const int ih = -pad_h + kh * dil_h + stride_h * oh, iw = -pad_w + kw * dil_w + stride_w * ow;
    const bool in = static_cast<unsigned>(ih) < static_cast<unsigned>(H) &&
                    static_cast<unsigned>(iw) < static_cast<unsigned>(W);
    col[idx] = in ? im[(static_cast<long long>(c) * H + ih) * W + iw] : 0.0f;
  }
}

__global__ void __launch_bounds__(256)
col2im_kernel(long long n, const float* __restrict__ col, int H, int W, int KH, int KW, int pad_h,
              int pad_w, int stride_h, int stride_w, int dil_h, int dil_w, int OH, int OW,
              float* __restrict__ im) {
  const long long stride = static_cast<long long>(gridDim.x) * blockDim.x;
  const int ext_w = (KW - 1) * dil_w + 1, ext_h = (KH - 1) * dil_h + 1;
  for (long long idx = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x; idx < n; idx += stride) {
    const int w_im = idx % W + pad_w, h_im = (idx / W) % H + pad_h;
    const int c = static_cast<int>(idx / (static_cast<long long>(W) * H));
    const int w0 = w_im < ext_w ? 0 : (w_im - ext_w) / stride_w + 1, w1 = min(w_im / stride_w + 1, OW);
    const int h0 = h_im < ext_h ? 0 : (h_im - ext_h) / stride_h + 1, h1 = min(h_im / stride_h + 1, OH);
    float v = 0.0f;
    for (int oh = h0; oh < h1; ++oh)
      for (int ow = w0; ow < w1; ++ow) {
        int hk = h_im - oh * stride_h, wk = w_im - ow * stride_w;
        if (hk % dil_h == 0 && wk % dil_w == 0) {
          hk /= dil_h; wk /= dil_w;
          v += col[((static_cast<long long>(c) * KH + hk) * KW + wk) * OH * OW + static_cast<long long>(oh) * OW + ow];
        }
      }
    im[idx] = v;
  }
}

}  // namespace conv
