// Convolution launchers for gfx950 and their C-ABI entry points.
//
// im2col / col2im have the argument lists of the reference kernels
// (opzoo/Convolution/Convolution.cpp:13-90) and are what
// `mobula.func.im2col / col2im` bind to.  The conv2d_* launchers have no
// counterpart in the reference: they are the whole products the reference's
// operator assembles from im2col/col2im and the framework's matrix product
// (opzoo/Convolution/Convolution.py:17-57), computed on the matrix cores
// without a column buffer.
#include <algorithm>

#include "runtime.h"
#include "conv_igemm.hip.h"
#include "conv_igemm_bf16.hip.h"

namespace {

using mobula_hip::arg_extent;
using mobula_hip::call_state;
using mobula_hip::failed;
using mobula_hip::set_error;

// option "conv_compute": 0 = fp32 operands (default), 1 = operands rounded to
// bf16, 2 = operands split into two bf16 each (three products); fp32 accumulation throughout
int compute_mode() {
  const int mode = mobula_hip::option("conv_compute", 0);
  return mode == conv::kBf16 || mode == conv::kBf16x3 ? mode : conv::kFp32;
}

// Workgroups of igemm_kernel<Ops, MODE> the device holds at a time.
template <typename Ops, int MODE>
int resident_workgroups() {
  static thread_local int cached_device = -1, cached = 0;
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) return 0;
  if (device != cached_device) {
    int per_cu = 0, cus = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, conv::igemm_kernel<Ops, MODE>, conv::Tile::NT, 0) !=
            hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess) {
      (void)hipGetLastError();
      return 0;
    }
    cached = per_cu * cus;
    cached_device = device;
  }
  return cached;
}

// Most piece workgroups a launch uses (sizes the piece buffer): no more than the
// device holds at a time, and no device is assumed to hold more than this.
constexpr int kMaxPieceBlocks = 2048;

conv::TileSplit split_tiles(int count, int steps, int resident) {
  conv::TileSplit split{count, 1, steps};
  resident = std::min(resident, kMaxPieceBlocks);
  if (resident <= 0 || steps < 2) return split;
  const int rest = count % resident;
  // a last round that fills less than half of the device is cut along K
  if (rest == 0 || rest > resident / 2) return split;
  int pieces = std::min(resident / rest, steps);
  if (pieces < 2) return split;
  split.steps_per_piece = (steps + pieces - 1) / pieces;
  split.pieces = (steps + split.steps_per_piece - 1) / split.steps_per_piece;
  split.whole = count - rest;
  return split;
}

template <typename Ops, int MODE>
void launch_igemm_mode(const Ops& ops, float* piece_buffer, hipStream_t stream) {
  const int row_tiles = (ops.M + conv::Tile::BM - 1) / conv::Tile::BM;
  const int count = row_tiles * ((ops.Ncols + conv::Tile::BN - 1) / conv::Tile::BN);
  const conv::TileSplit split = split_tiles(count, conv::k_steps(ops.K), resident_workgroups<Ops, MODE>());
  const int rest = count - split.whole;
  const dim3 grid(conv::tile_blocks(split.whole) + rest * split.pieces);
  conv::igemm_kernel<Ops, MODE><<<grid, conv::Tile::NT, 0, stream>>>(ops, row_tiles, split, piece_buffer);
  if (rest > 0)
    conv::reduce_pieces_kernel<Ops><<<rest * (conv::Tile::BM * conv::Tile::BN / 256), 256, 0, stream>>>(
        ops, row_tiles, split, piece_buffer);
}

template <typename Ops>
void launch_igemm(const Ops& ops, float* piece_buffer, hipStream_t stream) {
  switch (compute_mode()) {
    case conv::kBf16: launch_igemm_mode<Ops, conv::kBf16>(ops, piece_buffer, stream); break;
    case conv::kBf16x3: launch_igemm_mode<Ops, conv::kBf16x3>(ops, piece_buffer, stream); break;
    default: launch_igemm_mode<Ops, conv::kFp32>(ops, piece_buffer, stream);
  }
}

// Workgroups of igemm_b16_kernel<Ops, S> the device holds at a time.
template <typename Ops, typename S>
int resident_workgroups_b16() {
  static thread_local int cached_device = -1, cached = 0;
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) return 0;
  if (device != cached_device) {
    int per_cu = 0, cus = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, conv::igemm_b16_kernel<Ops, S>, 64 * S::WAVES, 0) !=
            hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess) {
      (void)hipGetLastError();
      return 0;
    }
    cached = per_cu * cus;
    cached_device = device;
  }
  return cached;
}

// The columns from n_base on (`columns` of them) of a bf16 product in tiles of shape S.  Pieces of
// these products are ROWS x 256 floats; the piece buffer holds kMaxPieceBlocks pieces of 128 x 128.
template <typename Ops, typename S>
void launch_igemm_b16_shape(const Ops& ops, int n_base, int columns, float* piece_buffer, hipStream_t stream) {
  const int row_tiles = (ops.M + S::ROWS - 1) / S::ROWS, count = row_tiles * ((columns + S::COLS - 1) / S::COLS);
  const int room = kMaxPieceBlocks * conv::Tile::BM * conv::Tile::BN / (S::ROWS * conv::TileB16::BN);
  const int resident = std::min(resident_workgroups_b16<Ops, S>(), room);
  const conv::TileSplit split = split_tiles(count, conv::k_steps_b16(ops.K), resident);
  const int rest = count - split.whole;
  const dim3 grid(conv::tile_blocks(split.whole) + rest * split.pieces);
  conv::igemm_b16_kernel<Ops, S><<<grid, 64 * S::WAVES, 0, stream>>>(ops, row_tiles, n_base, split, piece_buffer);
  if (rest > 0)
    conv::reduce_pieces_b16_kernel<Ops, S><<<rest * (S::ROWS * conv::TileB16::BN / 256), 256, 0, stream>>>(
        ops, row_tiles, n_base, split, piece_buffer);
}

// Tiles of 256 x 256, or 128 x 256 for products of at most 128 rows.  (Tried for a last round that
// fills between half and three quarters of the device: one round of narrower tiles, 256 x 160,
// over the same columns.  The two rounds then take as long as before -- the full round alone runs
// slower than beside a half-empty one -- so there is one shape per product.)
template <typename Ops>
void launch_igemm_b16(const Ops& ops, float* piece_buffer, hipStream_t stream) {
  if (ops.M <= 128) launch_igemm_b16_shape<Ops, conv::LowShapeB16>(ops, 0, ops.Ncols, piece_buffer, stream);
  else launch_igemm_b16_shape<Ops, conv::WideShapeB16>(ops, 0, ops.Ncols, piece_buffer, stream);
}

// workgroups the weight gradient aims at: four per CU of a 256-CU device
constexpr long long kWeightSlots = 1024;

int blocks_for(long long n) { return static_cast<int>(std::min<long long>((n + 255) / 256, 256ll * 32)); }
// (for kernels that take one element per thread and do not stride)
int blocks_for_all(long long n) { return static_cast<int>((n + 255) / 256); }

bool fits(const char* what, int arg, long long need) {
  const long long have = arg_extent(arg);
  if (have >= 0 && have < need) {
    set_error("%s: argument %d holds %lld elements, the shape needs %lld", what, arg, have, need);
    return false;
  }
  return true;
}

// Fills g from the scalar arguments; false (with the error text set) if they
// do not describe a convolution.
bool describe(conv::Geometry* g, const char* what, int N, int C, int H, int W, int D, int KH, int KW,
              int pad_h, int pad_w, int stride_h, int stride_w, int dil_h, int dil_w) {
  if (N < 0 || C <= 0 || H <= 0 || W <= 0 || D <= 0 || KH <= 0 || KW <= 0 || pad_h < 0 || pad_w < 0 ||
      stride_h <= 0 || stride_w <= 0 || dil_h <= 0 || dil_w <= 0) {
    set_error("%s: invalid shape N=%d C=%d H=%d W=%d D=%d K=%dx%d pad=%d,%d stride=%d,%d dilation=%d,%d",
              what, N, C, H, W, D, KH, KW, pad_h, pad_w, stride_h, stride_w, dil_h, dil_w);
    return false;
  }
  const int eh = (KH - 1) * dil_h + 1, ew = (KW - 1) * dil_w + 1;
  if (H + 2 * pad_h < eh || W + 2 * pad_w < ew) {
    set_error("%s: the %dx%d window does not fit the padded %dx%d input", what, eh, ew, H + 2 * pad_h,
              W + 2 * pad_w);
    return false;
  }
  g->N = N; g->C = C; g->H = H; g->W = W; g->D = D; g->KH = KH; g->KW = KW;
  g->pad_h = pad_h; g->pad_w = pad_w; g->stride_h = stride_h; g->stride_w = stride_w;
  g->dil_h = dil_h; g->dil_w = dil_w;
  g->OH = (H + 2 * pad_h - eh) / stride_h + 1;
  g->OW = (W + 2 * pad_w - ew) / stride_w + 1;
  const long long in = static_cast<long long>(N) * C * H * W, out = static_cast<long long>(N) * D * g->OH * g->OW;
  const long long wt = static_cast<long long>(D) * C * KH * KW;
  if (in >= (1ll << 31) || out >= (1ll << 31) || wt >= (1ll << 31) || KH * dil_h > 32767 || KW * dil_w > 32767) {
    set_error("%s: tensors beyond 32-bit indexing are not supported", what);
    return false;
  }
  return true;
}

conv::Tap* make_taps(int count, int KH, int KW, int plane, int dil_h, int dil_w, size_t extra_bytes,
                     char** extra, hipStream_t stream) {
  const size_t tap_bytes = (sizeof(conv::Tap) * count + 255) / 256 * 256;
  char* ws = static_cast<char*>(mobula_hip::workspace(tap_bytes + extra_bytes));
  if (failed()) return nullptr;
  conv::Tap* taps = reinterpret_cast<conv::Tap*>(ws);
  if (extra != nullptr) *extra = ws + tap_bytes;
  conv::build_taps_kernel<<<(count + 255) / 256, 256, 0, stream>>>(taps, count, KH, KW, plane, dil_h, dil_w);
  return taps;
}

// Workspace of a gathered product (forward, data gradient): the table of K
// steps and the weights in [Mpad][taps][Cpad] order.  channels = what K runs
// over besides the taps, plane_row = row length of the gathered tensor.
struct GatherPlan { conv::GatherStep* steps; float* weights; float* pieces; int K; };

bool plan_gather(GatherPlan* plan, const char* what, const conv::Geometry& g, const float* w, int M,
                 int channels, long long image_elems, int columns_per_image, int plane_row, int sign,
                 long long stride_m, long long stride_c, hipStream_t stream) {
  // a tile's columns span this many images at most; their byte offsets must stay below 2^31
  const long long span = (conv::Tile::BN - 1) / std::max(columns_per_image, 1) + 2;
  if (span * image_elems * 4 >= (1ll << 31)) {
    set_error("%s: images of %lld elements are too large for the 32-bit offsets of the gather", what, image_elems);
    return false;
  }
  const int taps = g.KH * g.KW, cpad = (channels + 15) / 16 * 16, per_tap = cpad / 16;
  const int mpad = (M + conv::Tile::BM - 1) / conv::Tile::BM * conv::Tile::BM;
  const long long k = static_cast<long long>(taps) * cpad, wcount = k * mpad;
  if (k >= (1ll << 31) || wcount >= (1ll << 31)) { set_error("%s: weights too large", what); return false; }
  const int count = taps * per_tap;
  const size_t step_bytes = (sizeof(conv::GatherStep) * count + 255) / 256 * 256;
  const size_t weight_bytes = (sizeof(float) * wcount + 255) / 256 * 256;
  const size_t piece_bytes = sizeof(float) * kMaxPieceBlocks * conv::Tile::BM * conv::Tile::BN;
  char* ws = static_cast<char*>(mobula_hip::workspace(step_bytes + weight_bytes + piece_bytes));
  if (failed()) return false;
  plan->steps = reinterpret_cast<conv::GatherStep*>(ws);
  plan->weights = reinterpret_cast<float*>(ws + step_bytes);
  plan->pieces = reinterpret_cast<float*>(ws + step_bytes + weight_bytes);
  plan->K = static_cast<int>(k);
  conv::build_gather_steps_kernel<<<(count + 255) / 256, 256, 0, stream>>>(plan->steps, count, per_tap, g.KW,
                                                                          g.dil_h, g.dil_w, plane_row, sign);
  conv::arrange_weights_kernel<<<blocks_for(wcount), 256, 0, stream>>>(w, plan->weights, M, mpad, channels, cpad,
                                                                       taps, stride_m, stride_c);
  return true;
}

// Workspace of a gathered product with bf16 operands in memory (conv_igemm_bf16.hip.h): the
// weights as [K step][Mpad][32] bf16, the gathered tensor `src` ([images][channels][src_pixels]
// fp32) as [images][channel block][src_pixels][32] bf16, the piece buffer.  Fills in the
// fields of `ops` that describe them.  split: two sets of each, heads then tails of the fp32
// values, and three passes over K.  *taken = false (and no error): the shape does not fit this
// path's 32-bit offsets with split operands; the caller has other kernels for that mode.
bool plan_gather_b16(conv::GatheredB16* ops, float** pieces, const char* what, const conv::Geometry& g,
                     const float* w, int M, int channels, const float* src, int images, int src_pixels,
                     int columns_per_image, long long stride_m, long long stride_c, bool split, bool* taken,
                     hipStream_t stream) {
  *taken = true;
  const int sets = split ? 2 : 1;
  const int taps = g.KH * g.KW, cpad = (channels + 31) / 32 * 32;
  const long long image_bytes = static_cast<long long>(src_pixels) * cpad * 2;
  // a tile's columns span this many images at most; their byte offsets must stay below 2^31
  const long long span = (conv::TileB16::BN - 1) / std::max(columns_per_image, 1) + 2;
  if (split && (span + images) * image_bytes >= (1ll << 31)) { *taken = false; return false; }
  if (span * image_bytes >= (1ll << 31)) {
    set_error("%s: images of %lld bytes are too large for the 32-bit offsets of the gather", what, image_bytes);
    return false;
  }
  const int mpad = (M + 255) / 256 * 256;   // (covers row tiles of 128 and of 256)
  const long long k = static_cast<long long>(taps) * cpad, wcount = k * mpad;
  const int weight_sets = split ? 3 : 1;   // (heads, heads again, tails: one per pass)
  if (3 * k >= (1ll << 31) || 2 * weight_sets * wcount >= (1ll << 31)) {
    if (split) { *taken = false; return false; }
    set_error("%s: weights too large", what);
    return false;
  }
  const size_t weight_bytes = (2 * weight_sets * wcount + 255) / 256 * 256;
  const size_t source_bytes = (static_cast<size_t>(sets) * images * image_bytes + 255) / 256 * 256;
  const size_t piece_bytes = sizeof(float) * kMaxPieceBlocks * conv::Tile::BM * conv::Tile::BN;
  char* ws = static_cast<char*>(mobula_hip::workspace(weight_bytes + source_bytes + piece_bytes));
  if (failed()) return false;
  unsigned short* const weights = reinterpret_cast<unsigned short*>(ws);
  unsigned short* const source = reinterpret_cast<unsigned short*>(ws + weight_bytes);
  *pieces = reinterpret_cast<float*>(ws + weight_bytes + source_bytes);
  ops->wp = weights; ops->src = source; ops->g = g; ops->M = M;
  ops->K = static_cast<int>((split ? 3 : 1) * k); ops->cpad = cpad; ops->mpad = mpad;
  ops->source_tail = split ? static_cast<int>(images * image_bytes) : 0;
  const size_t weight_tail = split ? static_cast<size_t>(wcount) : 0;                      // (in halves)
  const size_t source_tail = split ? static_cast<size_t>(images) * image_bytes / 2 : 0;
  conv::arrange_weights_bf16_kernel<<<blocks_for_all(wcount / 2), 256, 0, stream>>>(
      w, weights, M, mpad, channels, cpad, taps, stride_m, stride_c, weight_tail);
  const dim3 tgrid((src_pixels + 63) / 64, (cpad + 63) / 64, images);
  if (src_pixels % 4 == 0 && reinterpret_cast<uintptr_t>(src) % 16 == 0)
    conv::to_blocked_bf16_kernel<true><<<tgrid, 256, 0, stream>>>(src, source, channels, cpad, src_pixels,
                                                                  source_tail);
  else
    conv::to_blocked_bf16_kernel<false><<<tgrid, 256, 0, stream>>>(src, source, channels, cpad, src_pixels,
                                                                   source_tail);
  return true;
}

}  // namespace

// ---------------------------------------------------------------------------
// Launchers (scanned by the Python loader).
// ---------------------------------------------------------------------------

// One image: data_col[c, kh, kw, oh, ow] = data_im[c, ih, iw] or 0 in the padding.
template <typename T>
MOBULA_KERNEL im2col_kernel(const int n, const T* data_im, const int height, const int width,
                            const int kernel_h, const int kernel_w, const int pad_h, const int pad_w,
                            const int stride_h, const int stride_w, const int dilation_h,
                            const int dilation_w, const int height_col, const int width_col,
                            T* data_col) {
  if (n <= 0) return;
  if (!fits("im2col", 14, n)) return;
  conv::im2col_kernel<<<blocks_for(n), 256, 0, call_state().stream>>>(
      n, data_im, height, width, kernel_h, kernel_w, pad_h, pad_w, stride_h, stride_w, dilation_h,
      dilation_w, height_col, width_col, data_col);
  MOBULA_HIP_TRY(hipGetLastError());
}

// One image: data_im[c, h, w] = sum of the column entries that were read from it.
template <typename T>
MOBULA_KERNEL col2im_kernel(const int n, const T* data_col, const int height, const int width,
                            const int kernel_h, const int kernel_w, const int pad_h, const int pad_w,
                            const int stride_h, const int stride_w, const int dilation_h,
                            const int dilation_w, const int height_col, const int width_col,
                            T* data_im) {
  if (n <= 0) return;
  if (!fits("col2im", 14, n)) return;
  conv::col2im_kernel<<<blocks_for(n), 256, 0, call_state().stream>>>(
      n, data_col, height, width, kernel_h, kernel_w, pad_h, pad_w, stride_h, stride_w, dilation_h,
      dilation_w, height_col, width_col, data_im);
  MOBULA_HIP_TRY(hipGetLastError());
}

// y[N, D, OH, OW] = conv(x[N, C, H, W], weight[D, C, KH, KW]) (+ bias[D] if has_bias).
// n is the element count of y.
template <typename T>
MOBULA_KERNEL conv2d_forward_kernel(const int n, const T* x, const T* weight, const T* bias,
                                    const int has_bias, const int batch, const int channels,
                                    const int height, const int width, const int filters,
                                    const int kernel_h, const int kernel_w, const int pad_h,
                                    const int pad_w, const int stride_h, const int stride_w,
                                    const int dilation_h, const int dilation_w, T* y) {
  conv::Geometry g;
  if (!describe(&g, "conv2d_forward", batch, channels, height, width, filters, kernel_h, kernel_w, pad_h,
                pad_w, stride_h, stride_w, dilation_h, dilation_w))
    return;
  const long long out = static_cast<long long>(g.N) * g.D * g.OH * g.OW;
  if (n != out) { set_error("conv2d_forward: n=%d, the output has %lld elements", n, out); return; }
  if (!fits("conv2d_forward", 1, static_cast<long long>(g.N) * g.C * g.H * g.W) ||
      !fits("conv2d_forward", 2, static_cast<long long>(g.D) * g.C * g.KH * g.KW) ||
      (has_bias && !fits("conv2d_forward", 3, g.D)) || !fits("conv2d_forward", 18, out))
    return;
  if (out == 0) return;
  hipStream_t stream = call_state().stream;
  conv::ForwardOps ops;
  ops.x = x; ops.bias = has_bias ? bias : nullptr; ops.y = y; ops.g = g;
  ops.M = g.D; ops.Ncols = g.N * g.OH * g.OW;
  if ((compute_mode() == conv::kBf16 || compute_mode() == conv::kBf16x3) && g.N < 65536) {
    // operands as bf16 in memory: channel-blocked copy of x, weights by K step (heads and tails
    // of both with split operands)
    bool taken = true;
    {
      mobula_hip::KernelTimer timer("conv2d_forward", stream);
      conv::ForwardOpsB16 ob;
      ob.bias = ops.bias; ob.y = y; ob.Ncols = ops.Ncols;
      float* pieces = nullptr;
      const long long taps = g.KH * g.KW;
      if (plan_gather_b16(&ob, &pieces, "conv2d_forward", g, weight, g.D, g.C, x, g.N, g.H * g.W, g.OH * g.OW,
                          g.C * taps, taps, compute_mode() == conv::kBf16x3, &taken, stream)) {
        launch_igemm_b16(ob, pieces, stream);
        MOBULA_HIP_TRY(hipGetLastError());
        return;
      }
    }
    if (taken) return;   // (with an error; not taken: the kernels below split fp32 operands themselves)
  }
  {
    mobula_hip::KernelTimer timer("conv2d_forward", stream);
    GatherPlan plan;
    const long long taps = g.KH * g.KW;
    if (!plan_gather(&plan, "conv2d_forward", g, weight, g.D, g.C, static_cast<long long>(g.C) * g.H * g.W,
                     g.OH * g.OW, g.W, +1, g.C * taps, taps, stream))
      return;
    ops.wp = plan.weights; ops.steps = plan.steps; ops.K = plan.K;
    launch_igemm(ops, plan.pieces, stream);
  }
  MOBULA_HIP_TRY(hipGetLastError());
}

// dx[N, C, H, W] (+)= the gradient of conv2d_forward with respect to x.  n is the
// element count of dx.
template <typename T>
MOBULA_KERNEL conv2d_backward_data_kernel(const int n, const T* dy, const T* weight, const int accumulate,
                                          const int batch, const int channels, const int height,
                                          const int width, const int filters, const int kernel_h,
                                          const int kernel_w, const int pad_h, const int pad_w,
                                          const int stride_h, const int stride_w, const int dilation_h,
                                          const int dilation_w, T* dx) {
  conv::Geometry g;
  if (!describe(&g, "conv2d_backward_data", batch, channels, height, width, filters, kernel_h, kernel_w,
                pad_h, pad_w, stride_h, stride_w, dilation_h, dilation_w))
    return;
  const long long in = static_cast<long long>(g.N) * g.C * g.H * g.W;
  if (n != in) { set_error("conv2d_backward_data: n=%d, dx has %lld elements", n, in); return; }
  if (!fits("conv2d_backward_data", 1, static_cast<long long>(g.N) * g.D * g.OH * g.OW) ||
      !fits("conv2d_backward_data", 2, static_cast<long long>(g.D) * g.C * g.KH * g.KW) ||
      !fits("conv2d_backward_data", 17, in))
    return;
  if (in == 0) return;
  hipStream_t stream = call_state().stream;
  conv::BackwardDataOps ops;
  ops.dy = dy; ops.dx = dx; ops.g = g; ops.accumulate = accumulate;
  ops.M = g.C; ops.Ncols = g.N * g.H * g.W;
  if ((compute_mode() == conv::kBf16 || compute_mode() == conv::kBf16x3) && g.N < 65536) {
    bool taken = true;
    {
      mobula_hip::KernelTimer timer("conv2d_backward_data", stream);
      conv::BackwardDataOpsB16 ob;
      ob.dx = dx; ob.accumulate = accumulate; ob.Ncols = ops.Ncols;
      float* pieces = nullptr;
      const long long taps = g.KH * g.KW;
      // row m of the left operand is input channel m: element [m][tap][d] = weight[d][m][tap]
      if (plan_gather_b16(&ob, &pieces, "conv2d_backward_data", g, weight, g.C, g.D, dy, g.N, g.OH * g.OW,
                          g.H * g.W, taps, g.C * taps, compute_mode() == conv::kBf16x3, &taken, stream)) {
        launch_igemm_b16(ob, pieces, stream);
        MOBULA_HIP_TRY(hipGetLastError());
        return;
      }
    }
    if (taken) return;
  }
  {
    mobula_hip::KernelTimer timer("conv2d_backward_data", stream);
    GatherPlan plan;
    const long long taps = g.KH * g.KW;
    // row m of the left operand is input channel m: element [m][tap][d] = weight[d][m][tap]
    if (!plan_gather(&plan, "conv2d_backward_data", g, weight, g.C, g.D,
                     static_cast<long long>(g.D) * g.OH * g.OW, g.H * g.W, g.OW, -1, taps, g.C * taps, stream))
      return;
    ops.wp = plan.weights; ops.steps = plan.steps; ops.K = plan.K;
    launch_igemm(ops, plan.pieces, stream);
  }
  MOBULA_HIP_TRY(hipGetLastError());
}

// dw[D, C, KH, KW] (+)= the gradient with respect to the weights.  n is the
// element count of dw.
template <typename T>
MOBULA_KERNEL conv2d_backward_weight_kernel(const int n, const T* dy, const T* x, const int accumulate,
                                            const int batch, const int channels, const int height,
                                            const int width, const int filters, const int kernel_h,
                                            const int kernel_w, const int pad_h, const int pad_w,
                                            const int stride_h, const int stride_w, const int dilation_h,
                                            const int dilation_w, T* dw) {
  conv::Geometry g;
  if (!describe(&g, "conv2d_backward_weight", batch, channels, height, width, filters, kernel_h, kernel_w,
                pad_h, pad_w, stride_h, stride_w, dilation_h, dilation_w))
    return;
  const long long wt = static_cast<long long>(g.D) * g.C * g.KH * g.KW;
  if (n != wt) { set_error("conv2d_backward_weight: n=%d, dw has %lld elements", n, wt); return; }
  if (!fits("conv2d_backward_weight", 1, static_cast<long long>(g.N) * g.D * g.OH * g.OW) ||
      !fits("conv2d_backward_weight", 2, static_cast<long long>(g.N) * g.C * g.H * g.W) ||
      !fits("conv2d_backward_weight", 17, wt))
    return;
  if (static_cast<long long>(g.C) * g.H * g.W * 4 >= (1ll << 31)) {
    set_error("conv2d_backward_weight: images too large for 32-bit byte offsets");
    return;
  }
  hipStream_t stream = call_state().stream;
  if ((compute_mode() == conv::kBf16 || compute_mode() == conv::kBf16x3) && g.stride_h == 1 && g.stride_w == 1 &&
      wt > 0 && g.N > 0) {
    // bf16 operands in memory on a common padded grid, one plain product per tap.  With split
    // operands (head + tail, two bf16 for every fp32) the copies hold two sets of planes, heads
    // then tails, and the product walks the images three times: head x head, head x tail, tail x head.
    const bool split = compute_mode() == conv::kBf16x3;
    const int sets = split ? 2 : 1;
    const int Hg = g.H + 2 * g.pad_h, Wg = g.W + 2 * g.pad_w;
    const long long G = static_cast<long long>(Hg) * Wg, Gp = (G + 31) / 32 * 32;
    const long long dy_set = 2ll * g.N * g.D * Gp, x_set = 2ll * g.N * g.C * Gp;   // bytes of one set of planes
    const long long dy_bytes = sets * dy_set, x_bytes = sets * x_set;
    if (dy_bytes < (1ll << 31) && 2 * x_bytes < (1ll << 31) && 3ll * g.N * Gp < (1ll << 31) && g.OH <= Hg &&
        g.OW <= Wg) {
      mobula_hip::KernelTimer timer("conv2d_backward_weight", stream);
      const size_t dy_room = (dy_bytes + 255) / 256 * 256, x_room = (x_bytes + 255) / 256 * 256;
      const size_t piece_bytes = sizeof(float) * kMaxPieceBlocks * conv::Tile::BM * conv::Tile::BN;
      char* ws = static_cast<char*>(mobula_hip::workspace(dy_room + 2 * x_room + piece_bytes));
      if (failed()) return;
      conv::WeightGradOpsB16 ob;
      unsigned short* const dyg = reinterpret_cast<unsigned short*>(ws);
      unsigned short* const xg = reinterpret_cast<unsigned short*>(ws + dy_room);
      ob.dyg = dyg; ob.xg = xg; ob.dw = dw; ob.g = g; ob.M = g.D; ob.Ncols = g.C * g.KH * g.KW;
      ob.split = split ? 1 : 0;
      ob.K = static_cast<int>((split ? 3 : 1) * g.N * Gp); ob.Gp = static_cast<int>(Gp); ob.Wg = Wg;
      ob.accumulate = accumulate;
      // the shifted copy follows the first one directly (x_bytes is a multiple of 64): the reads of
      // the last plane that run past its end then land in the other copy or beyond the buffer
      // (zeros), never in workspace bytes that nothing wrote
      ob.copy_bytes = static_cast<unsigned>(x_bytes);
      unsigned short* const xg1 = reinterpret_cast<unsigned short*>(ws + dy_room + x_bytes);
      const size_t dy_tail = split ? static_cast<size_t>(dy_set / 2) : 0, x_tail = split ? static_cast<size_t>(x_set / 2) : 0;
      // whole grid rows per workgroup and 16-byte loads where rows of both tensors allow it (a span
      // of rows must be a multiple of 8 positions: Wg even and four rows, or any rows if Wg % 8 == 0)
      int rows = (conv::kPaddedSpan - 32) / Wg;   // (the last span also takes the tail of the plane: up to 31 positions)
      if (Wg % 8 != 0) rows = Wg % 2 == 0 ? rows / 4 * 4 : 0;
      const bool vec = rows > 0 && g.W % 4 == 0 && g.OW % 4 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0 &&
                       reinterpret_cast<uintptr_t>(dy) % 16 == 0;
      if (vec) {
        rows = std::min(rows, (Hg + 3) / 4 * 4);
        const unsigned spans = static_cast<unsigned>((Hg + rows - 1) / rows);
        conv::to_padded_bf16_rows_kernel<<<dim3(g.N * g.D, spans), 256, 0, stream>>>(
            dy, dyg, nullptr, g.OH, g.OW, 0, 0, Hg, Wg, static_cast<int>(Gp), rows, dy_tail);
        conv::to_padded_bf16_rows_kernel<<<dim3(g.N * g.C, spans), 256, 0, stream>>>(
            x, xg, xg1, g.H, g.W, g.pad_h, g.pad_w, Hg, Wg, static_cast<int>(Gp), rows, x_tail);
      } else {
        // a plane in as few, equally long spans as fit the kernel's LDS
        const int spans = static_cast<int>((Gp + conv::kPaddedSpan - 1) / conv::kPaddedSpan);
        const int span = static_cast<int>((Gp / 8 + spans - 1) / spans * 8);
        conv::to_padded_bf16_kernel<<<dim3(g.N * g.D, spans), 256, 0, stream>>>(dy, dyg, nullptr, g.OH, g.OW, 0, 0, Hg,
                                                                               Wg, static_cast<int>(Gp), span, dy_tail);
        conv::to_padded_bf16_kernel<<<dim3(g.N * g.C, spans), 256, 0, stream>>>(
            x, xg, xg1, g.H, g.W, g.pad_h, g.pad_w, Hg, Wg, static_cast<int>(Gp), span, x_tail);
      }
      launch_igemm_b16(ob, reinterpret_cast<float*>(ws + dy_room + 2 * x_room), stream);
      MOBULA_HIP_TRY(hipGetLastError());
      return;
    }
  }
  conv::BackwardWeightOps ops;
  ops.dy = dy; ops.x = x; ops.g = g;
  ops.M = g.D; ops.Ncols = g.C * g.KH * g.KW; ops.K = 0; ops.k_begin = 0;
  // K = N*OH*OW is long and the result small: K is cut into slices of whole K
  // steps, as many as give every CU four workgroups; the partial sums of the
  // slices are added in a fixed order afterwards.
  const int row_tiles = (ops.M + conv::Tile::BM - 1) / conv::Tile::BM;
  const long long per_slice_tiles = static_cast<long long>(row_tiles) * ((ops.Ncols + conv::Tile::BN - 1) / conv::Tile::BN);
  const long long k_total = static_cast<long long>(g.N) * g.OH * g.OW;   // < 2^31: checked by describe()
  if (per_slice_tiles >= (1ll << 20)) { set_error("conv2d_backward_weight: too many tiles"); return; }
  const long long k_steps = std::max<long long>(1, (k_total + conv::Tile::BK - 1) / conv::Tile::BK);
  long long slices = std::min<long long>(k_steps, std::max<long long>(1, kWeightSlots / per_slice_tiles));
  const long long k_per_slice = (k_steps + slices - 1) / slices * conv::Tile::BK;
  slices = std::max<long long>(1, (k_total + k_per_slice - 1) / k_per_slice);
  // a zero-padded copy of x saves the gathered operand its range tests where eight output pixels
  // of a row are eight neighbouring inputs (unit stride along a row); 32-bit offsets within an image
  const int Hp = g.H + 2 * g.pad_h, Wp = g.W + 2 * g.pad_w;
  const long long plane_p = static_cast<long long>(Hp) * Wp;
  const bool padded = g.stride_w == 1 && g.N > 0 && plane_p * g.C * 4 < (1ll << 31) && plane_p < (1ll << 22);
  const size_t partial_bytes = (sizeof(float) * static_cast<size_t>(slices) * wt + 255) / 256 * 256;
  const size_t padded_bytes = padded ? sizeof(float) * static_cast<size_t>(g.N) * g.C * plane_p : 0;
  char* extra = nullptr;
  ops.taps = make_taps(ops.Ncols, g.KH, g.KW, padded ? static_cast<int>(plane_p) : g.H * g.W, g.dil_h, g.dil_w,
                       partial_bytes + padded_bytes, &extra, stream);
  if (failed()) return;
  ops.partial = reinterpret_cast<float*>(extra);
  ops.xp = nullptr; ops.Hp = Hp; ops.Wp = Wp;
  {
    mobula_hip::KernelTimer timer("conv2d_backward_weight", stream);
    if (padded) {
      float* const xp = reinterpret_cast<float*>(extra + partial_bytes);
      conv::pad_planes_kernel<<<dim3(g.N * g.C, static_cast<unsigned>((plane_p + 2047) / 2048)), 256, 0, stream>>>(
          x, xp, g.H, g.W, g.pad_h, g.pad_w, Hp, Wp);
      ops.xp = xp;
    }
    const int tps = static_cast<int>(per_slice_tiles), count = tps * static_cast<int>(slices);
    const dim3 grid(conv::tile_blocks(count));
    switch (compute_mode()) {
      case conv::kBf16:
        conv::igemm_weight_kernel<conv::kBf16><<<grid, conv::Tile::NT, 0, stream>>>(
            ops, static_cast<int>(k_per_slice), static_cast<int>(k_total), row_tiles, tps, count); break;
      case conv::kBf16x3:
        conv::igemm_weight_kernel<conv::kBf16x3><<<grid, conv::Tile::NT, 0, stream>>>(
            ops, static_cast<int>(k_per_slice), static_cast<int>(k_total), row_tiles, tps, count); break;
      default:
        conv::igemm_weight_kernel<conv::kFp32><<<grid, conv::Tile::NT, 0, stream>>>(
            ops, static_cast<int>(k_per_slice), static_cast<int>(k_total), row_tiles, tps, count);
    }
    conv::reduce_slices_kernel<<<blocks_for(wt), 256, 0, stream>>>(ops.partial, dw, wt, static_cast<int>(slices), accumulate);
  }
  MOBULA_HIP_TRY(hipGetLastError());
}

// db[D] (+)= sum of dy over images and pixels.  n = D.
template <typename T>
MOBULA_KERNEL conv2d_backward_bias_kernel(const int n, const T* dy, const int accumulate, const int batch,
                                          const int pixels, T* db) {
  if (n <= 0) return;
  if (batch < 0 || pixels < 0) { set_error("conv2d_backward_bias: batch=%d pixels=%d", batch, pixels); return; }
  if (!fits("conv2d_backward_bias", 1, static_cast<long long>(batch) * n * pixels) ||
      !fits("conv2d_backward_bias", 5, n))
    return;
  conv::bias_grad_kernel<<<n, 256, 0, call_state().stream>>>(dy, db, batch, n, pixels, accumulate);
  MOBULA_HIP_TRY(hipGetLastError());
}

// ---------------------------------------------------------------------------
// Entry points.  Device pointers only: the convolution does not stage host
// buffers (device id -1 is an error here).
// ---------------------------------------------------------------------------
namespace {
bool on_device(const char* what, int device_id) {
  mobula_hip::begin_call();
  if (device_id >= 0) return true;
  set_error("%s: host buffers are not supported, pass device tensors", what);
  mobula_hip::finish_call();
  return false;
}
}  // namespace

#define CONV_GEOMETRY_PARAMS                                                                          \
  const int batch, const int channels, const int height, const int width, const int filters,          \
      const int kernel_h, const int kernel_w, const int pad_h, const int pad_w, const int stride_h,   \
      const int stride_w, const int dilation_h, const int dilation_w
#define CONV_GEOMETRY_ARGS                                                                             \
  batch, channels, height, width, filters, kernel_h, kernel_w, pad_h, pad_w, stride_h, stride_w,       \
      dilation_h, dilation_w

extern "C" {

void im2col_341af5d3(const int device_id, const int n, const float* data_im, const int height,
                     const int width, const int kernel_h, const int kernel_w, const int pad_h,
                     const int pad_w, const int stride_h, const int stride_w, const int dilation_h,
                     const int dilation_w, const int height_col, const int width_col, float* data_col) {
  if (!on_device("im2col", device_id)) return;
  mobula_hip::DeviceScope scope(device_id);
  if (scope.ok())
    im2col_kernel<float>(n, data_im, height, width, kernel_h, kernel_w, pad_h, pad_w, stride_h, stride_w,
                         dilation_h, dilation_w, height_col, width_col, data_col);
  mobula_hip::finish_call();
}

void col2im_341af5d3(const int device_id, const int n, const float* data_col, const int height,
                     const int width, const int kernel_h, const int kernel_w, const int pad_h,
                     const int pad_w, const int stride_h, const int stride_w, const int dilation_h,
                     const int dilation_w, const int height_col, const int width_col, float* data_im) {
  if (!on_device("col2im", device_id)) return;
  mobula_hip::DeviceScope scope(device_id);
  if (scope.ok())
    col2im_kernel<float>(n, data_col, height, width, kernel_h, kernel_w, pad_h, pad_w, stride_h, stride_w,
                         dilation_h, dilation_w, height_col, width_col, data_im);
  mobula_hip::finish_call();
}

void conv2d_forward_c6a7aa85(const int device_id, const int n, const float* x, const float* weight,
                            const float* bias, const int has_bias, CONV_GEOMETRY_PARAMS, float* y) {
  if (!on_device("conv2d_forward", device_id)) return;
  mobula_hip::DeviceScope scope(device_id);
  if (scope.ok()) conv2d_forward_kernel<float>(n, x, weight, bias, has_bias, CONV_GEOMETRY_ARGS, y);
  mobula_hip::finish_call();
}

void conv2d_backward_data_ecf81c91(const int device_id, const int n, const float* dy, const float* weight,
                                  const int accumulate, CONV_GEOMETRY_PARAMS, float* dx) {
  if (!on_device("conv2d_backward_data", device_id)) return;
  mobula_hip::DeviceScope scope(device_id);
  if (scope.ok()) conv2d_backward_data_kernel<float>(n, dy, weight, accumulate, CONV_GEOMETRY_ARGS, dx);
  mobula_hip::finish_call();
}

void conv2d_backward_weight_ecf81c91(const int device_id, const int n, const float* dy, const float* x,
                                    const int accumulate, CONV_GEOMETRY_PARAMS, float* dw) {
  if (!on_device("conv2d_backward_weight", device_id)) return;
  mobula_hip::DeviceScope scope(device_id);
  if (scope.ok()) conv2d_backward_weight_kernel<float>(n, dy, x, accumulate, CONV_GEOMETRY_ARGS, dw);
  mobula_hip::finish_call();
}

void conv2d_backward_bias_cd239a08(const int device_id, const int n, const float* dy, const int accumulate,
                                   const int batch, const int pixels, float* db) {
  if (!on_device("conv2d_backward_bias", device_id)) return;
  mobula_hip::DeviceScope scope(device_id);
  if (scope.ok()) conv2d_backward_bias_kernel<float>(n, dy, accumulate, batch, pixels, db);
  mobula_hip::finish_call();
}

}  // extern "C"

static mobula_hip::ExportRegistrar conv_exports(
    "im2col_341af5d3 col2im_341af5d3 conv2d_forward_c6a7aa85 conv2d_backward_data_ecf81c91 "
    "conv2d_backward_weight_ecf81c91 conv2d_backward_bias_cd239a08");
