// ROIAlign launchers for gfx950 and their C-ABI entry points.
//
// The MOBULA_KERNEL declarations below are what `mobula.op.load('ROIAlign')`
// scans to bind `mobula.func.roi_align_forward / roi_align_backward /
// roi_align_backward_assign`; argument lists and meaning are those of the
// reference kernels (opzoo/ROIAlign/ROIAlign.cpp:9-16, 78-83).  The extern "C"
// functions at the end carry the names the reference's loader derives for the
// same instantiations (mobula/func.py:13-50, op/templates/kernel_code.cpp:1-5).
#include <algorithm>
#include <mutex>
#include <type_traits>

#include "runtime.h"
#include "roialign_naive.hip.h"
#include "roialign_f64.hip.h"
#include "roialign_backward_blocked.hip.h"
#include "roialign_forward_blocked.hip.h"
#include "roialign_forward_merged.hip.h"

namespace {

using mobula_hip::arg_extent;
using mobula_hip::call_state;
using mobula_hip::failed;
using mobula_hip::set_error;

enum Impl { kAuto = 0, kTiled = 1, kNaive = 2 };

// Helper kernels move to a second stream only above these sizes (measured: below
// them the hand-over costs more than the overlap gains).
constexpr int kSideStreamRois = 4096;
constexpr int kOrderInCopyRois = 16384;   // ROIs that the workgroup riding along with the transposition sorts
constexpr long long kSideStreamBytes = 64ll << 20;
// Maps up to this size are gathered in the caller's ROI order: each of the eight
// L2 caches (4 MB) then holds its eighth of the map's channel blocks whole.
constexpr size_t kSortedAboveBytes = 24u << 20;

struct Problem {
  long long n_out;  // R*C*PH*PW
  int R, C, H, W, PH, PW, S;
  long long N;      // images in the feature map
  float scale;
  double scale64 = 0.0;  // the scale as given, for the binary64 kernels
  bool nhwc = false;   // map [N,H,W,C] and pooled tensor [R,PH,PW,C] instead of [N,C,H,W] / [R,C,PH,PW]
  // Scratch memory the caller of forward_device provides instead of the thread's
  // workspace (the entry point that allocates nothing): no allocation, no second
  // stream, no event is made on that path.
  char* fixed_scratch = nullptr;
  size_t fixed_scratch_bytes = 0;
};

// Shape checks shared by every entry point.  Returns false (with the error
// text set) if the arguments cannot describe a valid problem.  `ext_*` are
// the positions of the pointer arguments in the call, for the extents the
// caller may have declared.
bool describe(Problem* p, const char* what, int nthreads, float scale, int C, int H, int W,
              int PH, int PW, int S, int ext_map, int ext_rois, int ext_pooled,
              long long num_images_hint) {
  if (nthreads < 0 || C <= 0 || H <= 0 || W <= 0 || PH <= 0 || PW <= 0) {
    set_error("%s: non-positive dimension (nthreads=%d C=%d H=%d W=%d PH=%d PW=%d)", what,
              nthreads, C, H, W, PH, PW);
    return false;
  }
  const long long per_roi = static_cast<long long>(C) * PH * PW;
  if (nthreads % per_roi != 0) {
    set_error("%s: nthreads=%d is not a multiple of C*PH*PW=%lld", what, nthreads, per_roi);
    return false;
  }
  const long long plane = static_cast<long long>(H) * W;
  if (plane * C >= (1ll << 31)) {
    set_error("%s: C*H*W=%lld does not fit 32-bit indexing", what, plane * C);
    return false;
  }
  p->n_out = nthreads;
  p->R = static_cast<int>(nthreads / per_roi);
  p->C = C; p->H = H; p->W = W; p->PH = PH; p->PW = PW; p->S = S;
  p->scale = scale;
  p->N = num_images_hint;
  const long long e_map = arg_extent(ext_map), e_rois = arg_extent(ext_rois),
                  e_pool = arg_extent(ext_pooled);
  if (e_rois >= 0 && e_rois != 5ll * p->R) {
    set_error("%s: rois holds %lld values, expected R*5=%lld", what, e_rois, 5ll * p->R);
    return false;
  }
  if (e_pool >= 0 && e_pool != p->n_out) {
    set_error("%s: pooled tensor holds %lld values, expected %lld", what, e_pool, p->n_out);
    return false;
  }
  if (e_map >= 0) {
    if (e_map % (plane * C) != 0) {
      set_error("%s: feature map holds %lld values, not a multiple of C*H*W=%lld", what, e_map,
                plane * C);
      return false;
    }
    const long long n = e_map / (plane * C);
    if (p->N >= 0 && p->N != n) {
      set_error("%s: num_images=%lld but the feature map holds %lld images", what, p->N, n);
      return false;
    }
    p->N = n;
  }
  return true;
}

// Number of images when the caller gave neither extents nor a count: read the
// largest batch index back from the device (one blocking copy).
template <typename B>
long long images_from_rois(const B* d_rois, int R, hipStream_t stream) {
  if (R == 0) return 0;
  int* d_max = static_cast<int*>(mobula_hip::workspace(256));
  if (failed()) return 0;
  roialign::zero_words_kernel<<<1, 64, 0, stream>>>(reinterpret_cast<unsigned*>(d_max), 1);
  roialign::max_batch_kernel<<<std::min(64, (R + 255) / 256), 256, 0, stream>>>(d_rois, R, d_max);
  int h = 0;
  MOBULA_HIP_TRY(hipMemcpyAsync(&h, d_max, sizeof(int), hipMemcpyDeviceToHost, stream));
  MOBULA_HIP_TRY(hipStreamSynchronize(stream));
  return h;
}

// The fixed scratch buffer of roi_align_forward_noalloc: every GPU the library
// runs on holds its own copy of this array at its own address.  Host code never
// uses the array's name as an address; it asks once per device, with that
// device current, for the device address and keeps it.
constexpr size_t kNoAllocScratchBytes = 48u << 20;
constexpr int kNoAllocMaxDevices = 64;
}  // namespace
static __device__ __align__(256) unsigned char roialign_noalloc_scratch[kNoAllocScratchBytes];
namespace {
std::mutex g_noalloc_mutex;
char* g_noalloc_ptr[kNoAllocMaxDevices] = {};

// Device address of the current device's copy of the buffer (null and an error if it cannot be had).
char* noalloc_scratch(size_t* bytes) {
  *bytes = kNoAllocScratchBytes;
  int device = -1;
  MOBULA_HIP_TRY(hipGetDevice(&device));
  if (failed()) return nullptr;
  if (device < 0 || device >= kNoAllocMaxDevices) {
    set_error("roi_align_forward_noalloc: device %d is beyond the %d the fixed buffer is kept for", device,
              kNoAllocMaxDevices);
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(g_noalloc_mutex);
  if (g_noalloc_ptr[device] == nullptr) {
    void* ptr = nullptr;
    MOBULA_HIP_TRY(hipGetSymbolAddress(&ptr, HIP_SYMBOL(roialign_noalloc_scratch)));
    if (failed() || ptr == nullptr) {
      if (!failed()) set_error("roi_align_forward_noalloc: the fixed buffer has no address on device %d", device);
      return nullptr;
    }
    g_noalloc_ptr[device] = static_cast<char*>(ptr);
  }
  return g_noalloc_ptr[device];
}

int grid_for(long long n, int block) {
  return static_cast<int>(std::min<long long>((n + block - 1) / block, 256ll * 64));
}

bool use_tiled();

// True if the channels-last entry points take the shape (they have no
// straightforward fallback: the caller converts to NCHW instead).
template <typename T>
bool nhwc_forward_supported(const Problem& p) {
  return roialign::blocked_rows_per_pass<T>(p.C, p.H, p.W, p.PH, p.PW, p.S != 1 && p.S != 2) > 0 &&
         static_cast<long long>(p.H) * p.W * p.C * static_cast<long long>(sizeof(T)) < (1ll << 31);
}

template <typename T>
void forward_device(const Problem& p, const T* x, const float* rois, T* y, hipStream_t stream) {
  if (p.n_out == 0) return;
  using FB = roialign::FwdBlocked;
  constexpr int CB = roialign::BlockOf<T>::CB;
  const long long pixels = static_cast<long long>(p.H) * p.W;
  const int cblk = (p.C + CB - 1) / CB;
  const bool small_grid = p.S == 1 || p.S == 2;   // else: sampling grids above 2 x 2, merged lists
  const int rpp = roialign::blocked_rows_per_pass<T>(p.C, p.H, p.W, p.PH, p.PW, !small_grid);
  const int nw = small_grid ? FB::NW : roialign::FwdMerged::NW;   // wavefronts per workgroup of the gather
  const long long grid = roialign::blocked_grid(p.R, cblk, nw);
  const bool fits = rpp > 0 && p.N > 0 && p.N < 65536 && cblk < 65536 && grid < (1ll << 31);
  if (p.nhwc) {
    // the map is read where it lies: no copy, only the ROI ordering before the gather
    if (!fits || !nhwc_forward_supported<T>(p) || reinterpret_cast<size_t>(x) % 16 != 0 ||
        reinterpret_cast<size_t>(y) % 16 != 0) {
      set_error("roi_align_forward_nhwc: shape C=%d H=%d W=%d pooled %dx%d (or the alignment of the tensors) "
                "is not taken by the channels-last path", p.C, p.H, p.W, p.PH, p.PW);
      return;
    }
    int* order = nullptr;   // (a map that stays in the L2 caches is read in the caller's ROI order)
    if (sizeof(T) * p.N * pixels * p.C > kSortedAboveBytes) {
      order = static_cast<int*>(mobula_hip::workspace(sizeof(int) * p.R));
      if (failed()) return;
      roialign::roi_order_kernel<<<1, 1024, 0, stream>>>(rois, p.R, p.scale, p.H, p.W, p.N, order);
    }
    const long long grid = roialign::blocked_grid_nhwc(p.R, cblk, nw);
    if (small_grid) {
      mobula_hip::KernelTimer timer("forward_blocked_kernel", stream);
      roialign::forward_blocked_kernel<T, true><<<static_cast<unsigned>(grid), FB::NW * 64, 0, stream>>>(
          x, rois, order, y, p.scale, p.C, p.H, p.W, p.PH, p.PW, p.S, p.N, cblk, p.PH, p.R);
    } else {
      {
        mobula_hip::KernelTimer timer("forward_merged_kernel", stream);
        roialign::forward_merged_kernel<T, true><<<static_cast<unsigned>(grid), nw * 64, 0, stream>>>(
            x, rois, order, y, p.scale, p.C, p.H, p.W, p.PH, p.PW, p.S, p.N, cblk, p.PH, p.R);
      }
      // the boxes that kernel leaves out (sampling grids of more than 64 points per axis)
      if (p.S <= 0 || p.S > roialign::kSearchedGrid)
        roialign::forward_large_grid_kernel<T, true><<<static_cast<unsigned>(p.R), 64, 0, stream>>>(
          x, p.scale, p.C, p.H, p.W, p.PH, p.PW, p.S, rois, y, p.N);
    }
    MOBULA_HIP_TRY(hipGetLastError());
    return;
  }
  if (use_tiled() && fits) {
    // channel-blocked copy of the map, spatial ROI order, then the gather
    const size_t xt_bytes = (sizeof(T) * p.N * cblk * CB * pixels + 255) / 256 * 256;
    const bool fixed = p.fixed_scratch != nullptr;
    if (fixed && xt_bytes + sizeof(int) * p.R > p.fixed_scratch_bytes) {
      set_error("roi_align_forward_noalloc: the problem needs %zu bytes of scratch memory, the library's fixed "
                "buffer holds %zu (feature map too large for the entry point that allocates nothing)",
                xt_bytes + sizeof(int) * p.R, p.fixed_scratch_bytes);
      return;
    }
    char* const ws = fixed ? p.fixed_scratch : static_cast<char*>(mobula_hip::workspace(xt_bytes + sizeof(int) * p.R));
    if (failed()) return;
    T* const xt = reinterpret_cast<T*>(ws);
    // ROIs are visited in spatial order when the map is larger than the L2 caches
    // hold; a small map is read in the caller's order and the ordering kernel is left out
    int* const order = xt_bytes > kSortedAboveBytes ? reinterpret_cast<int*>(ws + xt_bytes) : nullptr;
    // the ROI ordering (one small workgroup) runs beside the transposition: in the same launch
    // for up to kOrderInCopyRois ROIs (nothing to hand over), on a second stream above that
    // (handing work to a second stream and waiting for it costs 10-15 us: only worth it when
    // the ordering of many ROIs would otherwise delay the gather)
    const bool order_in_copy = order != nullptr && p.R <= kOrderInCopyRois;
    mobula_hip::SideStream side(stream, !fixed && order != nullptr && !order_in_copy && p.R > kSideStreamRois);
    if (order != nullptr && !order_in_copy)
      roialign::roi_order_kernel<<<1, 1024, 0, side.get()>>>(rois, p.R, p.scale, p.H, p.W, p.N, order);
    const roialign::OrderArgs oa{rois, order_in_copy ? order : nullptr, static_cast<int>(p.R), p.scale, p.H, p.W, p.N};
    const dim3 tgrid(static_cast<unsigned>((pixels + 63) / 64) + (order_in_copy ? 1u : 0u),
                     static_cast<unsigned>(cblk), static_cast<unsigned>(p.N));
    const bool vec = pixels % 4 == 0 && reinterpret_cast<size_t>(x) % (4 * sizeof(T)) == 0;
    if (vec)
      roialign::transpose_to_blocked_kernel<T, true><<<tgrid, 256, 0, stream>>>(
          x, xt, p.C, static_cast<int>(pixels), oa);
    else
      roialign::transpose_to_blocked_kernel<T, false><<<tgrid, 256, 0, stream>>>(
          x, xt, p.C, static_cast<int>(pixels), oa);
    side.join();
    if (small_grid) {
      mobula_hip::KernelTimer timer("forward_blocked_kernel", stream, !fixed);   // (its events are allocations)
      roialign::forward_blocked_kernel<T, false><<<static_cast<unsigned>(grid), FB::NW * 64, 0, stream>>>(
          xt, rois, order, y, p.scale, p.C, p.H, p.W, p.PH, p.PW, p.S, p.N, cblk, rpp, p.R);
    } else {
      // every pixel of a bin is loaded once
      {
        mobula_hip::KernelTimer timer("forward_merged_kernel", stream, !fixed);
        roialign::forward_merged_kernel<T, false><<<static_cast<unsigned>(grid), nw * 64, 0, stream>>>(
            xt, rois, order, y, p.scale, p.C, p.H, p.W, p.PH, p.PW, p.S, p.N, cblk, rpp, p.R);
      }
      // the boxes that kernel leaves out (sampling grids of more than 64 points per axis), from the map itself
      if (p.S <= 0 || p.S > roialign::kSearchedGrid)
        roialign::forward_large_grid_kernel<T, false><<<static_cast<unsigned>(p.R), 64, 0, stream>>>(
          x, p.scale, p.C, p.H, p.W, p.PH, p.PW, p.S, rois, y, p.N);
    }
    MOBULA_HIP_TRY(hipGetLastError());
    return;
  }
  roialign::forward_naive_kernel<T><<<grid_for(p.n_out, 256), 256, 0, stream>>>(
      p.n_out, x, p.scale, p.C, p.H, p.W, p.PH, p.PW, p.S, rois, y, p.N);
  MOBULA_HIP_TRY(hipGetLastError());
}

// Scratch layout of the tile pre-pass, carved out of the device workspace.
struct TilePlan {
  bool dy_transposed = false;   // the pre-pass also wrote dyb (plan_tiles was given dy)
  roialign::TileGrid grid;
  roialign::TileBox* boxes;
  int* cursors;                // bump pointers: [0] ROI lists, [1] work lists
  int* tile_rois;
  roialign::ListLayout layout;
  roialign::AxisUnit* lists;
  float* dyb;                  // channel-blocked copy of dy (null for channels-last tensors)
  size_t dyb_bytes, list_bytes;   // dyb_bytes: of one channel block's slab
  roialign::WorkRange* ranges; // per (tile, tile row)
  roialign::WorkEntry* entries;
};

size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

// Runs the pre-pass (ROI boxes and sample tables, per-tile ROI and work lists) for tiles of th x tw
// pixels.  Returns false if the problem is too large for the list buffers (or
// on error); the caller then uses the straightforward kernels.
// How transpose_dy_blocked_kernel is launched for a problem: channel blocks per
// workgroup (what 32 KB of LDS hold, at most 4, at least one; 0: not even one in 64 KB), workgroups, LDS bytes.
struct DyLaunch { int per; long long blocks; size_t lds; int cap; };
template <typename T>
DyLaunch dy_launch(const Problem& p) {
  using BB = roialign::BwdBlocked;
  const int cblk = (p.C + BB::CB - 1) / BB::CB;
  const size_t chan_bytes = sizeof(T) * p.PH * p.PW, blk_bytes = BB::CB * chan_bytes;
  // (as many blocks as 32 KB hold, at least one if 64 KB hold it: with 25 KB blocks -- 14 x 14
  // pooled maps -- one block per workgroup copies at 5.8 TB/s where two manage 5.1: more
  // workgroups fit a CU)
  const int per = blk_bytes > 64 * 1024 ? 0 : static_cast<int>(std::min<size_t>(4, std::max<size_t>(1, (32 * 1024) / blk_bytes)));
  if (per > 0)
    return DyLaunch{per, static_cast<long long>(p.R) * ((cblk + per - 1) / per), per * blk_bytes, 0};
  // large pooled sizes: one channel block per workgroup, in passes of `cap` channels
  const int cap = static_cast<int>((64 * 1024) / chan_bytes) & ~3;
  return DyLaunch{0, cap >= 4 ? static_cast<long long>(p.R) * cblk : 0, cap * chan_bytes, cap};
}

// fuse_dy (optional): dy of the call; its transposition into plan->dyb then shares
// the launch of the list builder (plan->dy_transposed says whether it did).
template <typename T>
bool plan_tiles(const Problem& p, const float* rois, int th, int tw, bool with_dyb,
                hipStream_t stream, TilePlan* plan, const T* fuse_dy = nullptr) {
  // List items: the ROIs, or for sampling grids of more than 2 x 2 points the
  // windows of merged weights their bins are cut into.  How many depends on the
  // boxes, so their number has to come back from the device (one blocking copy:
  // not while the stream is being captured into a graph).
  const bool windows = roialign::lists_in_windows(p.S);
  long long items = p.R, window_entries = 0;
  // the head of the workspace: offsets[R + 1], info[3], counts[R], work[R] (see window_offsets_kernel)
  const size_t b_offsets = windows ? align_up(sizeof(int) * (p.R + 4) + sizeof(int) * p.R + 8, 256) +
                                         align_up(sizeof(long long) * p.R, 256) : 0;
  char* head = nullptr;
  auto number_windows = [&](char* at) {
    int* const offsets = reinterpret_cast<int*>(at);
    int* const counts = offsets + p.R + 4;
    long long* const work = reinterpret_cast<long long*>(at + align_up(sizeof(int) * (2 * p.R + 4) + 8, 256));
    if (p.R > 0)
      roialign::window_counts_kernel<<<grid_for(p.R, 256), 256, 0, stream>>>(rois, p.R, p.scale, p.PH, p.PW, p.S, p.H,
                                                                            p.W, tw, counts, work);
    roialign::window_offsets_kernel<<<1, 1024, 0, stream>>>(counts, work, p.R, offsets, offsets + p.R + 1);
  };
  if (p.S > roialign::kSearchedGrid) return false;   // (fixed grids of that size are not merged)
  if (windows) {
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &capture) != hipSuccess || capture != hipStreamCaptureStatusNone) {
      (void)hipGetLastError();
      return false;
    }
    head = static_cast<char*>(mobula_hip::workspace(b_offsets));
    if (failed()) return false;
    number_windows(head);
    int info[3] = {0, 1, 0};
    MOBULA_HIP_TRY(hipMemcpyAsync(info, reinterpret_cast<int*>(head) + p.R + 1, sizeof(info), hipMemcpyDeviceToHost,
                                  stream));
    MOBULA_HIP_TRY(hipStreamSynchronize(stream));
    if (failed() || info[1] != 0) return false;   // an adaptive grid too large to merge
    items = info[0];
    window_entries = info[2];
  }
  if (items > (1ll << 22)) return false;
  roialign::TileGrid& g = plan->grid;
  g.th = th; g.tw = tw;
  g.ty = (p.H + th - 1) / th;
  g.tx = (p.W + tw - 1) / tw;
  g.per_image = g.ty * g.tx;
  g.total = static_cast<long long>(g.per_image) * p.N;
  const long long list_cap = items * g.per_image;  // every item in every tile
  if (g.total <= 0 || g.total > (1ll << 24) || list_cap > (1ll << 27)) return false;
  const size_t b_recs = align_up(sizeof(roialign::TileBox) * std::max<long long>(items, 1), 256);
  const size_t b_cnt = 256;   // the two bump pointers
  const size_t b_list = align_up(sizeof(int) * std::max<long long>(list_cap, 1), 256);
  plan->layout = roialign::make_list_layout(g, p.PH, p.PW, p.S);
  const long long n_units = plan->layout.roi_stride * items;
  if (n_units > (1ll << 25)) return false;   // 512 MiB of sample lists: not worth it
  const size_t b_units = align_up(sizeof(roialign::AxisUnit) * n_units, 256) + 256;  // blocks are read whole
  const int cblk = (p.C + 31) / 32;
  // dyb: one slab per channel block (all ROIs), 256-byte aligned
  // (a multiple of 128 bytes; the slabs follow each other as the transposition writes them)
  const size_t b_slab = with_dyb ? sizeof(float) * 32 * p.PW * p.R * p.PH : 0;
  const size_t b_dyt = align_up(b_slab * cblk, 256);
  // work lists: every tap of every ROI once per tile column it spans
  // (windows: the bound that came back with their number)
  const long long n_entries = (windows ? window_entries : items * 2 * p.PH * (p.S == 1 ? 1 : 2) * g.tx) +
                              11 * roialign::kTileRows * g.total;
  if (n_entries > (1ll << 27)) return false;
  // the consumer addresses both with 32-bit byte offsets
  if (b_slab >= (1ull << 31) || b_units >= (1ull << 31)) return false;
  plan->dyb_bytes = b_slab; plan->list_bytes = b_units;
  const size_t b_ranges = align_up(sizeof(roialign::WorkRange) * g.total * roialign::kTileRows, 256);
  const size_t b_entries = align_up(sizeof(roialign::WorkEntry) * n_entries, 256) + 512;
  char* base = static_cast<char*>(mobula_hip::workspace(b_offsets + b_recs + b_cnt + b_list + b_units + b_dyt +
                                                        b_ranges + b_entries + 256));
  if (failed()) return false;
  int* offsets = nullptr;
  if (windows) {
    if (base != head) number_windows(base);   // the workspace has grown: it is another buffer now
    offsets = reinterpret_cast<int*>(base);
    base += b_offsets;
  }
  plan->boxes = reinterpret_cast<roialign::TileBox*>(base);
  plan->cursors = reinterpret_cast<int*>(base + b_recs);
  plan->tile_rois = reinterpret_cast<int*>(base + b_recs + b_cnt);
  plan->lists = reinterpret_cast<roialign::AxisUnit*>(base + b_recs + b_cnt + b_list);
  char* cur = base + b_recs + b_cnt + b_list + b_units;
  plan->dyb = with_dyb ? reinterpret_cast<float*>(cur) : nullptr;
  cur += b_dyt;
  plan->ranges = reinterpret_cast<roialign::WorkRange*>(cur);
  cur += b_ranges;
  plan->entries = reinterpret_cast<roialign::WorkEntry*>(cur);
  cur += b_entries;
  // two kernels: per-item tables (which also resets the bump pointers), then per-tile lists
  const int n_items = static_cast<int>(items);
  const roialign::ListsArgs la{rois, n_items, p.R, p.scale, p.PH, p.PW, p.S, p.H, p.W, p.N, g, plan->layout,
                               plan->boxes, plan->cursors, plan->lists, offsets};
  const long long list_blocks = std::max(1ll, (items * 64 + 255) / 256);
  const DyLaunch dl = dy_launch<T>(p);
  if (fuse_dy != nullptr && with_dyb && dl.per > 0 && dl.blocks > 0 && dl.blocks + list_blocks < (1ll << 31)) {
    roialign::lists_and_dy_kernel<T><<<static_cast<unsigned>(dl.blocks + list_blocks), 256, dl.lds, stream>>>(
        la, static_cast<unsigned>(list_blocks), fuse_dy, plan->dyb, cblk, dl.per, p.C);
    plan->dy_transposed = true;
  } else {
    roialign::build_lists_kernel<<<static_cast<unsigned>(list_blocks), 256, 0, stream>>>(la);
  }
  (windows ? roialign::build_tile_work_kernel<true> : roialign::build_tile_work_kernel<false>)
      <<<static_cast<unsigned>(g.total), roialign::kTileRows * 64, 0, stream>>>(
          plan->boxes, n_items, plan->tile_rois, plan->lists, g, plan->layout, plan->cursors, plan->ranges,
          plan->entries);
  MOBULA_HIP_TRY(hipGetLastError());
  return !failed();
}

bool use_tiled() { return mobula_hip::option("roialign_impl", kAuto) != kNaive; }

// Tile columns of the backward pass: chosen from the size of the map unless the
// option "roialign_tile_columns" names one of the two widths (tests do).
int tile_columns(const Problem& p) {
  using BB = roialign::BwdBlocked;
  const long long forced = mobula_hip::option("roialign_tile_columns", 0);
  if (forced == BB::TW || forced == BB::TW_SMALL) return static_cast<int>(forced);
  return roialign::backward_tile_columns(p.N, p.H, p.W, (p.C + BB::CB - 1) / BB::CB);
}

// Wavefronts per tile row of the backward pass (1, or BwdBlocked::NSPLIT for maps with few tile
// rows); the option "roialign_row_split" names one of the two (tests do).
int row_split(const Problem& p) {
  using BB = roialign::BwdBlocked;
  const long long forced = mobula_hip::option("roialign_row_split", 0);
  if (forced == 1 || forced == BB::NSPLIT) return static_cast<int>(forced);
  return roialign::backward_row_split(p.N, p.H, p.W, (p.C + BB::CB - 1) / BB::CB);
}

// The tile owner for a problem: tile columns tw, nsplit wavefronts per tile row (lists of
// merged windows are not split), sample lists or windows.
template <bool NHWC, typename T>
auto owner_kernel(int tw, int* nsplit, bool windows) {
  using BB = roialign::BwdBlocked;
  const bool wide = tw == BB::TW;
  if (windows) {
    *nsplit = 1;
    return wide ? roialign::backward_blocked_kernel<NHWC, T, BB::TW, 1, true>
                : roialign::backward_blocked_kernel<NHWC, T, BB::TW_SMALL, 1, true>;
  }
  if (*nsplit > 1)
    return wide ? roialign::backward_blocked_kernel<NHWC, T, BB::TW, BB::NSPLIT, false>
                : roialign::backward_blocked_kernel<NHWC, T, BB::TW_SMALL, BB::NSPLIT, false>;
  return wide ? roialign::backward_blocked_kernel<NHWC, T, BB::TW, 1, false>
              : roialign::backward_blocked_kernel<NHWC, T, BB::TW_SMALL, 1, false>;
}

// Any sampling grid the lists take: fixed ones up to kSearchedGrid points, adaptive ones
// (whether an adaptive one is small enough to merge depends on the boxes; if not the call
// fails: this path has no other kernel to fall back on).
bool nhwc_backward_supported(const Problem& p) {
  return roialign::backward_blocked_supports(p.PH, p.PW, p.S) && p.S <= roialign::kSearchedGrid &&
         p.C % 4 == 0 &&
         static_cast<long long>(p.R) * p.PH * p.PW * p.C * 4 < (1ll << 31);
}

template <typename T>
void backward_device(const Problem& p, const T* dy, const float* rois, T* dx, bool assign,
                     hipStream_t stream) {
  if (p.N <= 0) return;
  using BB = roialign::BwdBlocked;
  constexpr bool kFp32 = std::is_same<T, float>::value;
  TilePlan plan;
  if (p.nhwc) {
    // dy and dx are used where they lie: only the pre-pass before the tile owners
    const int cblk = (p.C + BB::CB - 1) / BB::CB;
    const int tw = tile_columns(p);
    if (!nhwc_backward_supported(p) || reinterpret_cast<size_t>(dy) % 16 != 0 ||
        reinterpret_cast<size_t>(dx) % 16 != 0 ||
        !plan_tiles<T>(p, rois, roialign::kTileRows, tw, /*with_dyb=*/false, stream, &plan) ||
        roialign::backward_blocked_grid(plan.grid.total, cblk) >= (1ll << 31)) {
      if (!failed())
        set_error("roi_align_backward_nhwc: shape C=%d pooled %dx%d sampling_ratio %d (or the type or alignment "
                  "of the tensors) is not taken by the channels-last path", p.C, p.PH, p.PW, p.S);
      return;
    }
    const unsigned dy_bytes = static_cast<unsigned>(sizeof(T) * p.n_out);
    mobula_hip::KernelTimer timer("backward_blocked_kernel", stream);
    int nsplit = row_split(p);
    const auto kernel = owner_kernel<true, T>(tw, &nsplit, plan.layout.windows != 0);
    kernel<<<static_cast<unsigned>(roialign::backward_blocked_grid(plan.grid.total, cblk)), BB::NT * nsplit, 0, stream>>>(
        dy, dx, plan.ranges, plan.entries, plan.lists,
        plan.grid, plan.layout, p.C, p.H, p.W, p.PH, p.PW, cblk, dy_bytes,
        static_cast<unsigned>(plan.list_bytes), assign ? 1 : 0);
    MOBULA_HIP_TRY(hipGetLastError());
    return;
  }
  // the pre-pass (small, latency-bound kernels) runs beside the dy transposition, when that is
  // long enough to hide it: the transposition on the second stream, the pre-pass -- the longer of
  // the two beside a copy that saturates the memory -- on the caller's, so that the tile owners
  // follow it without waiting for a signal from another queue
  // (without a second stream the transposition shares the launch of the list builder instead)
  const bool forked = static_cast<long long>(sizeof(T)) * p.n_out >= kSideStreamBytes &&
                      mobula_hip::option("side_stream", 1) != 0;
  if (forked) {
    // the helper stream forks from the caller's: whatever the caller's stream has to wait for
    // before the workspace may be written (a previous call on another stream) must be in it
    // before the fork
    (void)mobula_hip::workspace(256);
    if (failed()) return;
  }
  mobula_hip::SideStream side(stream, forked);
  const int tw = tile_columns(p);
  if (use_tiled() && roialign::backward_blocked_supports(p.PH, p.PW, p.S) &&
      plan_tiles<T>(p, rois, roialign::kTileRows, tw, /*with_dyb=*/true, stream, &plan,
                    side.get() == stream ? dy : nullptr)) {
    const int cblk = (p.C + BB::CB - 1) / BB::CB;
    const long long grid = roialign::backward_blocked_grid(plan.grid.total, cblk);
    const DyLaunch dl = dy_launch<T>(p);
    if (grid < (1ll << 31) && dl.blocks < (1ll << 31) && (dl.per > 0 || dl.cap >= 4)) {
      if (p.R > 0 && !plan.dy_transposed)
        roialign::transpose_dy_blocked_kernel<T><<<static_cast<unsigned>(dl.blocks), 256, dl.lds, side.get()>>>(
            dy, plan.dyb, p.C, p.PH, p.PW, cblk, dl.per, p.R, dl.cap);
      side.join();
      {
        mobula_hip::KernelTimer timer("backward_blocked_kernel", stream);
        int nsplit = row_split(p);
        // every row piece of dx starts at a multiple of four elements (tile widths are): four columns per store
        const bool quads = p.W % 4 == 0 && reinterpret_cast<size_t>(dx) % (4 * sizeof(T)) == 0 &&
                           mobula_hip::option("roialign_row_quads", 1) != 0;
        const auto kernel = owner_kernel<false, T>(tw, &nsplit, plan.layout.windows != 0);
        kernel<<<static_cast<unsigned>(grid), BB::NT * nsplit, 0, stream>>>(
            plan.dyb, dx, plan.ranges, plan.entries, plan.lists, plan.grid, plan.layout, p.C, p.H,
            p.W, p.PH, p.PW, cblk, static_cast<unsigned>(plan.dyb_bytes),
            static_cast<unsigned>(plan.list_bytes), (assign ? 1 : 0) | (quads ? 2 : 0));
      }
      MOBULA_HIP_TRY(hipGetLastError());
      return;
    }
  }
  side.join();
  if (failed()) return;
  // straightforward kernel: float atomics into an fp32 map (the caller's, or for fp16 a scratch copy)
  const long long map = static_cast<long long>(p.N) * p.C * p.H * p.W;
  float* sums = reinterpret_cast<float*>(dx);
  if (!kFp32) {
    sums = static_cast<float*>(mobula_hip::workspace(sizeof(float) * map));
    if (failed()) return;
    if (!assign)
      roialign::widen_kernel<T><<<grid_for(map, 256), 256, 0, stream>>>(dx, sums, map);
  }
  if (assign)
    roialign::zero_words_kernel<<<grid_for(map, 256), 256, 0, stream>>>(reinterpret_cast<unsigned*>(sums), map);
  if (p.n_out > 0)
    roialign::backward_naive_kernel<T><<<grid_for(p.n_out, 256), 256, 0, stream>>>(
        p.n_out, dy, p.scale, p.C, p.H, p.W, p.PH, p.PW, p.S, sums, rois, p.N);
  if (!kFp32)
    roialign::narrow_kernel<T><<<grid_for(map, 256), 256, 0, stream>>>(sums, dx, map);
  MOBULA_HIP_TRY(hipGetLastError());
}

// binary64: the straightforward kernels only.
void forward_device(const Problem& p, const double* x, const double* rois, double* y, hipStream_t stream) {
  if (p.n_out == 0) return;
  roialign::roialign_f64_kernel<0><<<grid_for(p.n_out, 256), 256, 0, stream>>>(
      p.n_out, x, p.scale64, p.C, p.H, p.W, p.PH, p.PW, p.S, rois, y, p.N);
  MOBULA_HIP_TRY(hipGetLastError());
}

void backward_device(const Problem& p, const double* dy, const double* rois, double* dx, bool assign,
                     hipStream_t stream) {
  const long long map = static_cast<long long>(p.N) * p.C * p.H * p.W;
  if (assign && map > 0)
    roialign::zero_words_kernel<<<grid_for(2 * map, 256), 256, 0, stream>>>(reinterpret_cast<unsigned*>(dx), 2 * map);
  if (p.n_out > 0)
    roialign::roialign_f64_kernel<1><<<grid_for(p.n_out, 256), 256, 0, stream>>>(
        p.n_out, dy, p.scale64, p.C, p.H, p.W, p.PH, p.PW, p.S, rois, dx, p.N);
  MOBULA_HIP_TRY(hipGetLastError());
}

// Number of images a host ROI list implies: the largest batch index + 1.  Indices
// that cannot name an image of a map with 32-bit offsets (negative, not a number,
// beyond `limit`) are left out; the kernels skip such ROIs as well.
template <typename B>
long long host_images(const B* rois, int R, long long limit) {
  long long n = 0;
  for (int r = 0; r < R; ++r) {
    const B b = rois[5 * r];
    if (!(b >= static_cast<B>(0)) || !(b < static_cast<B>(limit))) continue;
    n = std::max<long long>(n, static_cast<long long>(b) + 1);
  }
  return n;
}

}  // namespace

// ---------------------------------------------------------------------------
// Launchers (scanned by the Python loader).
// ---------------------------------------------------------------------------

// T: element type of the map and of the pooled tensor; B: type of the boxes and of
// the scale.  The reference has one parameter for both (ROIAlign.cpp:9-16): its
// float and double instantiations are <float>, <double> here too (B defaults to
// T); binary16 maps come with binary32 boxes, <half, float>.
template <typename T, typename B = T>
MOBULA_KERNEL roi_align_forward_kernel(const int nthreads, const T* bottom_data,
                                       const B spatial_scale, const int channels,
                                       const int height, const int width,
                                       const int pooled_height, const int pooled_width,
                                       const int sampling_ratio, const B* bottom_rois,
                                       T* top_data) {
  Problem p;
  if (!describe(&p, "roi_align_forward", nthreads, static_cast<float>(spatial_scale), channels, height,
                width, pooled_height, pooled_width, sampling_ratio, 1, 9, 10, -1))
    return;
  p.scale64 = spatial_scale;
  hipStream_t stream = call_state().stream;
  if (p.N < 0) p.N = images_from_rois(bottom_rois, p.R, stream);
  if (failed()) return;
  forward_device(p, bottom_data, bottom_rois, top_data, stream);
}

template <typename T, typename B = T>
MOBULA_KERNEL roi_align_backward_kernel(const int nthreads, const T* top_diff,
                                        const B spatial_scale, const int channels,
                                        const int height, const int width,
                                        const int pooled_height, const int pooled_width,
                                        const int sampling_ratio, T* bottom_diff,
                                        const B* bottom_rois) {
  Problem p;
  if (!describe(&p, "roi_align_backward", nthreads, static_cast<float>(spatial_scale), channels, height,
                width, pooled_height, pooled_width, sampling_ratio, 9, 10, 1, -1))
    return;
  p.scale64 = spatial_scale;
  hipStream_t stream = call_state().stream;
  if (p.N < 0) p.N = images_from_rois(bottom_rois, p.R, stream);
  if (failed()) return;
  backward_device(p, top_diff, bottom_rois, bottom_diff, /*assign=*/false, stream);
}

// Not in the reference: backward that OVERWRITES bottom_diff (every element is
// written exactly once; elements no ROI touches become zero), i.e. the
// operator's "zero dx, then scatter" (opzoo/ROIAlign/ROIAlign.py:33-39) as one
// entry point.  num_images is the N of the [N,C,H,W] gradient.
template <typename T, typename B = T>
MOBULA_KERNEL roi_align_backward_assign_kernel(const int nthreads, const T* top_diff,
                                               const B spatial_scale, const int channels,
                                               const int height, const int width,
                                               const int pooled_height, const int pooled_width,
                                               const int sampling_ratio, const int num_images,
                                               T* bottom_diff, const B* bottom_rois) {
  Problem p;
  if (num_images < 0) {
    set_error("roi_align_backward_assign: num_images=%d", num_images);
    return;
  }
  if (!describe(&p, "roi_align_backward_assign", nthreads, static_cast<float>(spatial_scale), channels,
                height, width, pooled_height, pooled_width, sampling_ratio, 10, 11, 1, num_images))
    return;
  p.scale64 = spatial_scale;
  backward_device(p, top_diff, bottom_rois, bottom_diff, /*assign=*/true, call_state().stream);
}

// Not in the reference: the forward pass for callers that cannot allocate device
// memory (code under HIP graph capture, serving loops, harnesses that forbid
// it).  The channel-blocked copy of the map and the ROI order live in a fixed
// buffer of the library (kNoAllocScratchBytes per GPU, held until the process
// ends) instead of the thread's workspace: the call makes no allocation, no
// stream and no event.  num_images is the N of the [N,C,H,W] map.  Problems
// whose scratch need exceeds the buffer are an error.  All calls on one GPU
// share the buffer: calls that overlap in time on one GPU race.
template <typename T, typename B = T>
MOBULA_KERNEL roi_align_forward_noalloc_kernel(const int nthreads, const T* bottom_data,
                                               const B spatial_scale, const int channels,
                                               const int height, const int width,
                                               const int pooled_height, const int pooled_width,
                                               const int sampling_ratio, const int num_images,
                                               const B* bottom_rois, T* top_data) {
  Problem p;
  if (num_images < 0) {
    set_error("roi_align_forward_noalloc: num_images=%d", num_images);
    return;
  }
  if (!describe(&p, "roi_align_forward_noalloc", nthreads, static_cast<float>(spatial_scale), channels, height,
                width, pooled_height, pooled_width, sampling_ratio, 1, 10, 11, num_images))
    return;
  p.scale64 = spatial_scale;
  p.fixed_scratch = noalloc_scratch(&p.fixed_scratch_bytes);
  if (failed()) return;
  forward_device(p, bottom_data, bottom_rois, top_data, call_state().stream);
}

// Not in the reference: the same three operations on channels-last tensors, the
// map as [N,H,W,C] and the pooled tensor as [R,PH,PW,C] (what a torch tensor in
// torch.channels_last format holds).  The kernels read and write these where
// they lie, so the copies into the blocked layouts are not made.  Shapes the
// fast kernels do not take are an error here (see
// mobula_hip_roialign_nhwc_supported); device memory only.
template <typename T>
MOBULA_KERNEL roi_align_forward_nhwc_kernel(const int nthreads, const T* bottom_data,
                                            const float spatial_scale, const int channels,
                                            const int height, const int width,
                                            const int pooled_height, const int pooled_width,
                                            const int sampling_ratio, const float* bottom_rois,
                                            T* top_data) {
  Problem p;
  if (!describe(&p, "roi_align_forward_nhwc", nthreads, spatial_scale, channels, height, width,
                pooled_height, pooled_width, sampling_ratio, 1, 9, 10, -1))
    return;
  p.nhwc = true;
  hipStream_t stream = call_state().stream;
  if (p.N < 0) p.N = images_from_rois(bottom_rois, p.R, stream);
  if (failed()) return;
  forward_device<T>(p, bottom_data, bottom_rois, top_data, stream);
}

template <typename T>
MOBULA_KERNEL roi_align_backward_nhwc_kernel(const int nthreads, const T* top_diff,
                                             const float spatial_scale, const int channels,
                                             const int height, const int width,
                                             const int pooled_height, const int pooled_width,
                                             const int sampling_ratio, T* bottom_diff,
                                             const float* bottom_rois) {
  Problem p;
  if (!describe(&p, "roi_align_backward_nhwc", nthreads, spatial_scale, channels, height, width,
                pooled_height, pooled_width, sampling_ratio, 9, 10, 1, -1))
    return;
  p.nhwc = true;
  hipStream_t stream = call_state().stream;
  if (p.N < 0) p.N = images_from_rois(bottom_rois, p.R, stream);
  if (failed()) return;
  backward_device(p, top_diff, bottom_rois, bottom_diff, /*assign=*/false, stream);
}

template <typename T>
MOBULA_KERNEL roi_align_backward_nhwc_assign_kernel(const int nthreads, const T* top_diff,
                                                    const float spatial_scale, const int channels,
                                                    const int height, const int width,
                                                    const int pooled_height, const int pooled_width,
                                                    const int sampling_ratio, const int num_images,
                                                    T* bottom_diff, const float* bottom_rois) {
  Problem p;
  if (num_images < 0) {
    set_error("roi_align_backward_nhwc_assign: num_images=%d", num_images);
    return;
  }
  if (!describe(&p, "roi_align_backward_nhwc_assign", nthreads, spatial_scale, channels, height, width,
                pooled_height, pooled_width, sampling_ratio, 10, 11, 1, num_images))
    return;
  p.nhwc = true;
  backward_device(p, top_diff, bottom_rois, bottom_diff, /*assign=*/true, call_state().stream);
}

// ---------------------------------------------------------------------------
// Entry-point plumbing: device selection, staging of host buffers (device id
// -1), completion.
// ---------------------------------------------------------------------------
namespace {

int staging_device() { return static_cast<int>(mobula_hip::option("host_staging_device", 0)); }

template <typename T, typename B>
void forward_entry(int device_id, int nthreads, const T* x, B scale, int C, int H, int W,
                   int PH, int PW, int S, const B* rois, T* y) {
  mobula_hip::begin_call();
  if (device_id >= 0) {
    mobula_hip::DeviceScope scope(device_id);
    if (scope.ok()) roi_align_forward_kernel<T, B>(nthreads, x, scale, C, H, W, PH, PW, S, rois, y);
    mobula_hip::finish_call();
    return;
  }
  // Host memory: mirror the buffers on the staging device.
  mobula_hip::DeviceScope scope(staging_device());
  auto& st = call_state();
  const hipStream_t saved_stream = st.stream;
  st.stream = nullptr;
  Problem p;
  if (scope.ok() && describe(&p, "roi_align_forward", nthreads, static_cast<float>(scale), C, H, W, PH,
                             PW, S, 1, 9, 10, -1)) {
    if (p.N < 0) p.N = host_images(rois, p.R, (1ll << 31) / (static_cast<long long>(C) * H * W));
    st.extents.assign(11, -1);
    st.extents[1] = p.N * C * H * W;
    mobula_hip::HostStaging stage;
    const T* dx = static_cast<const T*>(stage.in(x, sizeof(T) * p.N * C * H * W));
    const B* dr = static_cast<const B*>(stage.in(rois, sizeof(B) * 5 * p.R));
    T* dy = static_cast<T*>(stage.inout(y, sizeof(T) * p.n_out, /*upload=*/false));
    if (!failed()) roi_align_forward_kernel<T, B>(nthreads, dx, scale, C, H, W, PH, PW, S, dr, dy);
    if (!failed()) stage.flush(nullptr);
    mobula_hip::finish_call();   // (on the staging device, before the caller's stream comes back)
  }
  st.stream = saved_stream;
  st.extents.clear();
}

template <typename T, typename B>
void backward_entry(int device_id, int nthreads, const T* dy, B scale, int C, int H, int W,
                    int PH, int PW, int S, int num_images, T* dx, const B* rois) {
  mobula_hip::begin_call();
  const bool assign = num_images >= 0;
  if (device_id >= 0) {
    mobula_hip::DeviceScope scope(device_id);
    if (scope.ok()) {
      if (assign)
        roi_align_backward_assign_kernel<T, B>(nthreads, dy, scale, C, H, W, PH, PW, S, num_images,
                                               dx, rois);
      else
        roi_align_backward_kernel<T, B>(nthreads, dy, scale, C, H, W, PH, PW, S, dx, rois);
    }
    mobula_hip::finish_call();
    return;
  }
  mobula_hip::DeviceScope scope(staging_device());
  auto& st = call_state();
  const hipStream_t saved_stream = st.stream;
  st.stream = nullptr;
  Problem p;
  const int e_map = assign ? 10 : 9, e_rois = assign ? 11 : 10;
  if (scope.ok() && describe(&p, "roi_align_backward", nthreads, static_cast<float>(scale), C, H, W, PH,
                             PW, S, e_map, e_rois, 1, assign ? num_images : -1)) {
    if (p.N < 0) p.N = host_images(rois, p.R, (1ll << 31) / (static_cast<long long>(C) * H * W));
    mobula_hip::HostStaging stage;
    const T* ddy = static_cast<const T*>(stage.in(dy, sizeof(T) * p.n_out));
    const B* dr = static_cast<const B*>(stage.in(rois, sizeof(B) * 5 * p.R));
    T* ddx = static_cast<T*>(stage.inout(dx, sizeof(T) * p.N * C * H * W, /*upload=*/!assign));
    st.extents.assign(12, -1);
    st.extents[e_map] = p.N * C * H * W;
    if (!failed()) {
      if (assign)
        roi_align_backward_assign_kernel<T, B>(nthreads, ddy, scale, C, H, W, PH, PW, S,
                                               static_cast<int>(p.N), ddx, dr);
      else
        roi_align_backward_kernel<T, B>(nthreads, ddy, scale, C, H, W, PH, PW, S, ddx, dr);
    }
    if (!failed()) stage.flush(nullptr);
    mobula_hip::finish_call();
  }
  st.stream = saved_stream;
  st.extents.clear();
}

}  // namespace

extern "C" {

// float instantiations: the symbols the reference binding resolves.
void roi_align_forward_ab78de3c(const int device_id, const int nthreads, const float* bottom_data,
                                const float spatial_scale, const int channels, const int height,
                                const int width, const int pooled_height, const int pooled_width,
                                const int sampling_ratio, const float* bottom_rois,
                                float* top_data) {
  forward_entry<float, float>(device_id, nthreads, bottom_data, spatial_scale, channels, height, width,
                       pooled_height, pooled_width, sampling_ratio, bottom_rois, top_data);
}

void roi_align_backward_f318a24e(const int device_id, const int nthreads, const float* top_diff,
                                 const float spatial_scale, const int channels, const int height,
                                 const int width, const int pooled_height, const int pooled_width,
                                 const int sampling_ratio, float* bottom_diff,
                                 const float* bottom_rois) {
  backward_entry<float, float>(device_id, nthreads, top_diff, spatial_scale, channels, height, width,
                        pooled_height, pooled_width, sampling_ratio, -1, bottom_diff, bottom_rois);
}

// double instantiations.  The reference builds the forward only (its atomic_add
// takes float); the two backward symbols follow its naming scheme.
void roi_align_forward_6b9e6c9b(const int device_id, const int nthreads, const double* bottom_data,
                                const double spatial_scale, const int channels, const int height,
                                const int width, const int pooled_height, const int pooled_width,
                                const int sampling_ratio, const double* bottom_rois,
                                double* top_data) {
  forward_entry<double, double>(device_id, nthreads, bottom_data, spatial_scale, channels, height, width,
                                pooled_height, pooled_width, sampling_ratio, bottom_rois, top_data);
}

void roi_align_backward_2b6c6dfa(const int device_id, const int nthreads, const double* top_diff,
                                 const double spatial_scale, const int channels, const int height,
                                 const int width, const int pooled_height, const int pooled_width,
                                 const int sampling_ratio, double* bottom_diff,
                                 const double* bottom_rois) {
  backward_entry<double, double>(device_id, nthreads, top_diff, spatial_scale, channels, height, width,
                                 pooled_height, pooled_width, sampling_ratio, -1, bottom_diff, bottom_rois);
}

void roi_align_backward_assign_4620f85e(const int device_id, const int nthreads, const double* top_diff,
                                        const double spatial_scale, const int channels, const int height,
                                        const int width, const int pooled_height, const int pooled_width,
                                        const int sampling_ratio, const int num_images,
                                        double* bottom_diff, const double* bottom_rois) {
  mobula_hip::begin_call();
  if (num_images < 0) {
    set_error("roi_align_backward_assign: num_images=%d", num_images);
    mobula_hip::finish_call();
    return;
  }
  backward_entry<double, double>(device_id, nthreads, top_diff, spatial_scale, channels, height, width,
                                 pooled_height, pooled_width, sampling_ratio, num_images, bottom_diff,
                                 bottom_rois);
}

// Extensions (no counterpart in the reference); names follow the same scheme.
void roi_align_backward_assign_a8793cbe(const int device_id, const int nthreads,
                                        const float* top_diff, const float spatial_scale,
                                        const int channels, const int height, const int width,
                                        const int pooled_height, const int pooled_width,
                                        const int sampling_ratio, const int num_images,
                                        float* bottom_diff, const float* bottom_rois) {
  mobula_hip::begin_call();
  if (num_images < 0) {
    set_error("roi_align_backward_assign: num_images=%d", num_images);
    mobula_hip::finish_call();
    return;
  }
  backward_entry<float, float>(device_id, nthreads, top_diff, spatial_scale, channels, height, width,
                        pooled_height, pooled_width, sampling_ratio, num_images, bottom_diff,
                        bottom_rois);
}

// The forward pass that allocates nothing (see roi_align_forward_noalloc_kernel); device memory only.
void roi_align_forward_noalloc_83212f20(const int device_id, const int nthreads, const float* bottom_data,
                                        const float spatial_scale, const int channels, const int height,
                                        const int width, const int pooled_height, const int pooled_width,
                                        const int sampling_ratio, const int num_images,
                                        const float* bottom_rois, float* top_data) {
  mobula_hip::begin_call();
  if (device_id < 0) {
    set_error("roi_align_forward_noalloc takes device memory only");
    mobula_hip::finish_call();
    return;
  }
  mobula_hip::DeviceScope scope(device_id);
  if (scope.ok())
    roi_align_forward_noalloc_kernel<float, float>(nthreads, bottom_data, spatial_scale, channels, height, width,
                                                   pooled_height, pooled_width, sampling_ratio, num_images,
                                                   bottom_rois, top_data);
  mobula_hip::finish_call();
}

// Sets up the fixed buffer of roi_align_forward_noalloc on `device_id` ahead of
// the first call there (the first call does it otherwise); returns its size in
// bytes, or -1 with the error text set.
long long mobula_hip_roialign_noalloc_init(const int device_id) {
  mobula_hip::begin_call();
  mobula_hip::DeviceScope scope(device_id);
  size_t bytes = 0;
  if (!scope.ok() || noalloc_scratch(&bytes) == nullptr) return -1;
  return static_cast<long long>(bytes);
}

// Backward with binary16 top_diff / bottom_diff (sums in fp32, rounded once).
void roi_align_backward_23175303(const int device_id, const int nthreads, const __half* top_diff,
                                 const float spatial_scale, const int channels, const int height,
                                 const int width, const int pooled_height, const int pooled_width,
                                 const int sampling_ratio, __half* bottom_diff, const float* bottom_rois) {
  backward_entry<__half, float>(device_id, nthreads, top_diff, spatial_scale, channels, height, width,
                         pooled_height, pooled_width, sampling_ratio, -1, bottom_diff, bottom_rois);
}

void roi_align_backward_assign_7924dbc8(const int device_id, const int nthreads, const __half* top_diff,
                                        const float spatial_scale, const int channels, const int height,
                                        const int width, const int pooled_height, const int pooled_width,
                                        const int sampling_ratio, const int num_images,
                                        __half* bottom_diff, const float* bottom_rois) {
  mobula_hip::begin_call();
  if (num_images < 0) {
    set_error("roi_align_backward_assign: num_images=%d", num_images);
    mobula_hip::finish_call();
    return;
  }
  backward_entry<__half, float>(device_id, nthreads, top_diff, spatial_scale, channels, height, width,
                         pooled_height, pooled_width, sampling_ratio, num_images, bottom_diff, bottom_rois);
}

// The same three with bfloat16 storage.
void roi_align_forward_f951d439(const int device_id, const int nthreads, const roialign::bfloat16* bottom_data,
                                const float spatial_scale, const int channels, const int height,
                                const int width, const int pooled_height, const int pooled_width,
                                const int sampling_ratio, const float* bottom_rois,
                                roialign::bfloat16* top_data) {
  forward_entry<roialign::bfloat16, float>(device_id, nthreads, bottom_data, spatial_scale, channels, height,
                                           width, pooled_height, pooled_width, sampling_ratio, bottom_rois,
                                           top_data);
}

void roi_align_backward_0c43e974(const int device_id, const int nthreads, const roialign::bfloat16* top_diff,
                                 const float spatial_scale, const int channels, const int height,
                                 const int width, const int pooled_height, const int pooled_width,
                                 const int sampling_ratio, roialign::bfloat16* bottom_diff,
                                 const float* bottom_rois) {
  backward_entry<roialign::bfloat16, float>(device_id, nthreads, top_diff, spatial_scale, channels, height,
                                            width, pooled_height, pooled_width, sampling_ratio, -1, bottom_diff,
                                            bottom_rois);
}

void roi_align_backward_assign_86156afd(const int device_id, const int nthreads,
                                        const roialign::bfloat16* top_diff, const float spatial_scale,
                                        const int channels, const int height, const int width,
                                        const int pooled_height, const int pooled_width,
                                        const int sampling_ratio, const int num_images,
                                        roialign::bfloat16* bottom_diff, const float* bottom_rois) {
  mobula_hip::begin_call();
  if (num_images < 0) {
    set_error("roi_align_backward_assign: num_images=%d", num_images);
    mobula_hip::finish_call();
    return;
  }
  backward_entry<roialign::bfloat16, float>(device_id, nthreads, top_diff, spatial_scale, channels, height,
                                            width, pooled_height, pooled_width, sampling_ratio, num_images,
                                            bottom_diff, bottom_rois);
}

// Channels-last variants (extensions): device pointers only.
#define MOBULA_NHWC_ENTRY(call)                                                            \
  mobula_hip::begin_call();                                                                \
  if (device_id < 0) {                                                                     \
    set_error("the channels-last entry points take device memory only");                   \
    mobula_hip::finish_call();                                                             \
    return;                                                                                \
  }                                                                                        \
  {                                                                                        \
    mobula_hip::DeviceScope scope(device_id);                                              \
    if (scope.ok()) call;                                                                  \
    mobula_hip::finish_call();                                                             \
  }

void roi_align_forward_nhwc_ab78de3c(const int device_id, const int nthreads, const float* bottom_data,
                                     const float spatial_scale, const int channels, const int height,
                                     const int width, const int pooled_height, const int pooled_width,
                                     const int sampling_ratio, const float* bottom_rois, float* top_data) {
  MOBULA_NHWC_ENTRY(roi_align_forward_nhwc_kernel<float>(nthreads, bottom_data, spatial_scale, channels, height,
                                                         width, pooled_height, pooled_width, sampling_ratio,
                                                         bottom_rois, top_data))
}

void roi_align_forward_nhwc_e874c59a(const int device_id, const int nthreads, const __half* bottom_data,
                                     const float spatial_scale, const int channels, const int height,
                                     const int width, const int pooled_height, const int pooled_width,
                                     const int sampling_ratio, const float* bottom_rois, __half* top_data) {
  MOBULA_NHWC_ENTRY(roi_align_forward_nhwc_kernel<__half>(nthreads, bottom_data, spatial_scale, channels, height,
                                                          width, pooled_height, pooled_width, sampling_ratio,
                                                          bottom_rois, top_data))
}

void roi_align_forward_nhwc_f951d439(const int device_id, const int nthreads,
                                     const roialign::bfloat16* bottom_data, const float spatial_scale,
                                     const int channels, const int height, const int width,
                                     const int pooled_height, const int pooled_width, const int sampling_ratio,
                                     const float* bottom_rois, roialign::bfloat16* top_data) {
  MOBULA_NHWC_ENTRY(roi_align_forward_nhwc_kernel<roialign::bfloat16>(nthreads, bottom_data, spatial_scale,
                                                                      channels, height, width, pooled_height,
                                                                      pooled_width, sampling_ratio, bottom_rois,
                                                                      top_data))
}

void roi_align_backward_nhwc_f318a24e(const int device_id, const int nthreads, const float* top_diff,
                                      const float spatial_scale, const int channels, const int height,
                                      const int width, const int pooled_height, const int pooled_width,
                                      const int sampling_ratio, float* bottom_diff, const float* bottom_rois) {
  MOBULA_NHWC_ENTRY(roi_align_backward_nhwc_kernel<float>(nthreads, top_diff, spatial_scale, channels, height,
                                                          width, pooled_height, pooled_width, sampling_ratio,
                                                          bottom_diff, bottom_rois))
}

#define MOBULA_NHWC_BACKWARD_16(suffix, assign_suffix, type)                                                   \
  void roi_align_backward_nhwc_##suffix(const int device_id, const int nthreads, const type* top_diff,         \
                                        const float spatial_scale, const int channels, const int height,      \
                                        const int width, const int pooled_height, const int pooled_width,     \
                                        const int sampling_ratio, type* bottom_diff, const float* bottom_rois) { \
    MOBULA_NHWC_ENTRY(roi_align_backward_nhwc_kernel<type>(nthreads, top_diff, spatial_scale, channels, height, \
                                                           width, pooled_height, pooled_width, sampling_ratio, \
                                                           bottom_diff, bottom_rois))                          \
  }                                                                                                            \
  void roi_align_backward_nhwc_assign_##assign_suffix(                                                         \
      const int device_id, const int nthreads, const type* top_diff, const float spatial_scale,                \
      const int channels, const int height, const int width, const int pooled_height, const int pooled_width,  \
      const int sampling_ratio, const int num_images, type* bottom_diff, const float* bottom_rois) {           \
    MOBULA_NHWC_ENTRY(roi_align_backward_nhwc_assign_kernel<type>(nthreads, top_diff, spatial_scale, channels, \
                                                                  height, width, pooled_height, pooled_width,  \
                                                                  sampling_ratio, num_images, bottom_diff,     \
                                                                  bottom_rois))                                \
  }
MOBULA_NHWC_BACKWARD_16(23175303, 7924dbc8, __half)
MOBULA_NHWC_BACKWARD_16(0c43e974, 86156afd, roialign::bfloat16)
#undef MOBULA_NHWC_BACKWARD_16

void roi_align_backward_nhwc_assign_a8793cbe(const int device_id, const int nthreads, const float* top_diff,
                                             const float spatial_scale, const int channels, const int height,
                                             const int width, const int pooled_height, const int pooled_width,
                                             const int sampling_ratio, const int num_images, float* bottom_diff,
                                             const float* bottom_rois) {
  MOBULA_NHWC_ENTRY(roi_align_backward_nhwc_assign_kernel<float>(nthreads, top_diff, spatial_scale, channels,
                                                                 height, width, pooled_height, pooled_width,
                                                                 sampling_ratio, num_images, bottom_diff,
                                                                 bottom_rois))
}
#undef MOBULA_NHWC_ENTRY

// 1 if the channels-last entry points take the shape, else 0.  backward != 0 asks
// about the backward entry points, elem_bytes is 4 (fp32) or 2 (fp16, bfloat16).
int mobula_hip_roialign_nhwc_supported(int backward, int elem_bytes, int channels, int height, int width,
                                       int pooled_height, int pooled_width, int sampling_ratio,
                                       long long num_rois) {
  if (channels <= 0 || height <= 0 || width <= 0 || pooled_height <= 0 || pooled_width <= 0 || num_rois < 0 ||
      num_rois > (1ll << 30))
    return 0;
  Problem p;
  p.R = static_cast<int>(num_rois); p.C = channels; p.H = height; p.W = width;
  p.PH = pooled_height; p.PW = pooled_width; p.S = sampling_ratio;
  if (backward) return (elem_bytes == 4 || elem_bytes == 2) && nhwc_backward_supported(p) ? 1 : 0;
  if (elem_bytes == 4) return nhwc_forward_supported<float>(p) ? 1 : 0;
  if (elem_bytes == 2) return nhwc_forward_supported<__half>(p) ? 1 : 0;
  return 0;
}

void roi_align_forward_e874c59a(const int device_id, const int nthreads, const __half* bottom_data,
                                const float spatial_scale, const int channels, const int height,
                                const int width, const int pooled_height, const int pooled_width,
                                const int sampling_ratio, const float* bottom_rois,
                                __half* top_data) {
  forward_entry<__half, float>(device_id, nthreads, bottom_data, spatial_scale, channels, height, width,
                        pooled_height, pooled_width, sampling_ratio, bottom_rois, top_data);
}

}  // extern "C"

static mobula_hip::ExportRegistrar roialign_exports(
    "roi_align_forward_ab78de3c roi_align_backward_f318a24e roi_align_backward_assign_a8793cbe "
    "roi_align_forward_6b9e6c9b roi_align_backward_2b6c6dfa roi_align_backward_assign_4620f85e "
    "roi_align_forward_e874c59a roi_align_backward_23175303 roi_align_backward_assign_7924dbc8 "
    "roi_align_forward_f951d439 roi_align_backward_0c43e974 roi_align_backward_assign_86156afd "
    "roi_align_forward_nhwc_ab78de3c roi_align_forward_nhwc_e874c59a roi_align_forward_nhwc_f951d439 "
    "roi_align_backward_nhwc_f318a24e roi_align_backward_nhwc_assign_a8793cbe "
    "roi_align_backward_nhwc_23175303 roi_align_backward_nhwc_assign_7924dbc8 "
    "roi_align_backward_nhwc_0c43e974 roi_align_backward_nhwc_assign_86156afd "
    "mobula_hip_roialign_nhwc_supported roi_align_forward_noalloc_83212f20 mobula_hip_roialign_noalloc_init");
