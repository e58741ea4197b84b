// Backward ROIAlign: tile owners accumulate in LDS, 16 bytes per lane.
//
// dx is cut into tiles of 16 rows x 56 columns x 32 channels (28 columns for maps
// that would give the SIMDs too few wavefronts otherwise), and a tile into
// bands of TH rows (TH = 1: single rows).  One workgroup owns one band, keeps
// it in LDS as acc[row][column][channel] and is the only writer of that piece
// of dx: no atomics anywhere and a summation order fixed by the ROI order.
// Wavefront w owns row w of the band, so wavefronts never touch the same cell
// and need no barrier.  Nothing but the launch ties the wavefronts of a
// workgroup together, so small bands (many workgroups resident per CU) keep a
// CU busy when the rows of a tile have work lists of different length.
// The 64 lanes of a wavefront
// are 8 pooled columns x 8 channel quads: a lane folds the row taps of a ROI
// into four gradients (its pooled column, its four channels) and adds them to
// the two cells of each of its column samples with 16-byte LDS accesses.
// Pooled columns whose cells may coincide (the pre-pass stores the spacing at
// which they cannot) are not added in the same instruction: the two columns of
// a pair of lane groups are taken one after the other by both groups, one group
// adding the low corners and the other the high ones -- an LDS instruction
// costs the same with eight active lanes as with 64, so nobody sits out.
// Sampling grids of more than two points per bin come as windows of merged
// weights instead (WIN): up to seven consecutive cells per pooled column.
//
// dy is read from a channel-blocked copy dyb[C/32][R][PH][PW][32]: one 16-byte
// load per lane fetches (eight pooled columns of) a pooled row, up to 1 KB; the
// slab of a channel block is addressed with 32-bit offsets (up to 2 GiB each).
#pragma once
#include <type_traits>

#include "roialign_taps.hip.h"

namespace roialign {

struct BwdBlocked {
  static constexpr int TH = 1;           // rows of a band = wavefronts of a workgroup
  static constexpr int BANDS = kTileRows / TH;   // bands per tile
  static constexpr int TW = 56;          // tile columns ...
  static constexpr int TW_SMALL = 28;    // ... and for maps that give few tiles (see backward_tile_columns)
  static constexpr int CB = 32;          // channels per workgroup
  static constexpr int NW = TH;
  static constexpr int NT = NW * 64;
  // floats per cell: the 32 channels, no padding.  (Measured: 36 spreads the banks of the
  // write-out but costs a tenth of the wavefronts a CU holds: 222 instead of 216 us at
  // 4x256x200x336 with 4000 ROIs; 40 is slower still.)
  static constexpr int CS = 32;
  static constexpr int G = 4;            // work entries per pipeline stage
  static constexpr int PWB = 8;          // pooled columns per turn (one per group of 8 lanes)
  static constexpr int NSPLIT = 4;       // wavefronts that share a tile row of a map with few tile rows
};

inline bool backward_blocked_supports(int PH, int PW, int S) { return lists_supported(PH, PW, S); }

// Tile width for a map: narrow tiles double the number of (shorter) work lists,
// which pays only while the wide ones would leave the SIMDs short of wavefronts
// (measured: 2048 wavefronts 82 -> 65 us, 40000 wavefronts 222 -> 262 us).
inline int backward_tile_columns(long long images, int H, int W, int cblk) {
  const long long wide = images * ((H + kTileRows - 1) / kTileRows) * ((W + BwdBlocked::TW - 1) / BwdBlocked::TW);
  return wide * kTileRows * cblk < 8192 ? BwdBlocked::TW_SMALL : BwdBlocked::TW;
}

// Wavefronts per tile row: the same maps also split every row's work list.
inline int backward_row_split(long long images, int H, int W, int cblk) {
  const long long wide = images * ((H + kTileRows - 1) / kTileRows) * ((W + BwdBlocked::TW - 1) / BwdBlocked::TW);
  return wide * kTileRows * cblk < 8192 ? BwdBlocked::NSPLIT : 1;
}

// dy[r][c][ph][pw] -> dyb[cb][r][ph][pw][32] (R: number of ROIs), zero where the channel does
// not exist.  One workgroup per (ROI, group of `per` channel blocks): the input words of the
// group are contiguous and so are the output words of each of its blocks.
// LDS holds the input as it is; the transposition happens in the reads.
// T is the element type of dy (float or __half); dyb is fp32 either way.
// `block`: index among the workgroups (of 256 threads) that transpose.
// `cap`: channels LDS holds at a time.  With per >= 1 whole blocks fit (cap is not used);
// per == 0 says that not even one block does (large pooled sizes): the workgroup then takes one
// channel block in passes of `cap` channels (a multiple of 4).
template <typename T>
__device__ __forceinline__ void transpose_dy_blocked_body(unsigned block, const T* __restrict__ dy,
                                                          float* __restrict__ dyb, int C, int PH, int PW,
                                                          int cblk, int per, int R, int cap) {
  constexpr int CB = BwdBlocked::CB;
  constexpr int VEC = 16 / sizeof(T);   // elements per 16-byte word
  extern __shared__ __attribute__((aligned(16))) unsigned char tbuf_bytes[];   // [channels][PH * PW] of T
  T* const tbuf = reinterpret_cast<T*>(tbuf_bytes);
  const int blocks_per_group = per > 0 ? per : 1;
  const int groups = (cblk + blocks_per_group - 1) / blocks_per_group;
  const int r = block / groups, grp = block % groups;
  const int cb0 = grp * blocks_per_group, nblk = min(blocks_per_group, cblk - cb0);
  const int c0 = cb0 * CB, nch = min(nblk * CB, C - c0);
  const int bins = PH * PW;
  const int pass_ch = per > 0 ? nch : cap;
  typedef float f32x4s __attribute__((ext_vector_type(4)));
  for (int pc = 0; pc < nch; pc += pass_ch) {
    const int pn = min(pass_ch, nch - pc);
    const T* src = dy + (static_cast<size_t>(r) * C + c0 + pc) * bins;
    const int n_in = pn * bins;
    if (pc > 0) __syncthreads();   // the previous pass has been read
    if ((reinterpret_cast<size_t>(src) & 15) == 0) {
      const int nvec = n_in / VEC;
      typedef float f32x4 __attribute__((ext_vector_type(4)));
      for (int i = threadIdx.x; i < nvec; i += 256)   // dy is read once: no need to keep it in the caches
        reinterpret_cast<f32x4*>(tbuf)[i] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(src) + i);
      for (int i = VEC * nvec + threadIdx.x; i < n_in; i += 256) tbuf[i] = src[i];
    } else {
      for (int i = threadIdx.x; i < n_in; i += 256) tbuf[i] = src[i];
    }
    __syncthreads();
    const int per_blk = bins * (CB / 4);   // 16-byte pieces of one channel block
    if (per > 0) {
      for (int blk = 0; blk < nblk; ++blk) {
        // every channel block has a slab of its own (all ROIs): its owners address it with 32-bit offsets
        float* const dst = dyb + (static_cast<size_t>(cb0 + blk) * R + r) * bins * CB;
        for (int p = threadIdx.x; p < per_blk; p += 256) {
          const int cq = p & 7, cell = p >> 3, c = blk * CB + 4 * cq;   // channel quad, bin, first channel
          const T* in = tbuf + c * bins + cell;
          float4 v = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
          if (c + 0 < nch) v.x = to_float(in[0]);
          if (c + 1 < nch) v.y = to_float(in[bins]);
          if (c + 2 < nch) v.z = to_float(in[2 * bins]);
          if (c + 3 < nch) v.w = to_float(in[3 * bins]);
          __builtin_nontemporal_store(f32x4s{v.x, v.y, v.z, v.w}, reinterpret_cast<f32x4s*>(dst + static_cast<size_t>(p) * 4));
        }
      }
    } else {
      // the channel quads pc / 4 .. of the one block: 16-byte pieces, the quads of a cell side by side;
      // the last pass also writes the zero quads of channels that do not exist
      float* const dst = dyb + (static_cast<size_t>(cb0) * R + r) * bins * CB;
      const int q0 = pc / 4, nq = pc + pass_ch >= nch ? CB / 4 - q0 : pn / 4;
      for (int q = threadIdx.x; q < nq * bins; q += 256) {
        const int cell = q / nq, qi = q - cell * nq, c = 4 * qi;   // bin, channel quad and first channel within the pass
        const T* in = tbuf + c * bins + cell;
        float4 v = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        if (c + 0 < pn) v.x = to_float(in[0]);
        if (c + 1 < pn) v.y = to_float(in[bins]);
        if (c + 2 < pn) v.z = to_float(in[2 * bins]);
        if (c + 3 < pn) v.w = to_float(in[3 * bins]);
        __builtin_nontemporal_store(f32x4s{v.x, v.y, v.z, v.w},
                                    reinterpret_cast<f32x4s*>(dst + (static_cast<size_t>(cell) * 8 + q0 + qi) * 4));
      }
    }
  }
}

template <typename T>
__global__ void __launch_bounds__(256)
transpose_dy_blocked_kernel(const T* __restrict__ dy, float* __restrict__ dyb, int C, int PH,
                            int PW, int cblk, int per, int R, int cap) {
  transpose_dy_blocked_body<T>(blockIdx.x, dy, dyb, C, PH, PW, cblk, per, R, cap);
}

// Both in one launch, for inputs too small to be worth a second stream: the
// first list_blocks workgroups build the lists (few, and each a chain of
// dependent steps: they start first), the others transpose dy.  The two do not
// depend on each other; small kernels one after the other cost more in
// dependencies than in work.  Dynamic LDS as for transpose_dy_blocked_kernel.
template <typename T>
__global__ void __launch_bounds__(256)
lists_and_dy_kernel(ListsArgs lists, unsigned list_blocks, const T* __restrict__ dy, float* __restrict__ dyb,
                    int cblk, int per, int C) {
  if (blockIdx.x < list_blocks) {
    if (lists.window_offsets != nullptr) build_window_lists_body(blockIdx.x, lists);
    else build_lists_body(blockIdx.x, lists);
  }
  else
    transpose_dy_blocked_body<T>(blockIdx.x - list_blocks, dy, dyb, C, lists.PH, lists.PW, cblk, per, lists.R, 0);
}

// Number of workgroups for `tiles` tiles and cblk channel blocks (job decode at
// the top of backward_blocked_kernel).
inline long long backward_blocked_grid(long long tiles, int cblk) {
  tiles *= BwdBlocked::BANDS;   // one workgroup per band
  long long per_xcd;
  if (cblk >= 8) per_xcd = tiles * ((cblk + 7) / 8);
  else per_xcd = (tiles + (8 / cblk) - 1) / (8 / cblk);
  return 8 * per_xcd;
}

typedef int int16v __attribute__((ext_vector_type(16)));

// Element i (0..3) of the four consecutive values a lane loaded: four dwords of
// fp32, or two dwords holding four 16-bit values.
template <typename TI>
__device__ __forceinline__ float lane_value(const unsigned __attribute__((ext_vector_type(4)))& d, int i) {
  if constexpr (sizeof(TI) == 4) {
    return __uint_as_float(d[i]);
  } else {
    const unsigned short bits = static_cast<unsigned short>(d[i >> 1] >> (16 * (i & 1)));
    return to_float(__builtin_bit_cast(TI, bits));
  }
}

// TO is the element type of dx (float, __half or bfloat16; sums are formed in fp32 and
// rounded once).  TW: tile columns.  NSPLIT: wavefronts that share a tile row: each takes
// a contiguous part of the row's work list (whole items: an item belongs to the part its first
// entry lies in) into a row of its own in LDS, and the parts are added in part order on the
// way out -- for maps that give the SIMDs too few tile rows to keep them busy.
// WIN: the list items are windows of merged column weights (sampling grids of more than two
// points per bin and axis) instead of pairs of sample columns.
// dy_any: the blocked fp32 copy dyb, or for channels-last tensors the caller's
// dy[R][PH][PW][C] itself, of dx's element type.
template <bool NHWC, typename TO, int TW, int NSPLIT = 1, bool WIN = false>
__global__ void __launch_bounds__(BwdBlocked::NT * NSPLIT)
backward_blocked_kernel(const void* __restrict__ dy_any, TO* __restrict__ dx_any,
                        const WorkRange* __restrict__ ranges, const WorkEntry* __restrict__ entries,
                        const AxisUnit* __restrict__ lists, TileGrid tg, ListLayout ll, int C, int H,
                        int W, int PH, int PW, int cblk, unsigned dyb_bytes, unsigned list_bytes,
                        int assign) {   // assign: bit 0 = overwrite dx (else add to it), bit 1 = rows may be written four columns at a time
  using K = BwdBlocked;
  constexpr int RS = TW + 2;   // cells per row: one dummy on either side
  static_assert(K::TH == 1, "the parts of a split row take the place of the rows of a band");
  static_assert(TW % 4 == 0, "tiles start at multiples of four columns (the four-column write-out)");
  __shared__ __attribute__((aligned(16))) float acc[NSPLIT * RS * K::CS];

  // Job decode.  Workgroups are dealt to the 8 XCDs round-robin, so blockIdx % 8
  // names the XCD: it takes the channel blocks b with b % 8 == xcd (their slice
  // of dyb then stays in that XCD's L2) and walks the bands of the tiles in order; with
  // fewer than 8 blocks the tiles of a block are split into 8 / cblk ranges.
  const int xcd = blockIdx.x & 7;
  const long long wi = blockIdx.x >> 3;
  long long tile;
  int cb;
  if (cblk >= 8) {
    const int nx = (cblk - xcd + 7) >> 3;
    tile = wi / nx;
    cb = xcd + 8 * static_cast<int>(wi % nx);
  } else {
    const int parts = 8 / cblk;
    cb = xcd % cblk;
    const int part = xcd / cblk;
    const long long range = (tg.total * K::BANDS + parts - 1) / parts;
    if (part >= parts || wi >= range) return;
    tile = part * range + wi;
  }
  if (tile >= tg.total * K::BANDS) return;
  const int band = static_cast<int>(tile % K::BANDS);
  tile /= K::BANDS;
  const int n = static_cast<int>(tile / tg.per_image);
  const int t_in_img = static_cast<int>(tile % tg.per_image);
  const int ty = t_in_img / tg.tx, tx = t_in_img % tg.tx;
  const int r0 = ty * kTileRows + band * K::TH, q0 = tx * TW;
  const int c0 = cb * K::CB, nch = min(K::CB, C - c0);
  const int lane = threadIdx.x & 63;
  const int part = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // which part of the row's work list
  constexpr int wave = 0;                                               // the tile row owned within the band
  const int cols = min(TW, W - q0);
  if (r0 + wave >= H) return;   // (a band below the map: the same for every wavefront of the workgroup)
  const int grp = lane >> 3, quad = lane & 7;   // pooled column within a turn, channel quad

  float* const row = acc + part * (RS * K::CS);
  for (int i = lane; i < RS * K::CS / 4; i += 64)
    reinterpret_cast<float4*>(row)[i] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);

  const WorkRange wr = ranges[tile * kTileRows + band * K::TH + wave];
  const int n_entries = wr.count;   // a multiple of 2 * G, and G more entries follow: the lists are padded
  const int16v* const wl = reinterpret_cast<const int16v*>(entries + wr.begin);
  // this part's share: the items that start in [first_entry, end_entry), whole groups of 2 * G entries
  const int rounds = n_entries / (2 * K::G);
  const int first_entry = NSPLIT == 1 ? 0 : part * rounds / NSPLIT * (2 * K::G);
  const int end_entry = NSPLIT == 1 ? n_entries : (part + 1) * rounds / NSPLIT * (2 * K::G);
  float* const cell0 = row + quad * 4;   // this lane's four channels of cell 0 (the left dummy)

  // dyb and the sample lists as raw buffers: a scalar byte offset per entry
  // plus a fixed lane offset
  typedef typename std::conditional<NHWC, TO, float>::type TI;   // element type of what dy_any points to
  constexpr unsigned E = sizeof(TI);
  const unsigned dy_pw = (NHWC ? C : K::CB) * E;
  const unsigned dy_ph = static_cast<unsigned>(PW) * dy_pw;
  const unsigned dy_roi = dy_ph * PH;
  const unsigned list_roi = static_cast<unsigned>(ll.roi_stride) * sizeof(AxisUnit);
  // (dyb_bytes: the bytes of one channel block's slab of dyb, or of the caller's whole dy)
  const __amdgpu_buffer_rsrc_t dy_buf = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<char*>(static_cast<const char*>(dy_any)) + (NHWC ? 0 : static_cast<size_t>(cb) * dyb_bytes), 0,
      static_cast<int>(dyb_bytes), 0x00020000);
  const __amdgpu_buffer_rsrc_t list_buf = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<AxisUnit*>(lists), 0, static_cast<int>(list_bytes), 0x00020000);
  typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
  typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
  // what a lane holds of an item's column list: one dword of a ColPair, or two of a ColWindow
  typedef typename std::conditional<WIN, u32x2, unsigned>::type UT;

  // Each wavefront streams through the work list of its tile row: entries
  // (ROI, pooled row, weight) in ROI order, four at a time, double buffered:
  // while the taps of one group are folded and added, the dy rows and column
  // samples of the next are in flight (always eight loads per group, so the
  // wait before a group counts exactly the loads of the group after it).
  for (int pwb = 0; pwb < PW; pwb += K::PWB) {
    const unsigned dy_fixed = (NHWC ? cb * K::CB * E : 0u) + pwb * dy_pw;
    const unsigned list_fixed = static_cast<unsigned>(
        (static_cast<long long>(ll.ty) * ll.row_stride + static_cast<long long>(tx) * ll.col_stride +
         pwb * (WIN ? 2 : 1)) * sizeof(AxisUnit));
    // a lane whose pooled column or channels do not exist loads from outside the buffer (zero, no access)
    const int dy_lane = pwb + grp < PW && quad * 4 < nch ? static_cast<int>(grp * dy_pw + quad * 4 * E)
                                                         : static_cast<int>(0x80000000u);
    // The 16-byte column sample of the lane's pooled column comes as one dword per
    // lane (lane & 3 picks it; a 4-byte load costs the texture path half of a
    // 16-byte one) and is spread over the quad with DPP moves where it is used.
    // (The 32-byte window of merged weights: two dwords per lane.)
    const int list_lane = WIN ? grp * 32 + (lane & 3) * 8 : grp * 16 + (lane & 3) * 4;
    auto issue = [&](const int16v& e, u32x4 (&d)[K::G], UT (&u)[K::G]) {
#pragma unroll
      for (int j = 0; j < K::G; ++j) {
        // the item's lists, the dy of the ROI it belongs to
        const unsigned roi = e[4 * j], ph = e[4 * j + 1], owner = static_cast<unsigned>(e[4 * j + 3]) >> 2;
        if (E == 4) {
          d[j] = __builtin_amdgcn_raw_buffer_load_b128(dy_buf, dy_lane, owner * dy_roi + ph * dy_ph + dy_fixed, 0);
        } else {   // four 16-bit values: eight bytes
          const u32x2 w = __builtin_amdgcn_raw_buffer_load_b64(dy_buf, dy_lane, owner * dy_roi + ph * dy_ph + dy_fixed, 0);
          d[j] = u32x4{w.x, w.y, 0u, 0u};
        }
        if constexpr (WIN)
          u[j] = __builtin_amdgcn_raw_buffer_load_b64(list_buf, list_lane, roi * list_roi + list_fixed, 0);
        else
          u[j] = __builtin_amdgcn_raw_buffer_load_b32(list_buf, list_lane, roi * list_roi + list_fixed, 0);
      }
    };
    float g[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    // adds g * (weights of the two cells) to the cells pos, pos + 1 of the row
    auto add_sample = [&](int pos, float wlo, float whi) {
      float* const a = cell0 + pos * K::CS;
      float4 lo = *reinterpret_cast<const float4*>(a);
      float4 hi = *reinterpret_cast<const float4*>(a + K::CS);
      lo.x = fmaf(g[0], wlo, lo.x); lo.y = fmaf(g[1], wlo, lo.y);
      lo.z = fmaf(g[2], wlo, lo.z); lo.w = fmaf(g[3], wlo, lo.w);
      hi.x = fmaf(g[0], whi, hi.x); hi.y = fmaf(g[1], whi, hi.y);
      hi.z = fmaf(g[2], whi, hi.z); hi.w = fmaf(g[3], whi, hi.w);
      *reinterpret_cast<float4*>(a) = lo;
      *reinterpret_cast<float4*>(a + K::CS) = hi;
    };
    bool mine = NSPLIT == 1, done = false;   // (uniform) inside an item of this part; past the part's last item
    // adds g * w[i] to the cells a, a + 1, ... of the row (N of them; all reads before the first write)
    auto add_cells = [&](float* a, const float* w, auto count) {
      constexpr int N = decltype(count)::value;
      float4 v[N];
#pragma unroll
      for (int i = 0; i < N; ++i) v[i] = *reinterpret_cast<const float4*>(a + i * K::CS);
#pragma unroll
      for (int i = 0; i < N; ++i) {
        v[i].x = fmaf(g[0], w[i], v[i].x); v[i].y = fmaf(g[1], w[i], v[i].y);
        v[i].z = fmaf(g[2], w[i], v[i].z); v[i].w = fmaf(g[3], w[i], v[i].w);
      }
#pragma unroll
      for (int i = 0; i < N; ++i) *reinterpret_cast<float4*>(a + i * K::CS) = v[i];
    };
    auto process = [&](const int16v& e, const u32x4 (&d)[K::G], const UT (&u)[K::G], int at) {
#pragma unroll
      for (int j = 0; j < K::G; ++j) {
        const float wy = __int_as_float(e[4 * j + 2]);
        const int fl = e[4 * j + 3];
        if (NSPLIT > 1) {
          if ((fl & 1) == 0) {   // an item starts here: this part's if it starts before the part's end
            mine = at + j < end_entry;
            done = !mine;
          }
          if (!mine) continue;
        }
        if ((fl & 1) != 0) {   // (the same for the whole wavefront)
#pragma unroll
          for (int i = 0; i < 4; ++i) g[i] = fmaf(lane_value<TI>(d[j], i), wy, g[i]);
        } else {               // first tap of an item: the sum starts afresh, whatever the last one held
#pragma unroll
          for (int i = 0; i < 4; ++i) g[i] = lane_value<TI>(d[j], i) * wy;
        }
        if constexpr (WIN) {
          if ((fl & 2) != 0) {
            // last tap of this item on this row: g times the weights of the window's cells.
            // The lanes lane & 3 = k of a quad hold dwords 2k and 2k + 1 of the window:
            // quad_perm [k, k, k, k] hands them to everyone
            const int ulo = static_cast<int>(u[j][0]), uhi = static_cast<int>(u[j][1]);
            const int header = __builtin_amdgcn_mov_dpp(ulo, 0x00, 0xf, 0xf, true);
            const float w[kWindowCells] = {
                __int_as_float(__builtin_amdgcn_mov_dpp(uhi, 0x00, 0xf, 0xf, true)),
                __int_as_float(__builtin_amdgcn_mov_dpp(ulo, 0x55, 0xf, 0xf, true)),
                __int_as_float(__builtin_amdgcn_mov_dpp(uhi, 0x55, 0xf, 0xf, true)),
                __int_as_float(__builtin_amdgcn_mov_dpp(ulo, 0xaa, 0xf, 0xf, true)),
                __int_as_float(__builtin_amdgcn_mov_dpp(uhi, 0xaa, 0xf, 0xf, true)),
                __int_as_float(__builtin_amdgcn_mov_dpp(ulo, 0xff, 0xf, 0xf, true)),
                __int_as_float(__builtin_amdgcn_mov_dpp(uhi, 0xff, 0xf, 0xf, true))};
            float* const a = cell0 + (header & 0xffff) * K::CS;
            const int turns = 1 << ((__builtin_amdgcn_readfirstlane(header) >> 16) & 3);
            // (the eight lanes of a pooled column decide alike: a window that ends early costs the LDS nothing)
            auto add_window = [&] {
              if (w[0] != 0.0f || w[1] != 0.0f || w[2] != 0.0f || w[3] != 0.0f)
                add_cells(a, w, std::integral_constant<int, 4>());
              if (w[4] != 0.0f || w[5] != 0.0f || w[6] != 0.0f)
                add_cells(a + 4 * K::CS, w + 4, std::integral_constant<int, 3>());
            };
            if (turns == 1) {
              add_window();
            } else {
              // Neighbouring windows overlap.  An LDS instruction costs the same with few lanes as
              // with all, so the two windows of a pair of lane groups (a row of 16 lanes) are taken
              // one after the other by both groups together: one group adds the even cells, the
              // other the odd ones (the gradient and the window of the other group: its lanes,
              // eight further).
              const int which = grp & 1, pair = grp >> 1, rounds = turns >> 1;
              const int ulo_x = __builtin_amdgcn_mov_dpp(ulo, 0x128, 0xf, 0xf, true);   // row_ror:8
              const int uhi_x = __builtin_amdgcn_mov_dpp(uhi, 0x128, 0xf, 0xf, true);
              float gx[4];
#pragma unroll
              for (int i = 0; i < 4; ++i)
                gx[i] = __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(g[i]), 0x128, 0xf, 0xf, true));
#pragma unroll
              for (int t = 0; t < 2; ++t) {   // the pair's first window, then its second
                const bool own = which == t;
                const int vlo = own ? ulo : ulo_x, vhi = own ? uhi : uhi_x;
                const float gg[4] = {own ? g[0] : gx[0], own ? g[1] : gx[1], own ? g[2] : gx[2], own ? g[3] : gx[3]};
                const int hd = __builtin_amdgcn_mov_dpp(vlo, 0x00, 0xf, 0xf, true);
                const float x0 = __int_as_float(__builtin_amdgcn_mov_dpp(vhi, 0x00, 0xf, 0xf, true));
                const float x1 = __int_as_float(__builtin_amdgcn_mov_dpp(vlo, 0x55, 0xf, 0xf, true));
                const float x2 = __int_as_float(__builtin_amdgcn_mov_dpp(vhi, 0x55, 0xf, 0xf, true));
                const float x3 = __int_as_float(__builtin_amdgcn_mov_dpp(vlo, 0xaa, 0xf, 0xf, true));
                const float x4 = __int_as_float(__builtin_amdgcn_mov_dpp(vhi, 0xaa, 0xf, 0xf, true));
                const float x5 = __int_as_float(__builtin_amdgcn_mov_dpp(vlo, 0xff, 0xf, 0xf, true));
                const float x6 = __int_as_float(__builtin_amdgcn_mov_dpp(vhi, 0xff, 0xf, 0xf, true));
                const bool head = x0 != 0.0f || x1 != 0.0f || x2 != 0.0f || x3 != 0.0f;
                const bool tail = x4 != 0.0f || x5 != 0.0f || x6 != 0.0f;
                // this lane's cells: which, which + 2 of w[0..3]; 4 + which (and 6) of w[4..6]
                float* const b = cell0 + ((hd & 0xffff) + which) * K::CS;
                const float wa = which ? x1 : x0, wb = which ? x3 : x2, wc = which ? x5 : x4;
                auto fold = [&](float4& v, float w) {
                  v.x = fmaf(gg[0], w, v.x); v.y = fmaf(gg[1], w, v.y);
                  v.z = fmaf(gg[2], w, v.z); v.w = fmaf(gg[3], w, v.w);
                };
                for (int r = 0; r < rounds; ++r)
                  if ((pair & (rounds - 1)) == r) {
                    if (head) {
                      float4 va = *reinterpret_cast<const float4*>(b);
                      float4 vb = *reinterpret_cast<const float4*>(b + 2 * K::CS);
                      fold(va, wa); fold(vb, wb);
                      *reinterpret_cast<float4*>(b) = va;
                      *reinterpret_cast<float4*>(b + 2 * K::CS) = vb;
                    }
                    if (tail) {
                      float4 vc = *reinterpret_cast<const float4*>(b + 4 * K::CS);
                      float4 vd = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
                      if (which == 0) vd = *reinterpret_cast<const float4*>(b + 6 * K::CS);
                      fold(vc, wc); fold(vd, x6);
                      *reinterpret_cast<float4*>(b + 4 * K::CS) = vc;
                      if (which == 0) *reinterpret_cast<float4*>(b + 6 * K::CS) = vd;
                    }
                  }
              }
            }
          }
        } else if ((fl & 2) != 0) {
          // last tap of this ROI on this row: spread g over the column samples
          // dword k of the quad's four: quad_perm [k, k, k, k]
          const int uj = static_cast<int>(u[j]);
          const unsigned cells = static_cast<unsigned>(__builtin_amdgcn_mov_dpp(uj, 0x00, 0xf, 0xf, true));
          const int cf = __builtin_amdgcn_mov_dpp(uj, 0x55, 0xf, 0xf, true);
          const int pos0 = cells & 0xffff, pos1 = cells >> 16;
          const float l0 = __int_as_float(__builtin_amdgcn_mov_dpp(uj, 0xaa, 0xf, 0xf, true));
          const float l1 = __int_as_float(__builtin_amdgcn_mov_dpp(uj, 0xff, 0xf, 0xf, true));
          const int turns = 1 << ((__builtin_amdgcn_readfirstlane(cf) >> kColStrideShift) & kColStrideMask);
          // A sample with a corner in the tile adds to both its cells: a corner
          // outside the tile has its cell among the dummies, one of weight zero adds zero.
          auto add_both = [&] {
            if ((cf & 3) != 0) add_sample(pos0, 1.0f - l0, l0);
            if ((cf & 12) != 0) add_sample(pos1, 1.0f - l1, l1);
          };
          if (turns == 1) {
            add_both();
          } else {
            // Neighbouring pooled columns may share cells.  An LDS instruction costs the same with
            // few lanes as with all, so instead of letting every second column wait, the two
            // columns of a pair of lane groups (a row of 16 lanes) are taken one after the other
            // by both groups together: one group adds the low corners, the other the high ones
            // (the gradient and the column pair of the other group: its lanes, eight further).
            const int which = grp & 1, pair = grp >> 1, rounds = turns >> 1;
            const int uj_x = __builtin_amdgcn_mov_dpp(uj, 0x128, 0xf, 0xf, true);   // row_ror:8
            float gx[4];
#pragma unroll
            for (int i = 0; i < 4; ++i)
              gx[i] = __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(g[i]), 0x128, 0xf, 0xf, true));
#pragma unroll
            for (int t = 0; t < 2; ++t) {   // the pair's first column, then its second
              const bool own = which == t;
              const int uu = own ? uj : uj_x;
              const float gg[4] = {own ? g[0] : gx[0], own ? g[1] : gx[1], own ? g[2] : gx[2], own ? g[3] : gx[3]};
              const unsigned pc = static_cast<unsigned>(__builtin_amdgcn_mov_dpp(uu, 0x00, 0xf, 0xf, true));
              const int pf = __builtin_amdgcn_mov_dpp(uu, 0x55, 0xf, 0xf, true);
              const float m0 = __int_as_float(__builtin_amdgcn_mov_dpp(uu, 0xaa, 0xf, 0xf, true));
              const float m1 = __int_as_float(__builtin_amdgcn_mov_dpp(uu, 0xff, 0xf, 0xf, true));
              // this lane's corner of the two samples: its cell, its weight, whether it counts
              float* const a0 = cell0 + ((pc & 0xffff) + which) * K::CS;
              float* const a1 = cell0 + ((pc >> 16) + which) * K::CS;
              float w0 = which ? m0 : 1.0f - m0;
              const float w1 = which ? m1 : 1.0f - m1;
              const bool live0 = ((pf >> which) & 1) != 0;
              bool live1 = ((pf >> (2 + which)) & 1) != 0;
              // samples in one pixel pair (bins well under a pixel): one update of the cell for both
              // (only where the first sample's update is there anyway: the columns that share an
              // instruction are spaced so that their first samples touch different cells, and so
              // that their second samples do -- not first against second)
              if (live0 && live1 && a0 == a1) {
                w0 += w1;
                live1 = false;
              }
              auto add_corner = [&](float* a, float w) {
                float4 v = *reinterpret_cast<const float4*>(a);
                v.x = fmaf(gg[0], w, v.x); v.y = fmaf(gg[1], w, v.y);
                v.z = fmaf(gg[2], w, v.z); v.w = fmaf(gg[3], w, v.w);
                *reinterpret_cast<float4*>(a) = v;
              };
              for (int r = 0; r < rounds; ++r)
                if ((pair & (rounds - 1)) == r) {
                  if (live0) add_corner(a0, w0);
                  if (live1) add_corner(a1, w1);
                }
            }
          }
        }
      }
    };

    if (first_entry < end_entry) {
      const int w0 = first_entry >> 2;
      int16v e_cur = wl[w0], e_nx = wl[w0 + 1], e_n2;
      u32x4 d_a[K::G], d_b[K::G];
      UT u_a[K::G], u_b[K::G];
      issue(e_cur, d_a, u_a);
      // (a part goes on past its end until the item it is in has ended: to the next item start)
      for (int e0 = first_entry; e0 < n_entries && !done; e0 += 2 * K::G) {
        // group at e0 lives in set a, group at e0 + G in set b
        e_n2 = wl[(e0 >> 2) + 2];
        issue(e_nx, d_b, u_b);
        process(e_cur, d_a, u_a, e0);
        e_cur = e_nx; e_nx = e_n2;
        e_n2 = wl[(e0 >> 2) + 3];
        issue(e_nx, d_a, u_a);   // past the end this is the padding: loaded, never used
        process(e_cur, d_b, u_b, e0 + K::G);
        e_cur = e_nx; e_nx = e_n2;
      }
    }
  }

  if (NSPLIT > 1) __syncthreads();   // every part of the row is complete
  // element i of a cell, the parts added in part order
  auto total4 = [&](int cell) {
    float4 v = *reinterpret_cast<const float4*>(acc + cell * K::CS + quad * 4);
#pragma unroll
    for (int k = 1; k < NSPLIT; ++k) {
      const float4 w = *reinterpret_cast<const float4*>(acc + k * (RS * K::CS) + cell * K::CS + quad * 4);
      v.x += w.x; v.y += w.y; v.z += w.z; v.w += w.w;
    }
    return v;
  };
  if (NHWC) {
    // dx[n][row][col][C]: a pixel's channels of this block are contiguous;
    // eight pixels per step, a lane moves its four channels
    struct alignas(4 * sizeof(TO)) Four { TO v[4]; };
    TO* const px0 = dx_any + ((static_cast<size_t>(n) * H + r0 + wave) * W + q0) * C + c0 + quad * 4;
    if (quad * 4 < nch) {
      for (int col = grp + 8 * part; col < cols; col += 8 * NSPLIT) {
        const float4 v = total4(col + 1);
        Four* const dst = reinterpret_cast<Four*>(px0 + static_cast<size_t>(col) * C);
        Four o;
        if ((assign & 1) != 0) {
          o.v[0] = from_float<TO>(v.x); o.v[1] = from_float<TO>(v.y);
          o.v[2] = from_float<TO>(v.z); o.v[3] = from_float<TO>(v.w);
        } else {
          o = *dst;
          o.v[0] = from_float<TO>(to_float(o.v[0]) + v.x); o.v[1] = from_float<TO>(to_float(o.v[1]) + v.y);
          o.v[2] = from_float<TO>(to_float(o.v[2]) + v.z); o.v[3] = from_float<TO>(to_float(o.v[3]) + v.w);
        }
        *dst = o;
      }
    }
    return;
  }
  // The owner writes its row.
  TO* const out = dx_any + ((static_cast<size_t>(n) * C + c0) * H + r0 + wave) * W + q0;
  const size_t plane = static_cast<size_t>(H) * W;
  if ((assign & 2) != 0) {
    // Rows whose pieces start at multiples of four elements (the host says so): a lane reads its
    // channel quad of four neighbouring cells -- the eight lanes of a group cover all the
    // banks, as in the accumulation -- and writes four columns of each of its four planes at
    // once.  (Read with lanes along x instead, the cells lie 32 words apart: one bank.)
    struct alignas(4 * sizeof(TO)) Four { TO v[4]; };
    if (quad * 4 < nch) {
      for (int base = 4 * grp + 32 * part; base < cols; base += 32 * NSPLIT) {
        float4 v[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = total4(base + j + 1);
        const float t[4][4] = {{v[0].x, v[1].x, v[2].x, v[3].x}, {v[0].y, v[1].y, v[2].y, v[3].y},
                               {v[0].z, v[1].z, v[2].z, v[3].z}, {v[0].w, v[1].w, v[2].w, v[3].w}};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (quad * 4 + i >= nch) break;
          Four* const dst = reinterpret_cast<Four*>(out + (quad * 4 + i) * plane + base);
          Four o;
          if ((assign & 1) != 0) {
#pragma unroll
            for (int j = 0; j < 4; ++j) o.v[j] = from_float<TO>(t[i][j]);
          } else {
            o = *dst;
#pragma unroll
            for (int j = 0; j < 4; ++j) o.v[j] = from_float<TO>(to_float(o.v[j]) + t[i][j]);
          }
          *dst = o;
        }
      }
    }
    return;
  }
  // Any other row: one channel plane at a time, lanes along x.
  // LPC lanes per channel plane (a power of two that covers the tile's columns):
  // 64 / LPC planes are written per step
  constexpr int LPC = TW <= 32 ? 32 : 64, PLANES = 64 / LPC;
  const int col = lane & (LPC - 1), first = lane / LPC;
  if (col < cols) {
    const float* const src = acc + (col + 1) * K::CS;
    auto total = [&](int c) {
      float v = src[c];
#pragma unroll
      for (int k = 1; k < NSPLIT; ++k) v += src[k * (RS * K::CS) + c];
      return v;
    };
    if ((assign & 1) != 0) {
      for (int c = first + PLANES * part; c < nch; c += PLANES * NSPLIT) out[c * plane + col] = from_float<TO>(total(c));
    } else {
      for (int c = first + PLANES * part; c < nch; c += PLANES * NSPLIT)
        out[c * plane + col] = from_float<TO>(to_float(out[c * plane + col]) + total(c));
    }
  }
}

}  // namespace roialign
