// Tiled ROIAlign backward: every (tile, channel block) of dx is owned by one
// workgroup, accumulated in LDS and written to memory exactly once -- no global
// atomics and no separate zero-fill pass.
//
// LDS layout: acc[c][1 + row*33 + col], channel stride odd, so the 64 lanes of
// a wavefront (one channel each) always hit 64 different banks; weights and
// pixel positions are the same for all lanes.  Column 32 of row r and column
// -1 of row r+1 are one shared dummy cell, which lets every column unit be a
// two-cell read-modify-write even at the tile border.
// LDS float atomics are not used (they run at a few lanes per clock on this
// part): each of the eight compute wavefronts owns two tile rows instead.
//
// Pipeline per ROI of the tile's list: a ninth wavefront lists the sample
// units of the next ROI while the compute wavefronts work on the current one.
// The dy blocks [roi, c0:c0+64, ph_a:ph_b, :] (contiguous in memory) of the
// next DEPTH iterations are in flight in registers -- one workgroup per CU
// cannot hide a memory round trip any other way -- and each is dropped into
// LDS between two barriers when its turn comes.  The geometry records of the
// tile's ROIs are copied to LDS up front, 128 at a time.
//
// The inner loops are bound by vector-ALU issue, so everything uniform stays
// off the vector ALU: units are fetched with broadcast LDS reads, loop control
// and ownership tests run on scalar registers, no integer division per ROI.
//
// Arithmetic per cell: dx += (dy * (wy / count)) * wx, against the reference's
// (dy * (wy*wx)) / count (opzoo/ROIAlign/ROIAlign.cpp:143-157): same samples
// and weights, rounding differs in the last bits.
#pragma once
#include "roialign_taps.hip.h"

namespace roialign {

struct BwdTile {
  static constexpr int TH = 16, TW = 32, CH = 64;
  static constexpr int NWC = 8;                  // compute wavefronts
  static constexpr int NTC = NWC * 64;           // compute threads
  static constexpr int NT = NTC + 64;            // + one producer wavefront
  static constexpr int ROWS_PER_WAVE = TH / NWC;
  static constexpr int RS = TW + 1;              // row stride (one dummy cell per row)
  static constexpr int CS = TH * RS + 1;         // channel stride, odd
  static constexpr int DYS = 63;                 // channel stride of the staged dy, odd
  static constexpr int RU_CAP = 64, CU_CAP = 128;  // axis units per (tile, ROI): rows, columns
  static constexpr int DEPTH = 4;                // dy blocks in flight per thread
  static constexpr int REC_CHUNK = 128;          // ROI records held in LDS at a time
  static constexpr int STAGE_ITERS = (CH * DYS + NTC - 1) / NTC;
  static constexpr int MAX_PW = 32, MAX_PH = 64;
  static_assert(CS % 2 == 1 && ROWS_PER_WAVE == 2, "layout");
};

// Host-side gate: can the tiled backward kernel take this problem?  The unit
// lists of one (tile, ROI) pair must fit their LDS arrays for any box.  With a
// fixed grid all PH*S sample rows may fall into one tile; with the adaptive
// grid samples are more than half a pixel apart (or there is one per pooled
// row), so a tile sees at most 2*(T+2) + PH of them.
inline bool backward_tiled_supports(int PH, int PW, int S) {
  using K = BwdTile;
  if (PW > K::MAX_PW || PH > K::MAX_PH) return false;
  const long long rows = S > 0 ? static_cast<long long>(PH) * S : 2 * (K::TH + 2) + PH;
  const long long cols = S > 0 ? static_cast<long long>(PW) * S : 2 * (K::TW + 2) + PW;
  return rows <= K::RU_CAP && cols <= K::CU_CAP;
}

// Bit 16 of AxisUnit::bin of a column unit: its cells overlap those of the
// NEXT unit in the list (set by the producer).
constexpr int kOverlapsNext = 1 << 16;

// Adds one row tap (NR == 1) or one tap for each of two different tile rows
// (NR == 2) to the accumulator rows ra / rb: for every column unit u,
//   row[u.pos] += dy[u.bin]*wy*u.w0,  row[u.pos+1] += dy[u.bin]*wy*u.w1.
// Units are taken two at a time; when their cells are disjoint all loads are
// issued before the stores, otherwise unit after unit (LDS accesses of one
// wavefront complete in program order).  `units` is the same address in every
// lane, so the unit fetches are broadcast reads and their fields are uniform.
template <int NR>
__device__ __forceinline__ void scatter_rows(float* ra, float* rb, const float* dy_a,
                                             const float* dy_b, float wy_a, float wy_b,
                                             const AxisUnit* units, int n_units) {
  int k = 0;
  for (; k + 1 < n_units; k += 2) {
    const AxisUnit u0 = units[k], u1 = units[k + 1];
    const int pw0 = u0.bin & 0xffff, pw1 = u1.bin & 0xffff;
    const float ga0 = dy_a[pw0] * wy_a, ga1 = dy_a[pw1] * wy_a;
    float gb0 = 0.0f, gb1 = 0.0f;
    if (NR == 2) { gb0 = dy_b[pw0] * wy_b; gb1 = dy_b[pw1] * wy_b; }
    float* const pa0 = ra + u0.pos;
    float* const pa1 = ra + u1.pos;
    float* const pb0 = rb + u0.pos;
    float* const pb1 = rb + u1.pos;
    if ((__builtin_amdgcn_readfirstlane(u0.bin) & kOverlapsNext) == 0) {
      const float xa0 = pa0[0], ya0 = pa0[1], xa1 = pa1[0], ya1 = pa1[1];
      float xb0 = 0.0f, yb0 = 0.0f, xb1 = 0.0f, yb1 = 0.0f;
      if (NR == 2) { xb0 = pb0[0]; yb0 = pb0[1]; xb1 = pb1[0]; yb1 = pb1[1]; }
      pa0[0] = fmaf(ga0, u0.w0, xa0); pa0[1] = fmaf(ga0, u0.w1, ya0);
      pa1[0] = fmaf(ga1, u1.w0, xa1); pa1[1] = fmaf(ga1, u1.w1, ya1);
      if (NR == 2) {
        pb0[0] = fmaf(gb0, u0.w0, xb0); pb0[1] = fmaf(gb0, u0.w1, yb0);
        pb1[0] = fmaf(gb1, u1.w0, xb1); pb1[1] = fmaf(gb1, u1.w1, yb1);
      }
    } else {
      const float xa0 = pa0[0], ya0 = pa0[1];
      float xb0 = 0.0f, yb0 = 0.0f;
      if (NR == 2) { xb0 = pb0[0]; yb0 = pb0[1]; }
      pa0[0] = fmaf(ga0, u0.w0, xa0); pa0[1] = fmaf(ga0, u0.w1, ya0);
      if (NR == 2) { pb0[0] = fmaf(gb0, u0.w0, xb0); pb0[1] = fmaf(gb0, u0.w1, yb0); }
      const float xa1 = pa1[0], ya1 = pa1[1];
      float xb1 = 0.0f, yb1 = 0.0f;
      if (NR == 2) { xb1 = pb1[0]; yb1 = pb1[1]; }
      pa1[0] = fmaf(ga1, u1.w0, xa1); pa1[1] = fmaf(ga1, u1.w1, ya1);
      if (NR == 2) { pb1[0] = fmaf(gb1, u1.w0, xb1); pb1[1] = fmaf(gb1, u1.w1, yb1); }
    }
  }
  if (k < n_units) {
    const AxisUnit u0 = units[k];
    const int pw0 = u0.bin & 0xffff;
    const float ga0 = dy_a[pw0] * wy_a;
    float* const pa0 = ra + u0.pos;
    const float xa0 = pa0[0], ya0 = pa0[1];
    pa0[0] = fmaf(ga0, u0.w0, xa0); pa0[1] = fmaf(ga0, u0.w1, ya0);
    if (NR == 2) {
      const float gb0 = dy_b[pw0] * wy_b;
      float* const pb0 = rb + u0.pos;
      const float xb0 = pb0[0], yb0 = pb0[1];
      pb0[0] = fmaf(gb0, u0.w0, xb0); pb0[1] = fmaf(gb0, u0.w1, yb0);
    }
  }
}

struct alignas(16) BwdHeader { int n_ru; int n_cu; float inv_count; int pad; };

__global__ void __launch_bounds__(BwdTile::NT)
backward_tiled_kernel(const float* __restrict__ dy, float* __restrict__ dx,
                      const RoiRec* __restrict__ recs, const int* __restrict__ tile_offset,
                      const int* __restrict__ tile_rois, TileGrid tg, int C, int H, int W, int PH,
                      int PW, int cblocks, long long num_jobs, int assign
#ifdef ROIALIGN_PROFILE
                      , unsigned long long* prof
#endif
                      ) {
  using K = BwdTile;
#ifdef ROIALIGN_PROFILE
  long long pt[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  const long long t_start = clock64();
#define PROF_T(var) const long long var = clock64()
#define PROF_ADD(i, a, b) pt[i] += (b) - (a)
#else
#define PROF_T(var)
#define PROF_ADD(i, a, b)
#endif
  __shared__ float acc[K::CH * K::CS];
  __shared__ float dyb[K::CH * K::DYS + 4];   // + a trash word for masked staging stores
  __shared__ AxisUnit runit[2][K::RU_CAP];
  __shared__ AxisUnit cunit[2][K::CU_CAP];
  __shared__ BwdHeader header[2];
  __shared__ TileRoi rec_s[K::REC_CHUNK];

  // XCD-aware job order: consecutive workgroup ids go round-robin to the 8
  // XCDs, so give each XCD a contiguous run of logical jobs (neighbouring
  // tiles of one image and channel block share dy blocks through that XCD's L2).
  const long long per_xcd = gridDim.x / 8;
  const long long job = static_cast<long long>(blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
  if (job >= num_jobs) return;
  const int t_in_img = static_cast<int>(job % tg.per_image);
  const int cb = static_cast<int>((job / tg.per_image) % cblocks);
  const int n = static_cast<int>(job / (static_cast<long long>(tg.per_image) * cblocks));
  const long long tile = static_cast<long long>(n) * tg.per_image + t_in_img;
  const int r0 = (t_in_img / tg.tx) * K::TH, q0 = (t_in_img % tg.tx) * K::TW;
  const int c0 = cb * K::CH;
  const int nch = min(K::CH, C - c0);
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const bool producer = wave == K::NWC;
  const int rows = min(K::TH, H - r0), cols = min(K::TW, W - q0);
  float* const plane0 = dx + (static_cast<size_t>(n) * C + c0) * H * W;

  const int list_begin = tile_offset[tile], list_end = tile_offset[tile + 1];
  const int n_rois = list_end - list_begin;
  if (n_rois == 0) {
    if (assign) {
      for (int i = tid; i < nch * K::TH * K::TW; i += K::NT) {
        const int col = i % K::TW, row = (i / K::TW) % K::TH, c = i / (K::TW * K::TH);
        if (row < rows && col < cols)
          plane0[static_cast<size_t>(c) * H * W + static_cast<size_t>(r0 + row) * W + q0 + col] = 0.0f;
      }
    }
    return;
  }

  for (int i = tid; i < K::CH * K::CS; i += K::NT) acc[i] = 0.0f;

  // dy staging map of the compute threads: element idx = tid + k*NTC of a
  // [CH][seg] block, seg = words per channel and chunk.  Fixed for the kernel:
  // st_src = offset inside the ROI's dy block, st_dst = LDS word (the trash
  // word for elements this thread does not stage).
  const int bins = PH * PW;
  const int nphc = min(PH, K::DYS / PW);   // pooled rows per staged chunk
  const int nchunks = (PH + nphc - 1) / nphc;
  const int seg = nphc * PW;
  const int last_valid = (PH - (nchunks - 1) * nphc) * PW;  // words/channel of the last chunk
  int st_src[K::STAGE_ITERS], st_dst[K::STAGE_ITERS], st_j[K::STAGE_ITERS];
  float st_v[K::DEPTH][K::STAGE_ITERS];
#pragma unroll
  for (int k = 0; k < K::STAGE_ITERS; ++k) {
    const int idx = tid + k * K::NTC;
    const int c = idx / seg, j = idx - c * seg;
    const bool mine = !producer && c < nch;
    st_j[k] = mine ? j : 0x7fffffff;
    st_src[k] = mine ? c * bins + j : 0;
    st_dst[k] = mine ? c * K::DYS + j : K::CH * K::DYS;
  }

  auto load_recs = [&](int first) {   // records [first, first+REC_CHUNK) of the list -> LDS
    for (int i = tid; i < K::REC_CHUNK && first + i < n_rois; i += K::NT) {
      const int roi = tile_rois[list_begin + first + i];
      const RoiRec r = recs[roi];
      rec_s[i] = TileRoi{r.start_h, r.start_w, r.bin_h, r.bin_w, r.grid_h, r.grid_w, r.count, roi};
    }
  };
  // issue the global loads of one iteration: ROI slot `slot` of rec_s, pooled-row chunk `chunk`
  auto prefetch = [&](int slot, int chunk, float (&dst)[K::STAGE_ITERS]) {
    const int roi = __builtin_amdgcn_readfirstlane(rec_s[slot].roi);
    const float* src = dy + (static_cast<size_t>(roi) * C + c0) * bins + chunk * seg;
    if (chunk == nchunks - 1 && last_valid != seg) {
#pragma unroll
      for (int k = 0; k < K::STAGE_ITERS; ++k) dst[k] = src[st_j[k] < last_valid ? st_src[k] : 0];
    } else {
#pragma unroll
      for (int k = 0; k < K::STAGE_ITERS; ++k) dst[k] = src[st_src[k]];
    }
  };
  auto produce = [&](int slot, int b) {
#ifdef LAB_NO_PRODUCE
    if (lane == 0) header[b] = BwdHeader{0, 0, 1.0f, 0};
    return;
#endif
    const TileRoi t = rec_s[slot];
    const int n_ru = build_axis_units(t.start_h, t.bin_h, PH, t.grid_h, H, r0, K::TH, lane,
                                      runit[b], K::RU_CAP);
    const int n_cu = build_axis_units(t.start_w, t.bin_w, PW, t.grid_w, W, q0, K::TW, lane,
                                      cunit[b], K::CU_CAP);
    if (lane == 0) header[b] = BwdHeader{n_ru, n_cu, 1.0f / t.count, 0};
    // mark column units whose cells overlap the next unit's
    for (int k = lane; k + 1 < n_cu; k += 64) {
      const int d = cunit[b][k + 1].pos - cunit[b][k].pos;
      if (d >= -1 && d <= 1) cunit[b][k].bin |= kOverlapsNext;
    }
  };

  // One pipeline step of iteration (slot, chunk); `mine` is the register set
  // that holds its dy block, (nslot, nchunk) the iteration DEPTH steps ahead.
  auto step = [&](int slot, int chunk, int b, bool more_rois, bool refill, int nslot, int nchunk,
                  float (&mine)[K::STAGE_ITERS]) {
    PROF_T(t0);
    __syncthreads();  // A: previous iteration fully consumed, dyb is free
    PROF_T(t1);
#pragma unroll
    for (int k = 0; k < K::STAGE_ITERS; ++k) dyb[st_dst[k]] = mine[k];
    PROF_T(t2);
    __syncthreads();  // B: dyb and the unit lists of this ROI are visible
    PROF_T(t3);
    PROF_ADD(0, t0, t1); PROF_ADD(1, t1, t2); PROF_ADD(2, t2, t3);
    if (producer) {
      if (chunk == nchunks - 1 && more_rois) produce(slot + 1, b ^ 1);
      PROF_T(t4);
      PROF_ADD(4, t3, t4);
      return;
    }
    if (refill) prefetch(nslot, nchunk, mine);

    const BwdHeader hd = header[b];
    const int n_ru = __builtin_amdgcn_readfirstlane(hd.n_ru);
    const int n_cu = __builtin_amdgcn_readfirstlane(hd.n_cu);
    if (n_ru > 0 && n_cu > 0) {
      const int ph_a = chunk * nphc, ph_b = min(PH, ph_a + nphc);
      // Lane i looks at row unit i: which part of it lands on the two tile rows
      // this wavefront owns (row_a, row_a + 1)?
      const AxisUnit ru = lane < n_ru ? runit[b][lane] : AxisUnit{0, -4, 0.0f, 0.0f};
      const int row_a = wave * K::ROWS_PER_WAVE;
      const bool in_chunk = ru.bin >= ph_a && ru.bin < ph_b;
      const float w_a = !in_chunk ? 0.0f : ru.pos == row_a ? ru.w0 : ru.pos + 1 == row_a ? ru.w1 : 0.0f;
      const float w_b = !in_chunk ? 0.0f : ru.pos == row_a + 1 ? ru.w0 : ru.pos == row_a ? ru.w1 : 0.0f;
      unsigned long long m_a = __ballot(w_a != 0.0f), m_b = __ballot(w_b != 0.0f);
      if (lane < nch) {
        float* const row_ptr_a = acc + lane * K::CS + 1 + row_a * K::RS;
        float* const row_ptr_b = row_ptr_a + K::RS;
        const float* const dy_lane = dyb + lane * K::DYS - ph_a * PW;
        const AxisUnit* const units = cunit[b];
        while ((m_a | m_b) != 0) {
          // next tap of each owned row; a row without one sits this round out
          const bool has_a = m_a != 0, has_b = m_b != 0;
          const int i_a = has_a ? __builtin_ctzll(m_a) : 0, i_b = has_b ? __builtin_ctzll(m_b) : 0;
          m_a &= m_a - 1; m_b &= m_b - 1;
          const float wy_a = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(w_a), i_a)) * hd.inv_count;
          const float wy_b = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(w_b), i_b)) * hd.inv_count;
          const float* const dy_a = dy_lane + __builtin_amdgcn_readlane(ru.bin, i_a) * PW;
          const float* const dy_b = dy_lane + __builtin_amdgcn_readlane(ru.bin, i_b) * PW;
#ifdef LAB_NO_SCATTER
          if (wy_a == 12345.f) acc[lane] = wy_b + dy_a[0] + dy_b[0];
          continue;
#endif
          if (has_a && has_b)
            scatter_rows<2>(row_ptr_a, row_ptr_b, dy_a, dy_b, wy_a, wy_b, units, n_cu);
          else if (has_a)
            scatter_rows<1>(row_ptr_a, row_ptr_a, dy_a, dy_a, wy_a, wy_a, units, n_cu);
          else
            scatter_rows<1>(row_ptr_b, row_ptr_b, dy_b, dy_b, wy_b, wy_b, units, n_cu);
        }
      }
    }
    PROF_T(t5);
    PROF_ADD(3, t3, t5);
  };

  // Driver: records are (re)loaded every REC_CHUNK ROIs and the pipeline is
  // refilled after each reload.  Iterations run over (ROI, chunk), chunk fastest.
  for (int first = 0; first < n_rois; first += K::REC_CHUNK) {
    __syncthreads();
    load_recs(first);
    __syncthreads();
    const int here = min(K::REC_CHUNK, n_rois - first);   // ROIs in this batch
    // (slot, chunk) of the iteration being executed and of the one DEPTH ahead
    int slot = 0, chunk = 0, nslot = 0, nchunk = 0;
    if (producer) {
      produce(0, 0);
    } else {
#pragma unroll
      for (int s = 0; s < K::DEPTH; ++s) {
        if (nslot < here) prefetch(nslot, nchunk, st_v[s]);
        if (++nchunk == nchunks) { nchunk = 0; ++nslot; }
      }
    }
    while (slot < here) {
#pragma unroll
      for (int s = 0; s < K::DEPTH; ++s) {
        if (slot < here) {
          step(slot, chunk, slot & 1, slot + 1 < here, nslot < here, nslot, nchunk, st_v[s]);
          if (++chunk == nchunks) { chunk = 0; ++slot; }
          if (++nchunk == nchunks) { nchunk = 0; ++nslot; }
        }
      }
    }
  }
  PROF_T(t_w0);
  __syncthreads();

  // Owner writes its tile: two 32-pixel rows per wavefront access.
  for (int i = tid; i < nch * K::TH * K::TW; i += K::NT) {
    const int col = i % K::TW, row = (i / K::TW) % K::TH, c = i / (K::TW * K::TH);
    if (row < rows && col < cols) {
      float* p = plane0 + static_cast<size_t>(c) * H * W + static_cast<size_t>(r0 + row) * W + q0 + col;
      const float v = acc[c * K::CS + 1 + row * K::RS + col];
      *p = assign ? v : *p + v;
    }
  }
#ifdef ROIALIGN_PROFILE
  const long long t_end = clock64();
  if (lane == 0 && (wave == 0 || producer)) {
    if (wave == 0) {
      atomicAdd(prof + 0, (unsigned long long)(t_end - t_start));
      atomicAdd(prof + 1, (unsigned long long)pt[0]);
      atomicAdd(prof + 2, (unsigned long long)pt[1]);
      atomicAdd(prof + 3, (unsigned long long)pt[2]);
      atomicAdd(prof + 4, (unsigned long long)pt[3]);
      atomicAdd(prof + 5, (unsigned long long)(t_end - t_w0));
    } else {
      atomicAdd(prof + 6, (unsigned long long)pt[4]);
      atomicAdd(prof + 7, (unsigned long long)(pt[0] + pt[2]));
    }
  }
#endif
#undef PROF_T
#undef PROF_ADD
}

}  // namespace roialign
