// Exact-fp32 recurrence kernels for the Block Two-Pass operator on gfx950 (MI355X).
//
// They replace the reference's sm90 kernels
//   btp_forward_kernel   csrc/btp/btp-forward.cu:85-457
//   btp_backward_kernel  csrc/btp/btp-backwards.cu:165-808
// and compute the same function,
//   y_t = sum_{s = w(t)}^{t} (prod_{j=s+1..t} a_j) x_s ,  w(t) = first step of the block before
//   t's block (k = 2) or of t's own block (k = 1),
// but are organised for CDNA4 rather than translated:
//
//   * One wavefront owns a span of 128 consecutive steps (8 blocks) of one (batch, head) row:
//     a [16 channel x 128 step] slab, 4 KiB in bf16. The slab is moved between HBM and LDS with
//     16-byte-per-lane accesses in which 16 consecutive lanes cover 256 contiguous bytes of one
//     channel row (for L = 128 a whole instruction covers 1 KiB of contiguous memory).
//   * In LDS the slab is stored with its 16-byte chunks XOR-swizzled by the channel index, so
//     that both the row-major (memory order) and the per-channel (compute order) access patterns
//     are bank-conflict free without padding.
//   * For the arithmetic, lane (j, d) = (lane / 16, lane % 16) owns channel d of blocks 2j and
//     2j+1 of the span and runs the linear recurrence h <- a*h + x in registers. The decay
//     "matrix" of the reference (16x16 per block, built with exp/log and rounded to bf16 for the
//     tensor-core MMA, btp-forward.cu:214-274) is never materialised: a block's contribution is
//     a 16-step recurrence started from zero, and the one-hop carry of the second pass is the
//     same recurrence started from the previous block's local terminal state. All products are
//     plain fp32 multiplications in linear space, so there is no log/exp, no 0*Inf and no
//     cancellation; results agree with a float64 evaluation to fp32 rounding.
//   * The previous block's terminal state travels between lane groups with one ds_bpermute
//     (the reference uses shared memory plus a DSMEM bulk copy and cluster barriers,
//     btp-forward.cu:287-374). At the left edge of a span it comes from the neighbouring
//     wavefront of the workgroup through LDS (one workgroup barrier, rows of several spans only),
//     and at the left edge of a workgroup it is recomputed from the 16 steps before the span (a
//     halo read), so workgroups are fully independent: no flags, no look-back, no second kernel,
//     and the carry is never dropped at a launch-shape boundary (the reference drops it at
//     cluster boundaries, btp-forward.cu:359-366).
//   * Row lengths other than whole spans get one of two more instances of each kernel (movement_for in
//     btp_staging.h picks): kFlat cuts spans from the blocks of all rows in order, for rows that would leave a span
//     partly empty (short rows then share a wavefront, and no carry crosses a row start); kLines moves whole
//     128-byte lines for rows of several spans that do not end on a line, wavefronts passing the row ends to each
//     other through LDS. The arithmetic is the same in all three.
//
// Backward uses, per block i with local index r (g = dy, c = carry into the block,
// dC = carry of the gradient coming back from block i+1):
//   v_r  = a_r v_{r-1} + x_r            (v_{-1} = 0)      local forward state
//   A_r  = g_r + a_{r+1} A_{r+1}        (A_16  = 0)       local reverse state
//   dx_r = g_r + a_{r+1} dx_{r+1}       (a_16 dx_16 := dC) reverse state with the gradient carry
//   dC_{i-1} = a_0 A_0                                    what block i sends to block i-1
//   dA_r = <dx_r, v_{r-1}> + (prod_{j<r} a_j) <A_r, c>    (sum over the 16 channels)
// which is the derivative the reference assembles from "Part V" and "Part A"
// (btp-backwards.cu:372-413, 637-796) but needs no division by a_r, no max-shifted exponentials
// and no special cases: it is finite and correct at a_r = 0.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "btp_device.h"
#include "btp_launch.h"
#include "btp_staging.h"

// Tuning knobs (compile-time). The defaults are the measured best on MI355X.
#ifndef SPEAR_BTP_FWD_WAVES_PER_EU
#define SPEAR_BTP_FWD_WAVES_PER_EU 0
#endif
#ifndef SPEAR_BTP_BWD_WAVES_PER_EU  // 4 waves per SIMD need <= 128 VGPRs; the backward body is ordered to fit
#define SPEAR_BTP_BWD_WAVES_PER_EU 4
#endif
#ifndef SPEAR_BTP_HANDOVER  // 1: carries between the spans of a workgroup go through LDS; 0: every span reads its halo
#define SPEAR_BTP_HANDOVER 1
#endif
#ifndef SPEAR_BTP_SETPRIO  // 1: wavefronts run at raised priority while they issue their global loads / stores
#define SPEAR_BTP_SETPRIO 0
#endif
#if SPEAR_BTP_SETPRIO
#define SPEAR_BTP_PRIO(n) __builtin_amdgcn_s_setprio(n)
#else
#define SPEAR_BTP_PRIO(n) ((void)0)
#endif
#if SPEAR_BTP_FWD_WAVES_PER_EU > 0
#define SPEAR_BTP_FWD_OCC __attribute__((amdgpu_waves_per_eu(SPEAR_BTP_FWD_WAVES_PER_EU)))
#else
#define SPEAR_BTP_FWD_OCC
#endif
#if SPEAR_BTP_BWD_WAVES_PER_EU > 0
#define SPEAR_BTP_BWD_OCC __attribute__((amdgpu_waves_per_eu(SPEAR_BTP_BWD_WAVES_PER_EU)))
#else
#define SPEAR_BTP_BWD_OCC
#endif

namespace spear_btp {

namespace {

// ==========================================================================================
// Forward
// ==========================================================================================
#ifndef SPEAR_BTP_BWD_LINES_WAVES  // same for backward: 0 = as for rows of whole lines, else kWaves or kWavesLong
#define SPEAR_BTP_BWD_LINES_WAVES 0
#endif
#ifndef SPEAR_BTP_FWD_LINES_WAVES  // wavefronts per workgroup of the forward kernel that moves whole lines
#define SPEAR_BTP_FWD_LINES_WAVES 4
#endif
constexpr int kFwdLinesWaves = SPEAR_BTP_FWD_LINES_WAVES;

// kLines: rows of several spans whose byte length is not a multiple of 128; x and y move as whole cache lines
// (line_place in btp_staging.h), at the price of two more workgroup barriers.
// kFlat: rows that leave a span partly empty; spans are cut from the block sequence of the whole tensor (flat_lane in
// btp_staging.h). `spans_per_row` holds the blocks in a row and `total_spans` the blocks in the tensor then, and
// kStreamIn says that no row straddles two spans.
template <class E, class C, class OutT, bool kCheckpoint, bool kStreamIn, bool kLines = false,
          int kW = kLines ? kFwdLinesWaves : kWaves, bool kFlat = false>
__global__ __launch_bounds__(64 * kW) SPEAR_BTP_FWD_OCC void btp_fwd_scan_kernel(
    const typename C::elem* __restrict__ coeff, const uint16_t* __restrict__ x, OutT* __restrict__ y,
    float* __restrict__ ckpt, int L, int spans_per_row, long total_spans, int k) {
  constexpr bool kOutF32 = std::is_same<OutT, float>::value;
  constexpr int kImgBytes = kOutF32 ? 8192 : 4096;
  // kW: wavefronts in this workgroup (8 measured 1-3 % slower than 4 on rows of whole lines, unlike backward)
  constexpr int kImgStride = kImgBytes + kCoeffLdsBytes;
  __shared__ __align__(16) unsigned char lds[kW][kImgStride];
  // Rows longer than one span (kStreamIn == false): a span's first block needs the terminal local
  // state of the block before it. Inside a workgroup the neighbouring wavefront has just computed
  // it, so it is handed over through LDS with the kernel's only workgroup barrier; only the first
  // wavefront of a workgroup recomputes it from a halo read (measured: the halo reads of every span
  // added 12 % to the bytes fetched).
  constexpr bool kHandOver = SPEAR_BTP_HANDOVER && !kStreamIn && kW > 1;
  static_assert(!kLines || kHandOver, "whole-line staging is for rows of several spans");
  static_assert(!kFlat || (!kCheckpoint && !kLines), "flat spans: no carry store, no whole-line movement");
  __shared__ float left_state[kHandOver ? kW : 1][kChan];

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const long span = first_span_of_workgroup<(SPEAR_BTP_XCD_REMAP == 2) || (SPEAR_BTP_XCD_REMAP == 1 && !kStreamIn)>(kW) + wave;
  if (kFlat ? span * (kSpan / kTile) >= total_spans : span >= total_spans) {  // wave-uniform
    // keep the barrier count equal for every wavefront
    if constexpr (kLines) __syncthreads();
    if constexpr (kHandOver) __syncthreads();
    if constexpr (kLines) __syncthreads();
    return;
  }
  const SpanCoord sc = kFlat ? flat_coord(span, spans_per_row, total_spans) : span_coord(span, spans_per_row, L);

  unsigned char* img = lds[wave];
  float* a_lds = reinterpret_cast<float*>(img + kImgBytes);
  const uint16_t* xslab = x + (sc.row * kChan) * (long)L + sc.s0;
  const typename C::elem* arow = coeff + sc.row * (long)L + sc.s0;
  const int j = lane >> 4, d = lane & 15;

  // ---- all global reads are issued before anything waits on them
  // kStreamIn: the host sets it for rows that fit one span. Longer rows hand carries over between
  // the wavefronts of a workgroup (below); only a workgroup's first span re-reads 16 steps.
  constexpr bool kStreamOut = SPEAR_BTP_STREAM_STORES == 1;
  uint4 xin[4];
  [[maybe_unused]] uint4 xtail[2];
  [[maybe_unused]] LinePlace px;
  [[maybe_unused]] const uint16_t* xrows = x + (sc.row * kChan) * (long)L;
  // whether this wavefront moves the last chunks of its rows itself (wave-uniform)
  [[maybe_unused]] const bool tail = kLines && (wave == kW - 1 || sc.sp == spans_per_row - 1);
  if constexpr (kLines) {
    px = line_place(xrows, L, sc.sp, lane, wave == 0);
    line_global_to_regs<nt_loads(kStreamIn)>(xrows, L, sc.sp, px, lane, xin);
    if (tail) line_tail_global_to_regs(xrows, L, sc.sp, lane, xtail);
  } else if constexpr (kFlat) {
    pack_global_to_regs<nt_loads(kStreamIn)>(xrows, L, flat_lane<uint16_t>(lane, L, spans_per_row, sc.sp, sc.nvalid), xin);
  } else {
    slab16_global_to_regs<nt_loads(kStreamIn)>(xslab, L, sc.nvalid, lane, xin);
  }
  const typename C::pair_t ain = coeff_global_to_reg<C>(arow, sc.nvalid, lane);
  // flat spans: no carry enters a block with which a row starts (the same for the 16 lanes of a group)
  const bool startA = kFlat && (sc.sp + 2 * j) % spans_per_row == 0;
  const bool startB = kFlat && (sc.sp + 2 * j + 1) % spans_per_row == 0;

  const bool needs_left = (k == 2) && (sc.sp > 0);            // wave-uniform
  const bool halo = needs_left && !(kHandOver && wave > 0);     // recompute from a halo read
  float c_halo = 0.0f;
  if (halo && j == 0) {
    // local terminal state of the block just left of the span, channel d
    float ah[16], xh[16];
    C::load_block(arow - kTile, ah);
    const uint16_t* xp = xslab + (long)d * L - kTile;
    unpack8<E>(*reinterpret_cast<const uint4*>(xp), xh);
    unpack8<E>(*reinterpret_cast<const uint4*>(xp + 8), xh + 8);
    float h = 0.0f;
#pragma unroll
    for (int r = 0; r < 16; ++r) h = fmaf(ah[r], h, xh[r]);
    c_halo = h;
  }

  if constexpr (kLines) {
    line_regs_to_lds<uint16_t>(img, kImgStride, px, lane, xin);
    if (tail) line_tail_regs_to_lds(img, xrows, L, lane, xtail);
    coeff_reg_to_lds<C>(a_lds, lane, ain);
    __syncthreads();  // the neighbouring wavefronts have written into this image too
  } else {
    slab16_regs_to_lds(img, lane, xin);
    coeff_reg_to_lds<C>(a_lds, lane, ain);
    wave_lds_handover();
  }

  float xf[32], a[32];
  lane_read16<E>(img, j, d, xf);
  coeff_lane_read(a_lds, j, a);

  // chain 1: zero state at the start of block A, run through both blocks. The first 16 steps
  // give A's local states (only the terminal one is kept); continuing into B from that terminal
  // state yields exactly B's outputs for k = 2.
  float yv[32];
  float h = 0.0f;
#pragma unroll
  for (int r = 0; r < 16; ++r) h = fmaf(a[r], h, xf[r]);
  const float vA_last = h;
  h = (k == 2 && !startB) ? vA_last : 0.0f;
#pragma unroll
  for (int r = 16; r < 32; ++r) {
    h = fmaf(a[r], h, xf[r]);
    yv[r] = h;
  }
  // chain 2: B's local terminal state, needed by the next lane group's block A
  float vB_last = yv[31];
  if (k == 2) {
    float h3 = 0.0f;
#pragma unroll
    for (int r = 16; r < 32; ++r) h3 = fmaf(a[r], h3, xf[r]);
    vB_last = h3;
  }
  const float from_left = lane_rotate(vB_last, lane, -16);
  if constexpr (kHandOver) {
    if (j == 3) left_state[wave][d] = vB_last;  // terminal state of the span's last block
    __syncthreads();
    if (needs_left && wave > 0 && j == 0) c_halo = left_state[wave - 1][d];
  }
  const float cA = (k == 2 && !startA) ? (j == 0 ? c_halo : from_left) : 0.0f;
  // chain 3: block A started from its carry
  h = cA;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    h = fmaf(a[r], h, xf[r]);
    yv[r] = h;
  }

  if constexpr (kCheckpoint) {
    if (k == 2) {
      const long nb = L / kTile;
      const long tA = (long)sc.sp * (kSpan / kTile) + 2 * j;  // block index of A inside the row
      float* slot = ckpt + (sc.row * nb + tA) * kChan + d;    // slot of block A's own state
      if (32 * j < sc.nvalid && tA >= 1) slot[-kChan] = cA;   // carry consumed by block A
      if (32 * j + 16 < sc.nvalid) slot[0] = vA_last;         // carry consumed by block B
    }
  }

  // ---- results back through LDS so that the global writes are coalesced (whole lines: the wavefront after
  // this one stores the end of this image, hence the workgroup barrier there)
  wave_lds_handover();
  typedef typename std::conditional<kOutF32, float, uint16_t>::type Y;
  if constexpr (kOutF32) lane_write32(img, j, d, yv);
  else lane_write16<E>(img, j, d, yv);
  Y* yrows = reinterpret_cast<Y*>(y) + (sc.row * kChan) * (long)L;
  if constexpr (kLines) {
    __syncthreads();
    const LinePlace py = line_place(yrows, L, sc.sp, lane, wave == 0);
    line_lds_to_global<kStreamOut>(img, kImgStride, yrows, L, py, lane);
    if (tail) line_tail_lds_to_global(img, yrows, L, sc.sp, lane);
  } else if constexpr (kFlat) {
    wave_lds_handover();
    pack_lds_to_global<kStreamOut>(img, yrows, L, flat_lane<Y>(lane, L, spans_per_row, sc.sp, sc.nvalid), lane);
  } else {
    wave_lds_handover();
    if constexpr (kOutF32) slab32_lds_to_global<kStreamOut>(img, yrows + sc.s0, L, sc.nvalid, lane);
    else slab16_lds_to_global<kStreamOut>(img, yrows + sc.s0, L, sc.nvalid, lane);
  }
}

// ==========================================================================================
// Backward
// ==========================================================================================
// Wavefronts per workgroup of the backward kernels: the larger workgroup for rows of several spans
// where 4 waves per SIMD fit (16-bit dy, 16-bit coefficients). The other variants need more than
// 128 registers, and two 8-wave workgroups would then no longer fit a CU (measured: -33 %).
// Wavefronts per workgroup of the lean backward kernel on rows of one span (no hand-over there, so the
// size is free): 4 measured best at B*H = 32768 rows of L = 128 (1, 2 and 8 are 0.6-1.9 % slower).
#ifndef SPEAR_BTP_BWD_SHORT_ROW_WAVES
#define SPEAR_BTP_BWD_SHORT_ROW_WAVES kWaves
#endif
template <bool kLean, bool kStreamIn>
constexpr int bwd_waves() {
  if (!kLean) return kWaves;
  return kStreamIn ? SPEAR_BTP_BWD_SHORT_ROW_WAVES : kWavesLong;
}

template <class E, class C, class GradT, class DxT, bool kStreamIn, int kW, bool kLines = false, bool kFlat = false>
__device__ __forceinline__ void btp_bwd_scan_body(
    unsigned char (*lds)[4096 + (std::is_same<GradT, float>::value ? 8192 : 4096) + kCoeffLdsBytes],
    const typename C::elem* __restrict__ coeff, const uint16_t* __restrict__ x, const GradT* __restrict__ dy,
    DxT* __restrict__ dx, float* __restrict__ dA, int L, int spans_per_row, long total_spans,
    int k) {
  constexpr bool kGradF32 = std::is_same<GradT, float>::value;
  constexpr bool kDxF32 = std::is_same<DxT, float>::value;  // check mode: dx leaves unrounded
  constexpr int kGradBytes = kGradF32 ? 8192 : 4096;

  // Rows longer than one span: the carries that cross a span boundary inside the workgroup (the
  // forward state from the left neighbour, the gradient carry from the right one) are handed over
  // through LDS with one workgroup barrier; only the workgroup's outer edges read a halo.
  constexpr bool kHandOver = SPEAR_BTP_HANDOVER && !kStreamIn && kW > 1;
  // kLines: x, dy and dx move as whole cache lines (line_place in btp_staging.h); see the forward kernel
  static_assert(!kLines || (kHandOver && !kDxF32), "whole-line staging: 16-bit dx, rows of several spans");
  // kFlat: spans cut from the tensor's block sequence; see the forward kernel
  static_assert(!kFlat || !kLines, "flat spans move rows the plain way");
  constexpr int kImgStride = 4096 + kGradBytes + kCoeffLdsBytes;
  __shared__ float edge_state[kHandOver ? kW : 1][2][kChan];

  SPEAR_BTP_PRIO(3);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const long span = first_span_of_workgroup<(SPEAR_BTP_XCD_REMAP == 2) || (SPEAR_BTP_XCD_REMAP == 1 && !kStreamIn)>(kW) + wave;
  if (kFlat ? span * (kSpan / kTile) >= total_spans : span >= total_spans) {  // wave-uniform
    // keep the barrier count equal for every wavefront
    if constexpr (kLines) __syncthreads();
    if constexpr (kHandOver) __syncthreads();
    if constexpr (kLines) __syncthreads();
    return;
  }
  const SpanCoord sc = kFlat ? flat_coord(span, spans_per_row, total_spans) : span_coord(span, spans_per_row, L);

  unsigned char* img_x = lds[wave];
  unsigned char* img_g = img_x + 4096;
  float* a_lds = reinterpret_cast<float*>(img_g + kGradBytes);
  const long slab_off = (sc.row * kChan) * (long)L + sc.s0;
  const uint16_t* xslab = x + slab_off;
  const typename C::elem* arow = coeff + sc.row * (long)L + sc.s0;
  const int j = lane >> 4, d = lane & 15;

  // ---- global reads
  constexpr bool kStreamOut = SPEAR_BTP_STREAM_STORES == 1;  // see the forward kernel
  uint4 xin[4];
  uint4 gin[kGradF32 ? 8 : 4];
  [[maybe_unused]] uint4 xtail[2], gtail[2];
  [[maybe_unused]] LinePlace px, pg;
  const long rows_off = (sc.row * kChan) * (long)L;
  [[maybe_unused]] const uint16_t* xrows = x + rows_off;
  [[maybe_unused]] const GradT* grows = dy + rows_off;
  // whether this wavefront moves the last chunks of its rows itself (wave-uniform)
  [[maybe_unused]] const bool tail = kLines && (wave == kW - 1 || sc.sp == spans_per_row - 1);
  if constexpr (kLines) {
    px = line_place(xrows, L, sc.sp, lane, wave == 0);
    pg = line_place(grows, L, sc.sp, lane, wave == 0);
    line_global_to_regs<nt_loads(kStreamIn)>(xrows, L, sc.sp, px, lane, xin);
    line_global_to_regs<nt_loads(kStreamIn)>(grows, L, sc.sp, pg, lane, gin);
    if (tail) {
      line_tail_global_to_regs(xrows, L, sc.sp, lane, xtail);
      line_tail_global_to_regs(grows, L, sc.sp, lane, gtail);
    }
  } else if constexpr (kFlat) {
    pack_global_to_regs<nt_loads(kStreamIn)>(xrows, L, flat_lane<uint16_t>(lane, L, spans_per_row, sc.sp, sc.nvalid), xin);
    pack_global_to_regs<nt_loads(kStreamIn)>(grows, L, flat_lane<GradT>(lane, L, spans_per_row, sc.sp, sc.nvalid), gin);
  } else {
    slab16_global_to_regs<nt_loads(kStreamIn)>(xslab, L, sc.nvalid, lane, xin);
    if constexpr (kGradF32) {
      slab32_global_to_regs<nt_loads(kStreamIn)>(reinterpret_cast<const float*>(dy) + slab_off, L, sc.nvalid, lane, gin);
    } else {
      slab16_global_to_regs<nt_loads(kStreamIn)>(reinterpret_cast<const uint16_t*>(dy) + slab_off, L, sc.nvalid, lane, gin);
    }
  }
  const typename C::pair_t ain = coeff_global_to_reg<C>(arow, sc.nvalid, lane);

  const bool needs_left = (k == 2) && (sc.sp > 0);             // wave-uniform
  // (flat spans: the block after the span exists and belongs to the row of the span's last block)
  const int after = sc.sp + kSpan / kTile;  // flat spans: where the block after the span lies, counted from the first row
  const bool needs_right = (k == 2) && (kFlat ? ((span + 1) * (kSpan / kTile) < total_spans && after % spans_per_row != 0)
                                              : (sc.s0 + kSpan < L));  // wave-uniform
  // the right neighbour is in this workgroup unless this is its last wavefront or the last span overall
  const bool right_here = kHandOver && wave + 1 < kW &&
                          (kFlat ? (span + 1) * (kSpan / kTile) < total_spans : span + 1 < total_spans);
  const bool halo_left = needs_left && !(kHandOver && wave > 0);
  const bool halo_right = needs_right && !right_here;
  float c_halo = 0.0f, dc_halo = 0.0f;
  if (halo_left && j == 0) {
    float ah[16], xh[16];
    C::load_block(arow - kTile, ah);
    const uint16_t* xp = xslab + (long)d * L - kTile;
    unpack8<E>(*reinterpret_cast<const uint4*>(xp), xh);
    unpack8<E>(*reinterpret_cast<const uint4*>(xp + 8), xh + 8);
    float h = 0.0f;
#pragma unroll
    for (int r = 0; r < 16; ++r) h = fmaf(ah[r], h, xh[r]);
    c_halo = h;
  }
  if (halo_right && j == 3) {
    // gradient carry sent by the block just right of the span: a_0 * A_0 of that block
    float ah[16], gh[16];
    C::load_block(arow + kSpan, ah);
    // (flat spans: that block lies after / spans_per_row rows further on)
    const long right_off = kFlat ? ((sc.row + after / spans_per_row) * kChan + d) * (long)L + (after % spans_per_row) * kTile
                                 : slab_off + (long)d * L + kSpan;
    if constexpr (kGradF32) {
      const float* gp = reinterpret_cast<const float*>(dy) + right_off;
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const float4 q = *reinterpret_cast<const float4*>(gp + 4 * c);
        gh[4 * c + 0] = q.x; gh[4 * c + 1] = q.y; gh[4 * c + 2] = q.z; gh[4 * c + 3] = q.w;
      }
    } else {
      const uint16_t* gp = reinterpret_cast<const uint16_t*>(dy) + right_off;
      unpack8<E>(*reinterpret_cast<const uint4*>(gp), gh);
      unpack8<E>(*reinterpret_cast<const uint4*>(gp + 8), gh + 8);
    }
    float h = gh[15];
#pragma unroll
    for (int r = 14; r >= 0; --r) h = fmaf(ah[r + 1], h, gh[r]);
    dc_halo = ah[0] * h;
  }

  SPEAR_BTP_PRIO(0);
  if constexpr (kLines) {
    line_regs_to_lds<uint16_t>(img_x, kImgStride, px, lane, xin);
    line_regs_to_lds<GradT>(img_g, kImgStride, pg, lane, gin);
    if (tail) {
      line_tail_regs_to_lds(img_x, xrows, L, lane, xtail);
      line_tail_regs_to_lds(img_g, grows, L, lane, gtail);
    }
    coeff_reg_to_lds<C>(a_lds, lane, ain);
    __syncthreads();  // the neighbouring wavefronts have written into these images too
  } else {
    slab16_regs_to_lds(img_x, lane, xin);
    if constexpr (kGradF32) {
      slab32_regs_to_lds(img_g, lane, gin);
    } else {
      uint4 g4[4] = {gin[0], gin[1], gin[2], gin[3]};
      slab16_regs_to_lds(img_g, lane, g4);
    }
    coeff_reg_to_lds<C>(a_lds, lane, ain);
    wave_lds_handover();
  }

  // Register-lean ordering: x and dy are consumed by the two local recurrences and are dead
  // afterwards; dx is then formed in place from the local reverse state,
  //   dx_r = A_r + q_r ,  q_r = (prod_{j=r+1..15} a_j) dC      (reverse running product)
  //   e_r  = A_r (v_{r-1} + z_r) + q_r v_{r-1} ,  z_r = (prod_{j<r} a_j) c   (forward running product)
  // The coefficients are re-read from LDS in every phase (a broadcast read) rather than held in
  // 32 registers throughout; the compiler barriers keep the reads where they are written.
  float v[32];
  {
    float a[32], xf[32];
    coeff_lane_read(a_lds, j, a);
    lane_read16<E>(img_x, j, d, xf);
    float h = 0.0f;
#pragma unroll
    for (int r = 0; r < 16; ++r) { h = fmaf(a[r], h, xf[r]); v[r] = h; }
    h = 0.0f;
#pragma unroll
    for (int r = 16; r < 32; ++r) { h = fmaf(a[r], h, xf[r]); v[r] = h; }
  }
  asm volatile("" ::: "memory");
  float A[32];  // local reverse states, overwritten by dx below
  float out_left, dcA_raw;
  {
    float a[32], gf[32];
    coeff_lane_read(a_lds, j, a);
    if constexpr (kGradF32) {
      lane_read32(img_g, j, d, gf);
    } else {
      lane_read16<E>(img_g, j, d, gf);
    }
    float h = gf[15];
    A[15] = h;
#pragma unroll
    for (int r = 14; r >= 0; --r) { h = fmaf(a[r + 1], h, gf[r]); A[r] = h; }
    out_left = a[0] * h;
    h = gf[31];
    A[31] = h;
#pragma unroll
    for (int r = 30; r >= 16; --r) { h = fmaf(a[r + 1], h, gf[r]); A[r] = h; }
    dcA_raw = a[16] * h;
  }
  asm volatile("" ::: "memory");

  const bool two = (k == 2);
  const float from_left = lane_rotate(v[31], lane, -16);
  const float from_right = lane_rotate(out_left, lane, +16);
  if constexpr (kHandOver) {
    if (j == 3) edge_state[wave][0][d] = v[31];     // forward state leaving the span on the right
    if (j == 0) edge_state[wave][1][d] = out_left;  // gradient carry leaving the span on the left
    __syncthreads();
    if (needs_left && wave > 0 && j == 0) c_halo = edge_state[wave - 1][0][d];
    if (needs_right && right_here && j == 3) dc_halo = edge_state[wave + 1][1][d];
  }
  // flat spans: no carry crosses from one row into the next (the same for the 16 lanes of a group)
  const bool startA = kFlat && (sc.sp + 2 * j) % spans_per_row == 0;
  const bool startB = kFlat && (sc.sp + 2 * j + 1) % spans_per_row == 0;
  const bool endB = kFlat && (sc.sp + 2 * j + 2) % spans_per_row == 0;
  const float cA = (two && !startA) ? (j == 0 ? c_halo : from_left) : 0.0f;
  const float cB = (two && !startB) ? v[15] : 0.0f;
  const float dcA = (two && !startB) ? dcA_raw : 0.0f;
  const float dcB = (two && !endB) ? (j == 3 ? dc_halo : from_right) : 0.0f;

  float dA_A, dA_B;
#pragma unroll
  for (int blk = 0; blk < 2; ++blk) {
    const int o = 16 * blk;
    float a[16];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const float4 q4 = *reinterpret_cast<const float4*>(a_lds + coeff_slot(32 * j) + o + 4 * c);
      a[4 * c + 0] = q4.x; a[4 * c + 1] = q4.y; a[4 * c + 2] = q4.z; a[4 * c + 3] = q4.w;
    }
    float e[16];
    float z = blk ? cB : cA;
    e[0] = A[o] * z;
#pragma unroll
    for (int r = 1; r < 16; ++r) {
      z *= a[r - 1];
      e[r] = A[o + r] * (v[o + r - 1] + z);
    }
    float q = blk ? dcB : dcA;
    A[o + 15] += q;
    e[15] = fmaf(q, v[o + 14], e[15]);
#pragma unroll
    for (int r = 14; r >= 1; --r) {
      q *= a[r + 1];
      A[o + r] += q;
      e[r] = fmaf(q, v[o + r - 1], e[r]);
    }
    q *= a[1];
    A[o] += q;
    const float red = row_transpose_reduce(e, d);
    if (blk) dA_B = red; else dA_A = red;
    asm volatile("" ::: "memory");
  }
  float (&dxv)[32] = A;
  // dA leaves straight from registers: lane d of a group holds step d of its block, so every
  // group writes two 64-byte runs. (Gathering the span's 128 values in LDS first to write 512
  // contiguous bytes measured slower: the extra hand-over delays the last stores of the wave.)
  if constexpr (C::kLog) {
    // gradient w.r.t. the log-space gate: dg_t = a_t * dA_t (no division anywhere)
    dA_A *= a_lds[coeff_slot(32 * j) + d];
    dA_B *= a_lds[coeff_slot(32 * j) + 16 + d];
  }
  SPEAR_BTP_PRIO(3);
  float* dArow = dA + sc.row * (long)L + sc.s0 + 32 * j + d;
  if (32 * j < sc.nvalid) __builtin_nontemporal_store(dA_A, dArow);
  if (32 * j + 16 < sc.nvalid) __builtin_nontemporal_store(dA_B, dArow + 16);

  if constexpr (kDxF32) {
    // fp32 dx: an 8 KiB image (512 B per channel row) laid over the x and dy images, both dead by now
    wave_lds_handover();
    lane_write32(img_x, j, d, dxv);
    wave_lds_handover();
    if constexpr (kFlat) {
      pack_lds_to_global<kStreamOut>(img_x, dx + rows_off, L, flat_lane<float>(lane, L, spans_per_row, sc.sp, sc.nvalid), lane);
    } else {
      slab32_lds_to_global<kStreamOut>(img_x, dx + slab_off, L, sc.nvalid, lane);
    }
  } else {
    // dx goes back through the x image: every lane overwrites exactly the chunks it read
    lane_write16<E>(img_x, j, d, dxv);
    if constexpr (kLines) {
      __syncthreads();  // the wavefront after this one stores the end of this image
      uint16_t* dxrows = dx + rows_off;
      const LinePlace pd = line_place(dxrows, L, sc.sp, lane, wave == 0);
      line_lds_to_global<kStreamOut>(img_x, kImgStride, dxrows, L, pd, lane);
      if (tail) line_tail_lds_to_global(img_x, dxrows, L, sc.sp, lane);
    } else if constexpr (kFlat) {
      wave_lds_handover();
      pack_lds_to_global<kStreamOut>(img_x, dx + rows_off, L, flat_lane<uint16_t>(lane, L, spans_per_row, sc.sp, sc.nvalid), lane);
    } else {
      wave_lds_handover();
      slab16_lds_to_global<kStreamOut>(img_x, dx + slab_off, L, sc.nvalid, lane);
    }
  }
}

// 16-bit dy and 16-bit coefficients (the reference's operands): the body fits 128 VGPRs, so four
// waves per SIMD are requested explicitly.
template <class E, class C, bool kStreamIn, int kW = bwd_waves<true, kStreamIn>(), bool kLines = false, bool kFlat = false>
__global__ __launch_bounds__((64 * kW)) SPEAR_BTP_BWD_OCC void btp_bwd_scan_kernel(
    const typename C::elem* __restrict__ coeff, const uint16_t* __restrict__ x, const uint16_t* __restrict__ dy,
    uint16_t* __restrict__ dx, float* __restrict__ dA, int L, int spans_per_row, long total_spans, int k) {
  __shared__ __align__(16) unsigned char lds[kW][4096 + 4096 + kCoeffLdsBytes];
  btp_bwd_scan_body<E, C, uint16_t, uint16_t, kStreamIn, kW, kLines, kFlat>(lds, coeff, x, dy, dx, dA, L, spans_per_row,
                                                                        total_spans, k);
}

// fp32 dy (twice the staging registers and LDS), log-space gates (an exponential per coefficient)
// and the fp32-dx check mode: occupancy is left to the compiler.
template <class E, class C, class GradT, class DxT, bool kStreamIn, bool kLines = false, bool kFlat = false>
__global__ __launch_bounds__((64 * bwd_waves<false, kStreamIn>())) void btp_bwd_scan_kernel_relaxed(
    const typename C::elem* __restrict__ coeff, const uint16_t* __restrict__ x, const GradT* __restrict__ dy,
    DxT* __restrict__ dx, float* __restrict__ dA, int L, int spans_per_row, long total_spans, int k) {
  constexpr int kGradBytes = std::is_same<GradT, float>::value ? 8192 : 4096;
  constexpr int kW = bwd_waves<false, kStreamIn>();
  __shared__ __align__(16) unsigned char lds[kW][4096 + kGradBytes + kCoeffLdsBytes];
  btp_bwd_scan_body<E, C, GradT, DxT, kStreamIn, kW, kLines, kFlat>(lds, coeff, x, dy, dx, dA, L, spans_per_row,
                                                                    total_spans, k);
}

template <class E, class C, class OutT, bool kCheckpoint, bool kStreamIn, bool kLines = false, bool kFlat = false>
void launch_fwd_as(const FwdArgs& p, const Grid& g, hipStream_t s) {
  constexpr int kW = kLines ? kFwdLinesWaves : kWaves;
  hipLaunchKernelGGL((btp_fwd_scan_kernel<E, C, OutT, kCheckpoint, kStreamIn, kLines, kW, kFlat>), dim3(g.blocks),
                     dim3(64 * g.waves), 0, s, static_cast<const typename C::elem*>(p.coeff),
                     static_cast<const uint16_t*>(p.x), static_cast<OutT*>(p.y), p.checkpoint, p.L, g.spans_per_row,
                     g.total_spans, p.k);
}

template <class E, class C, class OutT>
hipError_t launch_fwd(const FwdArgs& p, hipStream_t s) {
  const long rows = (long)p.B * p.H;
  const bool ck = p.checkpoint != nullptr;
  const Movement move = movement_for(p.L);
  if (move == kMoveLines) {
    const Grid g = make_grid(rows, p.L, kFwdLinesWaves);
    if (ck) launch_fwd_as<E, C, OutT, true, false, true>(p, g, s);
    else launch_fwd_as<E, C, OutT, false, false, true>(p, g, s);
  } else if (move == kMoveFlat && !ck) {  // (the carry store keeps the per-row cut)
    const Grid g = flat_grid(rows, p.L);
    if (g.stream) launch_fwd_as<E, C, OutT, false, true, false, true>(p, g, s);
    else launch_fwd_as<E, C, OutT, false, false, false, true>(p, g, s);
  } else {
    const Grid g = make_grid(rows, p.L);
    const bool st = stream_inputs(g);
    if (ck) {
      if (st) launch_fwd_as<E, C, OutT, true, true>(p, g, s);
      else launch_fwd_as<E, C, OutT, true, false>(p, g, s);
    } else {
      if (st) launch_fwd_as<E, C, OutT, false, true>(p, g, s);
      else launch_fwd_as<E, C, OutT, false, false>(p, g, s);
    }
  }
  return hipGetLastError();
}

// `g` is the grid of the kernel this picks: see launch_bwd
template <class E, class C, class GradT, bool kStreamIn>
void launch_bwd_as(const BwdArgs& p, const Grid& g, hipStream_t s) {
  constexpr bool kGradF32 = std::is_same<GradT, float>::value;
  const auto* c = static_cast<const typename C::elem*>(p.coeff);
  const auto* x = static_cast<const uint16_t*>(p.x);
  const auto* dy = static_cast<const GradT*>(p.dy);
  auto go = [&](auto kernel, auto* dx) {
    hipLaunchKernelGGL(kernel, dim3(g.blocks), dim3(64 * g.waves), 0, s, c, x, dy, dx, p.dA, p.L, g.spans_per_row,
                       g.total_spans, p.k);
  };
  auto* dx16 = static_cast<uint16_t*>(p.dx);
  if (p.dx_f32) {  // fp32 check mode
    auto* dx32 = static_cast<float*>(p.dx);
    if (g.flat) return go(btp_bwd_scan_kernel_relaxed<E, C, GradT, float, kStreamIn, false, true>, dx32);
    return go(btp_bwd_scan_kernel_relaxed<E, C, GradT, float, kStreamIn>, dx32);
  }
  if constexpr (kGradF32 || C::kLog) {
    if (g.flat) return go(btp_bwd_scan_kernel_relaxed<E, C, GradT, uint16_t, kStreamIn, false, true>, dx16);
    // Rows that do not end on a cache line: whole lines with 16-bit dy (log-space gates: +2-3 % on rows of 8 spans
    // and more). With an fp32 dy, whose rows are twice as long and at worst 64 bytes off the lines, it measured
    // the same on long rows and 5 % slower at L = 272 (two more barriers at this kernel's lower occupancy).
    if constexpr (!kStreamIn && !kGradF32) {
      if (g.lines) return go(btp_bwd_scan_kernel_relaxed<E, C, GradT, uint16_t, false, true>, dx16);
    }
    return go(btp_bwd_scan_kernel_relaxed<E, C, GradT, uint16_t, kStreamIn>, dx16);
  } else if constexpr (kStreamIn) {
    if (g.flat) return go(btp_bwd_scan_kernel<E, C, true, bwd_waves<true, true>(), false, true>, dx16);
    return go(btp_bwd_scan_kernel<E, C, true>, dx16);
  } else {
    const bool small = g.waves == kWaves;  // rows of a few spans: the smaller workgroup
    if (g.flat) {
      return small ? go(btp_bwd_scan_kernel<E, C, false, kWaves, false, true>, dx16)
                   : go(btp_bwd_scan_kernel<E, C, false, kWavesLong, false, true>, dx16);
    }
    if (g.lines) {  // rows that do not end on a cache line
      return small ? go(btp_bwd_scan_kernel<E, C, false, kWaves, true>, dx16)
                   : go(btp_bwd_scan_kernel<E, C, false, kWavesLong, true>, dx16);
    }
    return small ? go(btp_bwd_scan_kernel<E, C, false, kWaves>, dx16) : go(btp_bwd_scan_kernel<E, C, false, kWavesLong>, dx16);
  }
}

template <class E, class C, class GradT>
hipError_t launch_bwd(const BwdArgs& p, hipStream_t s) {
  constexpr bool kGradF32 = std::is_same<GradT, float>::value;
  constexpr bool kLeanIo = !(kGradF32 || C::kLog);
  const bool lean = kLeanIo && !p.dx_f32;  // the kernel launch_bwd_as picks
  const long rows = (long)p.B * p.H;
  // Workgroups of kWavesLong wavefronts hand more carries over in LDS and read fewer halos; with the workgroups
  // dealt to the XCDs in runs (first_span_of_workgroup) halo lines are mostly L2 hits, and on rows of up to 8 spans
  // the smaller workgroup wins: 72.5 -> 69 us at L = 256 and 512 (B H L = 4 Mi), 135.5 -> 132.6 us at L = 1024;
  // from 16 spans on the two are within +-2 % of each other either way.
  int long_row_waves = (p.L + kSpan - 1) / kSpan <= 8 ? kWaves : bwd_waves<true, false>();
  if (SPEAR_BTP_BWD_LINES_WAVES && (p.L % 64) != 0) long_row_waves = SPEAR_BTP_BWD_LINES_WAVES;
  const int waves_long = lean ? long_row_waves : bwd_waves<false, false>();
  const int waves_short = lean ? bwd_waves<true, true>() : bwd_waves<false, true>();
  Movement move = movement_for(p.L);
  // whole lines are not taken with an fp32 dy or in the check mode (launch_bwd_as): those rows go flat or plain
  if (move == kMoveLines && (kGradF32 || p.dx_f32)) move = SPEAR_BTP_FLAT_SPANS ? kMoveFlat : kMovePlain;
  Grid g = move == kMoveFlat ? flat_grid(rows, p.L, waves_long, waves_short) : make_grid(rows, p.L, waves_long, waves_short);
  if (move != kMoveLines) g.lines = false;
  if (stream_inputs(g)) launch_bwd_as<E, C, GradT, true>(p, g, s);
  else launch_bwd_as<E, C, GradT, false>(p, g, s);
  return hipGetLastError();
}

template <class E, class C>
hipError_t forward_by_out(const FwdArgs& p, hipStream_t s) {
  return p.out_dtype == kF32 ? launch_fwd<E, C, float>(p, s) : launch_fwd<E, C, uint16_t>(p, s);
}

template <class E, class C>
hipError_t backward_by_grad(const BwdArgs& p, hipStream_t s) {
  return p.dy_dtype == kF32 ? launch_bwd<E, C, float>(p, s) : launch_bwd<E, C, uint16_t>(p, s);
}

}  // namespace

hipError_t scan_forward(const FwdArgs& p, hipStream_t s) {
  if (p.in_dtype == kBf16)
    return p.log_gate ? forward_by_out<Bf16, LogCoeff>(p, s) : forward_by_out<Bf16, LinCoeff<Bf16>>(p, s);
  return p.log_gate ? forward_by_out<Fp16, LogCoeff>(p, s) : forward_by_out<Fp16, LinCoeff<Fp16>>(p, s);
}

hipError_t scan_backward(const BwdArgs& p, hipStream_t s) {
  if (p.in_dtype == kBf16)
    return p.log_gate ? backward_by_grad<Bf16, LogCoeff>(p, s) : backward_by_grad<Bf16, LinCoeff<Bf16>>(p, s);
  return p.log_gate ? backward_by_grad<Fp16, LogCoeff>(p, s) : backward_by_grad<Fp16, LinCoeff<Fp16>>(p, s);
}

}  // namespace spear_btp
