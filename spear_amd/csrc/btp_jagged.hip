// Streaming form of the operator on gfx950: prompt prefill with the state hand-over, and the
// one-token decode step. They stand where the reference has pure PyTorch loops
//   jagged_band_infer_sequential  spear/nn/phalanx/inference.py:36-92
//   JaggedBandState.step          spear/nn/phalanx/inference.py:121-140
//   step_jagged                   spear/nn/phalanx/inference.py:178-278
//   parallel_jagged               spear/nn/phalanx/inference.py:281-360
//
// Prefill is the forward recurrence kernel (same span / lane layout, swizzled LDS images and
// halo recompute as btp_scan.hip) with three additions: the epilogue y * C + V applied in
// registers before the coalesced store, an optional carry into the first block, and the state a
// decoder continues from (block-local state, in-block gate product, previous block's terminal
// state) written by the 16 lanes that own the row's last step. Prompts have any length, so rows
// that are not 16-byte aligned are handled too, by realigning 32-bit words in registers. A second,
// element-granular kernel covers what the tiled one does not (fp32 tensors, other block lengths and
// head sizes).
//
// The step kernel is element-wise over [B, H, D]: a thread owns 8 consecutive channels of one head
// (one 16-byte access per 16-bit operand), the per-head scalars are read by every thread of the
// head and written by the first. State may alias (in-place update): every thread reads all it
// needs before it writes, and the threads that share a head's scalar sit in one wavefront.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "btp_device.h"
#include "btp_launch.h"
#include "btp_staging.h"

namespace spear_btp {

namespace {

// ---- run-time typed scalar access (state vectors and per-head scalars: a few values per row) ----
__device__ __forceinline__ float load_scalar(const void* p, long i, int dt) {
  if (dt == kF32) return static_cast<const float*>(p)[i];
  const uint32_t w = static_cast<const uint16_t*>(p)[i];
  return dt == kBf16 ? Bf16::lo(w) : Fp16::lo(w);
}

__device__ __forceinline__ void store_scalar(void* p, long i, int dt, float v) {
  if (dt == kF32) static_cast<float*>(p)[i] = v;
  else static_cast<uint16_t*>(p)[i] = (uint16_t)((dt == kBf16 ? Bf16::pack2(v, 0.0f) : Fp16::pack2(v, 0.0f)) & 0xffffu);
}

// Block-local state and inclusive gate product after step `upto` of the block starting at kFirst.
template <int kFirst>
__device__ __forceinline__ void local_state_at(const float (&a)[32], const float (&x)[32], int upto, float& h_at,
                                               float& r_at) {
  float h = 0.0f, r = 1.0f;
  h_at = 0.0f;
  r_at = 1.0f;
#pragma unroll
  for (int q = 0; q < 16; ++q) {
    h = fmaf(a[kFirst + q], h, x[kFirst + q]);
    r *= a[kFirst + q];
    if (q == upto) { h_at = h; r_at = r; }
  }
}

// ==========================================================================================
// Prefill, tiled: 16-bit tensors, 16 channels, block length 16
// ==========================================================================================
// kAlign: what every channel row's start is aligned to, in bytes (1: rows alternate between a word and an odd
// element -- L odd, word-aligned tensors -- which is kRowsAlternate of the staging helpers). 16: L is a multiple of 8 and every
// pointer 16-byte aligned (16-byte accesses); 4 or 2: rows of any length (see
// slab16_global_to_regs_ragged), starting on words when L is even and the tensors are word-aligned.
template <class E, class C, bool kEpilogue, bool kStreamIn, int kAlign>
__global__ __launch_bounds__(64 * kWaves) void jagged_prefill_kernel(
    const typename C::elem* __restrict__ coeff, const uint16_t* __restrict__ x, const uint16_t* __restrict__ cmul,
    const uint16_t* __restrict__ vadd, const void* __restrict__ carry_init, uint16_t* __restrict__ y,
    void* __restrict__ h_tail, void* __restrict__ r_tail, void* __restrict__ c_prev_tail, int state_dtype,
    int r_dtype, int L, int spans_per_row, long total_spans) {
  constexpr bool kRagged = kAlign < 16;
  constexpr int kRows = kAlign == 4 ? kRowsOnWords : kAlign == 1 ? kRowsAlternate : kRowsAnywhere;
  constexpr int kImages = kEpilogue ? 3 : 1;
  __shared__ __align__(16) unsigned char lds[kWaves][kImages * 4096 + kCoeffLdsBytes];

  // rows of several spans: the carry into a span's first block comes from the neighbouring
  // wavefront through LDS (one workgroup barrier), as in the forward kernel
  constexpr bool kHandOver = !kStreamIn && kWaves > 1;
  __shared__ float left_state[kHandOver ? kWaves : 1][kChan];

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const long span = first_span_of_workgroup<(SPEAR_BTP_XCD_REMAP == 2) || (SPEAR_BTP_XCD_REMAP == 1 && !kStreamIn)>() + wave;
  if (span >= total_spans) {  // wave-uniform
    if constexpr (kHandOver) __syncthreads();  // keep the barrier count equal for every wavefront
    return;
  }
  const SpanCoord sc = span_coord(span, spans_per_row, L);

  unsigned char* img = lds[wave];
  float* a_lds = reinterpret_cast<float*>(img + kImages * 4096);
  const long slab_off = (sc.row * kChan) * (long)L + sc.s0;
  const typename C::elem* arow = coeff + sc.row * (long)L + sc.s0;
  const int j = lane >> 4, d = lane & 15;

  uint4 xin[4], cin[4], vin[4];
  uint32_t xw[kRagged ? 16 : 1], cw[kRagged ? 16 : 1], vw[kRagged ? 16 : 1];  // the ragged path's words
  uint32_t xe = 0u, ce = 0u, ve = 0u;
  typename C::pair_t ain;
  if constexpr (kRagged) {
    slab16_global_to_regs_ragged<kRows>(x + slab_off, L, sc.nvalid, lane, xw, xe);
    ain = coeff_global_to_reg_ragged<C>(arow, sc.nvalid, lane);
    if constexpr (kEpilogue) {
      slab16_global_to_regs_ragged<kRows>(cmul + slab_off, L, sc.nvalid, lane, cw, ce);
      slab16_global_to_regs_ragged<kRows>(vadd + slab_off, L, sc.nvalid, lane, vw, ve);
    }
  } else {
    slab16_global_to_regs<nt_loads(kStreamIn)>(x + slab_off, L, sc.nvalid, lane, xin);
    ain = coeff_global_to_reg<C>(arow, sc.nvalid, lane);
    if constexpr (kEpilogue) {
      slab16_global_to_regs<true>(cmul + slab_off, L, sc.nvalid, lane, cin);  // read once, by this span only
      slab16_global_to_regs<true>(vadd + slab_off, L, sc.nvalid, lane, vin);
    }
  }

  float c_halo = 0.0f;
  if (j == 0) {
    if (sc.sp > 0 && !(kHandOver && wave > 0)) {  // local terminal state of the block left of the span, channel d
      float ah[16], xh[16];
      const uint16_t* xp = x + slab_off + (long)d * L - kTile;
      if constexpr (kRagged) {
        C::load_block_ragged(arow - kTile, ah);
        unpack8<E>(load16_plain_unaligned(xp), xh);
        unpack8<E>(load16_plain_unaligned(xp + 8), xh + 8);
      } else {
        C::load_block(arow - kTile, ah);
        unpack8<E>(*reinterpret_cast<const uint4*>(xp), xh);
        unpack8<E>(*reinterpret_cast<const uint4*>(xp + 8), xh + 8);
      }
      float h = 0.0f;
#pragma unroll
      for (int r = 0; r < 16; ++r) h = fmaf(ah[r], h, xh[r]);
      c_halo = h;
    } else if (sc.sp == 0 && carry_init != nullptr) {
      c_halo = load_scalar(carry_init, sc.row * kChan + d, state_dtype);
    }
  }

  coeff_reg_to_lds<C>(a_lds, lane, ain);
  if constexpr (kRagged) {
    slab16_regs_realign<kRows>(x + slab_off, L, sc.nvalid, lane, xw, xe);
    slab16_regs_to_lds_ragged(img, lane, xw);
    if constexpr (kEpilogue) {
      slab16_regs_realign<kRows>(cmul + slab_off, L, sc.nvalid, lane, cw, ce);
      slab16_regs_to_lds_ragged(img + 4096, lane, cw);
      slab16_regs_realign<kRows>(vadd + slab_off, L, sc.nvalid, lane, vw, ve);
      slab16_regs_to_lds_ragged(img + 8192, lane, vw);
    }
  } else {
    slab16_regs_to_lds(img, lane, xin);
    if constexpr (kEpilogue) {
      slab16_regs_to_lds(img + 4096, lane, cin);
      slab16_regs_to_lds(img + 8192, lane, vin);
    }
  }
  wave_lds_handover();

  float xf[32], a[32], yv[32];
  lane_read16<E>(img, j, d, xf);
  coeff_lane_read(a_lds, j, a);

  // Same three chains as the forward kernel: local run through block A, continued into block B
  // (B's outputs); B's own local terminal state for the next lane group; A from its carry.
  float h = 0.0f;
#pragma unroll
  for (int r = 0; r < 16; ++r) h = fmaf(a[r], h, xf[r]);
  const float vA_last = h;
#pragma unroll
  for (int r = 16; r < 32; ++r) {
    h = fmaf(a[r], h, xf[r]);
    yv[r] = h;
  }
  float vB_last = 0.0f;
#pragma unroll
  for (int r = 16; r < 32; ++r) vB_last = fmaf(a[r], vB_last, xf[r]);
  const float from_left = lane_rotate(vB_last, lane, -16);
  if constexpr (kHandOver) {
    if (j == 3) left_state[wave][d] = vB_last;
    __syncthreads();
    if (sc.sp > 0 && wave > 0 && j == 0) c_halo = left_state[wave - 1][d];
  }
  const float cA = j == 0 ? c_halo : from_left;
  h = cA;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    h = fmaf(a[r], h, xf[r]);
    yv[r] = h;
  }

  // ---- hand-over state, by the lanes that own the row's last step (wave-uniform conditions)
  if (h_tail != nullptr && sc.sp == spans_per_row - 1) {
    const int p = sc.nvalid - 1, q = p & 31;
    if (j == (p >> 5)) {
      const bool in_b = q >= 16;  // the last step lies in the lane's second block
      float ht, rt;
      // two copies with constant indices: selecting between array elements at run time would
      // move the register arrays to scratch memory
      if (in_b) local_state_at<16>(a, xf, q & 15, ht, rt);
      else local_state_at<0>(a, xf, q & 15, ht, rt);
      const bool full = (q & 15) == 15;
      const float prev = in_b ? vA_last : cA;  // terminal local state of the block before (0 / carry_init at the row start)
      const long o = sc.row * kChan + d;
      store_scalar(h_tail, o, state_dtype, ht);
      store_scalar(c_prev_tail, o, state_dtype, full ? ht : prev);
      if (d == 0) store_scalar(r_tail, sc.row, r_dtype, full ? 1.0f : rt);
    }
  }

  if constexpr (kEpilogue) {
    float cf[32];
    lane_read16<E>(img + 4096, j, d, cf);
#pragma unroll
    for (int r = 0; r < 32; ++r) yv[r] *= cf[r];
    lane_read16<E>(img + 8192, j, d, cf);
#pragma unroll
    for (int r = 0; r < 32; ++r) yv[r] += cf[r];
  }

  wave_lds_handover();
  lane_write16<E>(img, j, d, yv);
  wave_lds_handover();
  if constexpr (kRagged) slab16_lds_to_global_ragged<kRows>(img, y + slab_off, L, sc.nvalid, lane, sc.nvalid == L);
  else slab16_lds_to_global<true>(img, y + slab_off, L, sc.nvalid, lane);
}

// ==========================================================================================
// Prefill, element-granular: any element type, row length, block length and head size.
// One thread per (row, channel, block); lanes run over blocks, so a wavefront still covers a
// contiguous stretch of one channel row.
// ==========================================================================================
struct F32Elt {};

template <class T>
struct Scalar;  // element access by index
template <>
struct Scalar<Bf16> {
  typedef uint16_t type;
  static __device__ __forceinline__ float get(const type* p, long i) { return Bf16::lo(p[i]); }
  static __device__ __forceinline__ void put(type* p, long i, float v) { p[i] = (uint16_t)(Bf16::pack2(v, 0.0f) & 0xffffu); }
};
template <>
struct Scalar<Fp16> {
  typedef uint16_t type;
  static __device__ __forceinline__ float get(const type* p, long i) { return Fp16::lo(p[i]); }
  static __device__ __forceinline__ void put(type* p, long i, float v) { p[i] = (uint16_t)(Fp16::pack2(v, 0.0f) & 0xffffu); }
};
template <>
struct Scalar<F32Elt> {
  typedef float type;
  static __device__ __forceinline__ float get(const type* p, long i) { return p[i]; }
  static __device__ __forceinline__ void put(type* p, long i, float v) { p[i] = v; }
};

template <class T>
__global__ __launch_bounds__(256) void jagged_prefill_any_kernel(
    const void* __restrict__ coeff, int a_dtype, int log_a, const typename Scalar<T>::type* __restrict__ x,
    const typename Scalar<T>::type* __restrict__ cmul, const typename Scalar<T>::type* __restrict__ vadd,
    const void* __restrict__ carry_init, typename Scalar<T>::type* __restrict__ y, void* __restrict__ h_tail,
    void* __restrict__ r_tail, void* __restrict__ c_prev_tail, int state_dtype, int r_dtype, long rows, int D, int L,
    int block_len, int nblk) {
  const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= rows * D * nblk) return;
  const int i = (int)(idx % nblk);
  const long rd = idx / nblk;
  const int d = (int)(rd % D);
  const long row = rd / D;
  const long xo = rd * (long)L, ao = row * (long)L;

  auto gate = [&](int t) {
    const float g = load_scalar(coeff, ao + t, a_dtype);
    return log_a ? __expf(g) : g;
  };

  float carry = 0.0f;
  if (i > 0) {  // terminal local state of the block before
    for (int t = (i - 1) * block_len; t < i * block_len; ++t) carry = fmaf(gate(t), carry, Scalar<T>::get(x, xo + t));
  } else if (carry_init != nullptr) {
    carry = load_scalar(carry_init, rd, state_dtype);
  }

  const int t0 = i * block_len, t1 = min(L, t0 + block_len);
  float hl = 0.0f, hc = carry, rp = 1.0f;
  for (int t = t0; t < t1; ++t) {
    const float a = gate(t), xv = Scalar<T>::get(x, xo + t);
    hl = fmaf(a, hl, xv);
    hc = fmaf(a, hc, xv);
    rp *= a;
    float out = hc;
    if (cmul != nullptr) out = fmaf(out, Scalar<T>::get(cmul, xo + t), Scalar<T>::get(vadd, xo + t));
    Scalar<T>::put(y, xo + t, out);
  }
  if (h_tail != nullptr && i == nblk - 1) {
    const bool full = (t1 - t0) == block_len;
    store_scalar(h_tail, rd, state_dtype, hl);
    store_scalar(c_prev_tail, rd, state_dtype, full ? hl : carry);
    if (d == 0) store_scalar(r_tail, row, r_dtype, full ? 1.0f : rp);
  }
}

// ==========================================================================================
// Decode step
// ==========================================================================================
template <class T>
struct Oct;  // 8 consecutive elements
template <class E16>
struct Oct16 {
  typedef uint16_t type;
  static __device__ __forceinline__ void get(const type* p, long i, float (&v)[8]) {
    unpack8<E16>(*reinterpret_cast<const uint4*>(p + i), v);
  }
  static __device__ __forceinline__ void put(type* p, long i, const float (&v)[8]) {
    *reinterpret_cast<uint4*>(p + i) = pack8<E16>(v);
  }
};
template <>
struct Oct<Bf16> : Oct16<Bf16> {};
template <>
struct Oct<Fp16> : Oct16<Fp16> {};
template <>
struct Oct<F32Elt> {
  typedef float type;
  static __device__ __forceinline__ void get(const type* p, long i, float (&v)[8]) {
    const float4 lo = *reinterpret_cast<const float4*>(p + i), hi = *reinterpret_cast<const float4*>(p + i + 4);
    v[0] = lo.x; v[1] = lo.y; v[2] = lo.z; v[3] = lo.w; v[4] = hi.x; v[5] = hi.y; v[6] = hi.z; v[7] = hi.w;
  }
  static __device__ __forceinline__ void put(type* p, long i, const float (&v)[8]) {
    *reinterpret_cast<float4*>(p + i) = make_float4(v[0], v[1], v[2], v[3]);
    *reinterpret_cast<float4*>(p + i + 4) = make_float4(v[4], v[5], v[6], v[7]);
  }
};

struct StepScalars {
  float a, r_new, r_store;
};

// Per-head scalar update: gate, inclusive in-block gate product (linear or log accumulator).
__device__ __forceinline__ StepScalars step_scalars(const JagStepArgs& p, long row) {
  StepScalars s;
  const float A = load_scalar(p.a_t, row, p.a_dtype);
  s.a = p.log_a ? __expf(A) : A;
  const float prev = p.r_in != nullptr ? load_scalar(p.r_in, row, p.r_dtype) : (p.log_r ? 0.0f : 1.0f);
  if (p.log_r) {
    const float lr = prev + __logf(fmaxf(s.a, p.tiny));
    s.r_new = __expf(lr);
    s.r_store = lr;
  } else {
    s.r_new = s.a * prev;
    s.r_store = s.r_new;
  }
  if (p.boundary) s.r_store = p.log_r ? 0.0f : 1.0f;
  return s;
}

template <class T, class S>
__global__ __launch_bounds__(256) void jagged_step_kernel(const JagStepArgs p, long octs, int octs_per_head) {
  const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= octs) return;
  const long row = idx / octs_per_head;
  const long e = idx * 8;
  typedef typename Oct<T>::type elt_t;
  typedef typename Oct<S>::type st_t;

  const StepScalars s = step_scalars(p, row);
  float h[8], x[8], cp[8], y[8], c[8], v[8];
  Oct<S>::get(static_cast<const st_t*>(p.h_in), e, h);
  Oct<S>::get(static_cast<const st_t*>(p.c_prev_in), e, cp);
  Oct<T>::get(static_cast<const elt_t*>(p.x_t), e, x);
  const bool epilogue = p.c_t != nullptr;  // its two loads go out with the others, ahead of any arithmetic
  if (epilogue) {
    Oct<T>::get(static_cast<const elt_t*>(p.c_t), e, c);
    Oct<T>::get(static_cast<const elt_t*>(p.v_t), e, v);
  }
#pragma unroll
  for (int q = 0; q < 8; ++q) {
    h[q] = s.a * h[q] + x[q];
    y[q] = h[q] + s.r_new * cp[q];
  }
  if (epilogue) {
#pragma unroll
    for (int q = 0; q < 8; ++q) y[q] = y[q] * c[q] + v[q];
  }
  Oct<T>::put(static_cast<elt_t*>(p.y_t), e, y);
  if (p.boundary) {
    Oct<S>::put(static_cast<st_t*>(p.c_prev_out), e, h);
#pragma unroll
    for (int q = 0; q < 8; ++q) h[q] = 0.0f;
  }
  Oct<S>::put(static_cast<st_t*>(p.h_out), e, h);
  if (idx % octs_per_head == 0) store_scalar(p.r_out, row, p.r_dtype, s.r_store);
}

// Any head size: one thread per head walks its channels (never races, whatever aliases).
template <class T, class S>
__global__ __launch_bounds__(256) void jagged_step_any_kernel(const JagStepArgs p, long rows, int D) {
  const long row = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (row >= rows) return;
  typedef typename Scalar<T>::type elt_t;
  typedef typename Scalar<S>::type st_t;
  const StepScalars s = step_scalars(p, row);
  for (int d = 0; d < D; ++d) {
    const long e = row * D + d;
    const float h = s.a * Scalar<S>::get(static_cast<const st_t*>(p.h_in), e) + Scalar<T>::get(static_cast<const elt_t*>(p.x_t), e);
    float yv = h + s.r_new * Scalar<S>::get(static_cast<const st_t*>(p.c_prev_in), e);
    if (p.c_t != nullptr)
      yv = yv * Scalar<T>::get(static_cast<const elt_t*>(p.c_t), e) + Scalar<T>::get(static_cast<const elt_t*>(p.v_t), e);
    Scalar<T>::put(static_cast<elt_t*>(p.y_t), e, yv);
    if (p.boundary) Scalar<S>::put(static_cast<st_t*>(p.c_prev_out), e, h);
    Scalar<S>::put(static_cast<st_t*>(p.h_out), e, p.boundary ? 0.0f : h);
  }
  store_scalar(p.r_out, row, p.r_dtype, s.r_store);
}

template <class T, class S>
hipError_t launch_step(const JagStepArgs& p, hipStream_t s) {
  const long rows = (long)p.B * p.H;
  // the 8-channel form needs whole octets per head, and heads whose threads share a wavefront
  // (64 % octets == 0) so that an aliased scalar is read by all of them before it is written
  const int oph = p.D / 8;
  if (p.aligned && p.D % 8 == 0 && 64 % oph == 0) {
    const long octs = rows * oph;
    hipLaunchKernelGGL((jagged_step_kernel<T, S>), dim3((unsigned)((octs + 255) / 256)), dim3(256), 0, s, p, octs, oph);
  } else {
    hipLaunchKernelGGL((jagged_step_any_kernel<T, S>), dim3((unsigned)((rows + 255) / 256)), dim3(256), 0, s, p, rows, p.D);
  }
  return hipGetLastError();
}

template <class T>
hipError_t step_by_state(const JagStepArgs& p, hipStream_t s) {
  if (p.state_dtype == p.x_dtype) return launch_step<T, T>(p, s);
  return launch_step<T, F32Elt>(p, s);  // validated by the caller: otherwise fp32 state
}

template <class E, class C>
void launch_prefill_tiled(const JagPrefillArgs& p, hipStream_t s) {
  const Grid g = make_grid((long)p.B * p.H, p.L);
  const auto* a = static_cast<const typename C::elem*>(p.a);
  const auto* x = static_cast<const uint16_t*>(p.x);
  const auto* c = static_cast<const uint16_t*>(p.c);
  const auto* v = static_cast<const uint16_t*>(p.v);
  auto* y = static_cast<uint16_t*>(p.y);
  const bool st = stream_inputs(g);
  auto word_aligned = [](const void* q) { return (reinterpret_cast<uintptr_t>(q) & 3u) == 0; };
  const bool on_words = word_aligned(p.x) && word_aligned(p.c) && word_aligned(p.v) && word_aligned(p.y);
  const int align = (p.L % 8 == 0 && p.aligned) ? 16 : !on_words ? 2 : (p.L % 2 == 0) ? 4 : 1;
#define SPEAR_JAG_LAUNCH(EPI, ST, AL)                                                                         \
  hipLaunchKernelGGL((jagged_prefill_kernel<E, C, EPI, ST, AL>), dim3(g.blocks), dim3(64 * kWaves), 0, s, a, x, \
                     c, v, p.carry_init, y, p.h_tail, p.r_tail, p.c_prev_tail, p.state_dtype, p.r_dtype, p.L,   \
                     g.spans_per_row, g.total_spans)
#define SPEAR_JAG_BY_SPAN(EPI, AL) \
  do {                             \
    if (st) SPEAR_JAG_LAUNCH(EPI, true, AL); \
    else SPEAR_JAG_LAUNCH(EPI, false, AL);   \
  } while (0)
#define SPEAR_JAG_BY_ALIGN(EPI)                       \
  do {                                                \
    if (align == 16) SPEAR_JAG_BY_SPAN(EPI, 16);      \
    else if (align == 4) SPEAR_JAG_BY_SPAN(EPI, 4);   \
    else if (align == 1) SPEAR_JAG_BY_SPAN(EPI, 1);   \
    else SPEAR_JAG_BY_SPAN(EPI, 2);                   \
  } while (0)
  if (p.c != nullptr) SPEAR_JAG_BY_ALIGN(true);
  else SPEAR_JAG_BY_ALIGN(false);
#undef SPEAR_JAG_BY_ALIGN
#undef SPEAR_JAG_BY_SPAN
#undef SPEAR_JAG_LAUNCH
}

template <class T>
void launch_prefill_any(const JagPrefillArgs& p, hipStream_t s) {
  typedef typename Scalar<T>::type elt_t;
  const long rows = (long)p.B * p.H;
  const int nblk = (p.L + p.block_len - 1) / p.block_len;
  const long threads = rows * p.D * nblk;
  hipLaunchKernelGGL((jagged_prefill_any_kernel<T>), dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, s, p.a,
                     p.a_dtype, p.log_a ? 1 : 0, static_cast<const elt_t*>(p.x), static_cast<const elt_t*>(p.c),
                     static_cast<const elt_t*>(p.v), p.carry_init, static_cast<elt_t*>(p.y), p.h_tail, p.r_tail,
                     p.c_prev_tail, p.state_dtype, p.r_dtype, rows, p.D, p.L, p.block_len, nblk);
}

}  // namespace

bool jagged_prefill_is_tiled(const JagPrefillArgs& p) {
  const bool own16 = p.a_dtype == p.x_dtype;        // a_t or log(a_t) in the tensors' 16-bit type
  const bool log32 = p.log_a && p.a_dtype == kF32;  // fp32 log-space gate
  return p.x_dtype != kF32 && p.D == kChan && p.block_len == kTile && (own16 || log32);
}

hipError_t jagged_prefill(const JagPrefillArgs& p, hipStream_t s) {
  if (jagged_prefill_is_tiled(p)) {
    if (p.x_dtype == kBf16) {
      if (!p.log_a) launch_prefill_tiled<Bf16, LinCoeff<Bf16>>(p, s);
      else if (p.a_dtype == kF32) launch_prefill_tiled<Bf16, LogCoeff>(p, s);
      else launch_prefill_tiled<Bf16, LogCoeff16<Bf16>>(p, s);
    } else {
      if (!p.log_a) launch_prefill_tiled<Fp16, LinCoeff<Fp16>>(p, s);
      else if (p.a_dtype == kF32) launch_prefill_tiled<Fp16, LogCoeff>(p, s);
      else launch_prefill_tiled<Fp16, LogCoeff16<Fp16>>(p, s);
    }
  } else if (p.x_dtype == kBf16) {
    launch_prefill_any<Bf16>(p, s);
  } else if (p.x_dtype == kF16) {
    launch_prefill_any<Fp16>(p, s);
  } else {
    launch_prefill_any<F32Elt>(p, s);
  }
  return hipGetLastError();
}

hipError_t jagged_step(const JagStepArgs& p, hipStream_t s) {
  if (p.x_dtype == kBf16) return step_by_state<Bf16>(p, s);
  if (p.x_dtype == kF16) return step_by_state<Fp16>(p, s);
  return launch_step<F32Elt, F32Elt>(p, s);
}

}  // namespace spear_btp
