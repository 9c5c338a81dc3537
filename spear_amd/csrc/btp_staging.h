// HBM <-> LDS staging shared by the BTP kernel families: swizzled LDS images of a wavefront's
// [16 channel x 128 step] slab, streaming (non-temporal) global accesses, the span's coefficient
// copy in LDS and the span coordinate arithmetic.
//
// These take the place of the reference's per-warp shared-memory tiles and their strided 2-byte
// loads/stores and padded transposes (csrc/btp/btp-forward.cu:45-78,247-253,427-452;
// csrc/btp/btp-backwards.cu:52-104,293-334,611-635).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "btp_device.h"

// Tuning knobs (compile-time). The defaults are the measured best on MI355X.
// Non-temporal slab loads. With the carries of neighbouring spans handed over through LDS almost
// nothing is read twice, and plain loads measured 1-2.5 % slower on long rows and fetched 6-12 % more
// than they used (one extra line per contiguous run of a workgroup). The MFMA kernel, whose spans all
// read their halo, keeps plain loads for rows of several spans.
#ifndef SPEAR_BTP_STREAM_LOADS   // 0: never, 1: always, 2: only when a row is a single span
#define SPEAR_BTP_STREAM_LOADS 1
#endif
#ifndef SPEAR_BTP_STREAM_STORES  // 0: never, 1: always
#define SPEAR_BTP_STREAM_STORES 1
#endif

namespace spear_btp {

// Byte offset, inside a wavefront's LDS image with `kRowBytes` per channel row, of the 16-byte
// chunk `chunk` of channel row `r`. XOR with the row index permutes chunks inside aligned groups
// of 16, i.e. inside one 256-byte bank period.
template <int kRowBytes>
__device__ __forceinline__ int swz(int r, int chunk) {
  return r * kRowBytes + ((chunk ^ r) << 4);
}

__device__ __forceinline__ uint4 zero4() { return make_uint4(0u, 0u, 0u, 0u); }

// Streaming (non-temporal) 16-byte global accesses: every byte of the operands is touched exactly
// once per launch, so the lines are marked for early eviction instead of displacing useful data
// in L2 and the last-level cache.
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint4 stream_load16(const void* p) {
  const u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p));
  return make_uint4(v[0], v[1], v[2], v[3]);
}

__device__ __forceinline__ void stream_store16(void* p, const uint4& q) {
  const u32x4_t v = {q.x, q.y, q.z, q.w};
  __builtin_nontemporal_store(v, reinterpret_cast<u32x4_t*>(p));
}

// ---- coefficient sources --------------------------------------------------------------------
// LinCoeff<E>: the reference's operand, linear-space decay a_t stored as a 16-bit float of the
//              same type as x (spear/ops/btp/interface.py:164-188, csrc/btp/_bindings.cu:29-31).
// LogCoeff:    fp32 log-space gate g_t with a_t = exp(g_t); lets callers keep gates such as
//              -softplus(.) at full precision (a bf16 a_t cannot represent 1 - 1e-4).
// Both deliver clamped fp32 a_t to the kernels; nothing downstream differs.
template <class E>
struct LinCoeff {
  typedef uint16_t elem;
  typedef uint32_t pair_t;  // two consecutive coefficients
  static constexpr bool kLog = false;
  static __device__ __forceinline__ pair_t load_pair(const elem* p) {
    return __builtin_nontemporal_load(reinterpret_cast<const uint32_t*>(p));
  }
  static __device__ __forceinline__ pair_t zero_pair() { return 0u; }
  static __device__ __forceinline__ float2 to_float(pair_t w) {
    return make_float2(clamp_coeff<E>(E::lo(w)), clamp_coeff<E>(E::hi(w)));
  }
  // the 16 coefficients of one block (wave-uniform address per lane group)
  static __device__ __forceinline__ void load_block(const elem* p, float (&a)[16]) {
    unpack8<E>(*reinterpret_cast<const uint4*>(p), a);
    unpack8<E>(*reinterpret_cast<const uint4*>(p + 8), a + 8);
#pragma unroll
    for (int i = 0; i < 16; ++i) a[i] = clamp_coeff<E>(a[i]);
  }
};

struct LogCoeff {
  typedef float elem;
  typedef float2 pair_t;
  static constexpr bool kLog = true;
  static __device__ __forceinline__ pair_t load_pair(const elem* p) {
    const floatx2_t v = __builtin_nontemporal_load(reinterpret_cast<const floatx2_t*>(p));
    return make_float2(v[0], v[1]);
  }
  static __device__ __forceinline__ pair_t zero_pair() { return make_float2(-INFINITY, -INFINITY); }
  static __device__ __forceinline__ float decay(float g) {
    // exp2(g * log2 e) on the transcendental unit: relative error ~1e-6 for |g| <= 20, far inside
    // the 1e-4 bound of the fp32 path, and cheap enough to be evaluated again in the halo code
    const float a = __expf(g);
    return a > kCoeffFloor ? a : 0.0f;
  }
  static __device__ __forceinline__ float2 to_float(pair_t g) { return make_float2(decay(g.x), decay(g.y)); }
  static __device__ __forceinline__ void load_block(const elem* p, float (&a)[16]) {
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const float4 q = *reinterpret_cast<const float4*>(p + 4 * c);
      a[4 * c + 0] = decay(q.x); a[4 * c + 1] = decay(q.y); a[4 * c + 2] = decay(q.z); a[4 * c + 3] = decay(q.w);
    }
  }
};

// ------------------------------------------------------------------------------------------
// Stage a [16 x 128] slab of 16-bit elements: coalesced global reads -> swizzled LDS image.
// Lane l of pass `it` handles channel row 4*it + l/16, chunk l%16 (8 steps).
// ------------------------------------------------------------------------------------------
template <bool kStream>
__device__ __forceinline__ uint4 load16(const void* p) {
  if constexpr (kStream) return stream_load16(p);
  return *reinterpret_cast<const uint4*>(p);
}

template <bool kStream>
__device__ __forceinline__ void slab16_global_to_regs(const uint16_t* slab, long L, int nvalid,
                                                      int lane, uint4 (&q)[4]) {
  const int lr = lane >> 4, lp = lane & 15;
  const bool ok = (lp << 3) < nvalid;
#pragma unroll
  for (int it = 0; it < 4; ++it) {
    const int r = it * 4 + lr;
    q[it] = ok ? load16<kStream>(slab + (long)r * L + (lp << 3)) : zero4();
  }
}

__device__ __forceinline__ void slab16_regs_to_lds(unsigned char* img, int lane, const uint4 (&q)[4]) {
  const int lr = lane >> 4, lp = lane & 15;
#pragma unroll
  for (int it = 0; it < 4; ++it) {
    const int r = it * 4 + lr;
    *reinterpret_cast<uint4*>(img + swz<256>(r, lp)) = q[it];
  }
}

template <bool kStream>
__device__ __forceinline__ void store16(void* p, const uint4& q) {
  if constexpr (kStream) stream_store16(p, q);
  else *reinterpret_cast<uint4*>(p) = q;
}

template <bool kStream>
__device__ __forceinline__ void slab16_lds_to_global(const unsigned char* img, uint16_t* slab, long L,
                                                     int nvalid, int lane) {
  const int lr = lane >> 4, lp = lane & 15;
  const bool ok = (lp << 3) < nvalid;
#pragma unroll
  for (int it = 0; it < 4; ++it) {
    const int r = it * 4 + lr;
    const uint4 v = *reinterpret_cast<const uint4*>(img + swz<256>(r, lp));
    if (ok) store16<kStream>(slab + (long)r * L + (lp << 3), v);
  }
}

// Same for a [16 x 128] slab of fp32 (512 B per row, 32 chunks of 4 steps).
// Lane l of pass `it` handles channel row 2*it + l/32, chunk l%32.
template <bool kStream>
__device__ __forceinline__ void slab32_global_to_regs(const float* slab, long L, int nvalid, int lane,
                                                      uint4 (&q)[8]) {
  const int lr = lane >> 5, lp = lane & 31;
  const bool ok = (lp << 2) < nvalid;
#pragma unroll
  for (int it = 0; it < 8; ++it) {
    const int r = it * 2 + lr;
    q[it] = ok ? load16<kStream>(slab + (long)r * L + (lp << 2)) : zero4();
  }
}

__device__ __forceinline__ void slab32_regs_to_lds(unsigned char* img, int lane, const uint4 (&q)[8]) {
  const int lr = lane >> 5, lp = lane & 31;
#pragma unroll
  for (int it = 0; it < 8; ++it) {
    const int r = it * 2 + lr;
    *reinterpret_cast<uint4*>(img + swz<512>(r, lp)) = q[it];
  }
}

template <bool kStream>
__device__ __forceinline__ void slab32_lds_to_global(const unsigned char* img, float* slab, long L,
                                                     int nvalid, int lane) {
  const int lr = lane >> 5, lp = lane & 31;
  const bool ok = (lp << 2) < nvalid;
#pragma unroll
  for (int it = 0; it < 8; ++it) {
    const int r = it * 2 + lr;
    const uint4 v = *reinterpret_cast<const uint4*>(img + swz<512>(r, lp));
    if (ok) store16<kStream>(slab + (long)r * L + (lp << 2), v);
  }
}

// Per-channel reads/writes of the lane's own 32 steps (blocks 2j and 2j+1 of channel d).
template <class E>
__device__ __forceinline__ void lane_read16(const unsigned char* img, int j, int d, float (&v)[32]) {
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const uint4 q = *reinterpret_cast<const uint4*>(img + swz<256>(d, 4 * j + c));
    unpack8<E>(q, v + 8 * c);
  }
}

template <class E>
__device__ __forceinline__ void lane_write16(unsigned char* img, int j, int d, const float (&v)[32]) {
#pragma unroll
  for (int c = 0; c < 4; ++c)
    *reinterpret_cast<uint4*>(img + swz<256>(d, 4 * j + c)) = pack8<E>(v + 8 * c);
}

__device__ __forceinline__ void lane_read32(const unsigned char* img, int j, int d, float (&v)[32]) {
#pragma unroll
  for (int c = 0; c < 8; ++c) {
    const float4 q = *reinterpret_cast<const float4*>(img + swz<512>(d, 8 * j + c));
    v[4 * c + 0] = q.x; v[4 * c + 1] = q.y; v[4 * c + 2] = q.z; v[4 * c + 3] = q.w;
  }
}

__device__ __forceinline__ void lane_write32(unsigned char* img, int j, int d, const float (&v)[32]) {
#pragma unroll
  for (int c = 0; c < 8; ++c)
    *reinterpret_cast<float4*>(img + swz<512>(d, 8 * j + c)) =
        make_float4(v[4 * c + 0], v[4 * c + 1], v[4 * c + 2], v[4 * c + 3]);
}

// Coefficients of the span: 2 per lane from global, clamped, as fp32 into LDS; every lane then
// reads back the 32 of its own two blocks (a broadcast read for the 16 lanes of a group).
template <class C>
__device__ __forceinline__ typename C::pair_t coeff_global_to_reg(const typename C::elem* arow, int nvalid, int lane) {
  return ((lane << 1) < nvalid) ? C::load_pair(arow + (lane << 1)) : C::zero_pair();
}

// The second half of the span is stored 16 floats further on, so that the four lane groups, which
// read four different 16-byte pieces in the same instruction, fall into four different sets of
// LDS banks (without the gap groups 0/2 and 1/3 would collide, 128 floats = two bank periods).
constexpr int kCoeffLdsBytes = (kSpan + 16) * 4;

__device__ __forceinline__ int coeff_slot(int t) { return t + ((t >> 6) << 4); }

template <class C>
__device__ __forceinline__ void coeff_reg_to_lds(float* a_lds, int lane, typename C::pair_t w) {
  *reinterpret_cast<float2*>(a_lds + coeff_slot(lane << 1)) = C::to_float(w);
}

__device__ __forceinline__ void coeff_lane_read(const float* a_lds, int j, float (&a)[32]) {
#pragma unroll
  for (int c = 0; c < 8; ++c) {
    const float4 q = *reinterpret_cast<const float4*>(a_lds + coeff_slot(32 * j) + 4 * c);
    a[4 * c + 0] = q.x; a[4 * c + 1] = q.y; a[4 * c + 2] = q.z; a[4 * c + 3] = q.w;
  }
}

struct SpanCoord {
  long row;    // (batch, head) row index
  int sp;      // span index inside the row
  int s0;      // first step of the span
  int nvalid;  // valid steps in the span (multiple of 16, <= 128)
};

__device__ __forceinline__ SpanCoord span_coord(long span, int spans_per_row, int L) {
  SpanCoord c;
  c.row = span / spans_per_row;
  c.sp = (int)(span - c.row * spans_per_row);
  c.s0 = c.sp * kSpan;
  c.nvalid = min(kSpan, L - c.s0);
  return c;
}

// Workgroup index -> first span. Workgroups are dealt round-robin to the 8 XCDs; with
// SPEAR_BTP_XCD_REMAP each XCD instead walks one contiguous eighth of the tensor.
#ifndef SPEAR_BTP_XCD_REMAP
#define SPEAR_BTP_XCD_REMAP 0
#endif
__device__ __forceinline__ long first_span_of_workgroup(int waves = kWaves) {
#if SPEAR_BTP_XCD_REMAP
  const unsigned n = gridDim.x, b = blockIdx.x;
  const unsigned per = n >> 3;
  const unsigned mapped = (b < (per << 3)) ? (b & 7u) * per + (b >> 3) : b;
  return (long)mapped * waves;
#else
  return (long)blockIdx.x * waves;
#endif
}

struct Grid {
  int spans_per_row;
  long total_spans;
  bool stream;     // kStreamIn of the kernels
  int waves;       // wavefronts per workgroup
  unsigned blocks;
};

// Rows that fit one span are read exactly once and can be streamed; longer rows are re-read by
// neighbouring spans' halo loads, so their lines should stay in L2. `waves_long` is the workgroup
// size (in wavefronts) the calling kernel family uses for those longer rows.
inline Grid make_grid(long rows, int L, int waves_long = kWaves) {
  Grid g;
  g.spans_per_row = (L + kSpan - 1) / kSpan;
  g.total_spans = rows * g.spans_per_row;
  g.stream = g.spans_per_row == 1;  // template argument kStreamIn of the kernels: rows of a single span
  g.waves = g.stream ? kWaves : waves_long;
  g.blocks = (unsigned)((g.total_spans + g.waves - 1) / g.waves);
  return g;
}

inline bool stream_inputs(const Grid& g) { return g.stream; }

// Whether a kernel instance reads its slabs with non-temporal loads, from the knob above and from
// whether its rows are single spans (the kernels' template argument).
constexpr bool nt_loads(bool single_span) {
  return SPEAR_BTP_STREAM_LOADS == 1 || (SPEAR_BTP_STREAM_LOADS == 2 && single_span);
}

}  // namespace spear_btp
