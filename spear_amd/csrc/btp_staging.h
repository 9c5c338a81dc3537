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
#ifndef SPEAR_BTP_WHOLE_LINES    // 1: rows of several spans that do not end on a 128-byte line move as whole lines
#define SPEAR_BTP_WHOLE_LINES 1
#endif
#ifndef SPEAR_BTP_FLAT_SPANS      // 1: rows that leave a span partly empty are cut from the tensor's block sequence
#define SPEAR_BTP_FLAT_SPANS 1
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

// 16 bytes from an address that is only 2-byte aligned (used by the row-of-any-length paths).
typedef uint32_t u32x4_a2_t __attribute__((ext_vector_type(4), aligned(2)));
__device__ __forceinline__ uint4 load16_plain_unaligned_fwd(const uint16_t* p) {
  const u32x4_a2_t v = *reinterpret_cast<const u32x4_a2_t*>(p);
  return make_uint4(v[0], v[1], v[2], v[3]);
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
  // element-aligned rows: a pair of which `n` (1 or 2) coefficients exist, and a whole block
  static __device__ __forceinline__ pair_t load_pair_ragged(const elem* p, int n) {
    return (uint32_t)p[0] | (n > 1 ? (uint32_t)p[1] << 16 : 0u);
  }
  static __device__ __forceinline__ void load_block_ragged(const elem* p, float (&a)[16]) {
    unpack8<E>(load16_plain_unaligned_fwd(p), a);
    unpack8<E>(load16_plain_unaligned_fwd(p + 8), a + 8);
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
  static __device__ __forceinline__ pair_t load_pair_ragged(const elem* p, int n) {
    return make_float2(p[0], n > 1 ? p[1] : -INFINITY);
  }
  static __device__ __forceinline__ void load_block_ragged(const elem* p, float (&a)[16]) {
#pragma unroll
    for (int i = 0; i < 16; ++i) a[i] = decay(p[i]);
  }
};

// Log-space gate stored in the tensors' own 16-bit type (prompt prefill with use_log_a on 16-bit
// tensors, spear/nn/phalanx/inference.py:296): a_t = exp(g_t) formed in fp32.
template <class E>
struct LogCoeff16 {
  typedef uint16_t elem;
  typedef uint32_t pair_t;
  static constexpr bool kLog = true;
  static __device__ __forceinline__ uint32_t minus_inf() { return E::pack2(-INFINITY, -INFINITY); }
  static __device__ __forceinline__ pair_t load_pair(const elem* p) {
    return __builtin_nontemporal_load(reinterpret_cast<const uint32_t*>(p));
  }
  static __device__ __forceinline__ pair_t zero_pair() { return minus_inf(); }
  static __device__ __forceinline__ float2 to_float(pair_t w) {
    return make_float2(LogCoeff::decay(E::lo(w)), LogCoeff::decay(E::hi(w)));
  }
  static __device__ __forceinline__ void load_block(const elem* p, float (&a)[16]) {
    unpack8<E>(*reinterpret_cast<const uint4*>(p), a);
    unpack8<E>(*reinterpret_cast<const uint4*>(p + 8), a + 8);
#pragma unroll
    for (int i = 0; i < 16; ++i) a[i] = LogCoeff::decay(a[i]);
  }
  static __device__ __forceinline__ pair_t load_pair_ragged(const elem* p, int n) {
    return (uint32_t)p[0] | (n > 1 ? (uint32_t)p[1] << 16 : minus_inf() & 0xffff0000u);
  }
  static __device__ __forceinline__ void load_block_ragged(const elem* p, float (&a)[16]) {
    unpack8<E>(load16_plain_unaligned_fwd(p), a);
    unpack8<E>(load16_plain_unaligned_fwd(p + 8), a + 8);
#pragma unroll
    for (int i = 0; i < 16; ++i) a[i] = LogCoeff::decay(a[i]);
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

// Lanes past the row's end read the row's first chunk instead (always there) and drop it afterwards, so the
// loads are unconditional straight-line code. With one branch per load ("valid ? load : 0") the compiler placed
// waits for earlier loads inside the branches, and a wavefront made two or three serial trips to memory.
template <bool kStream>
__device__ __forceinline__ void slab16_global_to_regs(const uint16_t* slab, long L, int nvalid,
                                                      int lane, uint4 (&q)[4]) {
  const int lr = lane >> 4, lp = lane & 15;
  const bool ok = (lp << 3) < nvalid;
  const uint16_t* src = slab + (long)lr * L + (ok ? (lp << 3) : 0);
#pragma unroll
  for (int it = 0; it < 4; ++it) q[it] = load16<kStream>(src + (long)(it * 4) * L);
#pragma unroll
  for (int it = 0; it < 4; ++it) q[it] = ok ? q[it] : zero4();
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

// ---- rows that do not end on a 128-byte line (rows of several spans) --------------------------
// A channel row of L 16-bit steps is 2 L bytes long. When that is not a multiple of 128 the rows start at
// different offsets inside their cache lines, the 256-byte piece a span owns of each row straddles three lines,
// and two of the three are shared with the neighbouring spans: measured, such launches move 0.60-0.69 of the
// peak rate where rows of whole lines move 0.8, whatever the access width or cache policy. Here the wavefronts
// of a workgroup therefore move whole lines instead: for each of its 16 rows, wavefront `sp` of a row moves the two
// lines [16 sp - m, 16 sp + 16 - m) (in 16-byte chunks of the row; m = chunks between the line boundary and the
// row's start, 0..7), drops the first m chunks into the image of the wavefront before it (they are the end of
// that wavefront's span) and finds the last m chunks of its own image delivered by the wavefront after it. Where
// there is no such neighbour in the workgroup -- its last wavefront, a row's last span -- the wavefront moves
// that tail itself (`tail`, at most 7 chunks per row). Rows 4 apart lie 8 L bytes apart, a whole number of lines
// because L is a multiple of 16, so a lane meets the same m in all of its four passes. Images are complete after
// a workgroup barrier; the arithmetic then runs on block-aligned spans exactly as in the plain path, and the
// results are bit-identical to it.
struct LinePlace {
  int c;      // chunk of the row that this lane moves, in each of its passes; may lie outside the row
  bool own;   // the chunk belongs to this wavefront's image (else to the image of the wavefront before it)
  bool here;  // the chunk exists and its image is in this workgroup
};

// The same movement for 16-bit rows (T = uint16_t: 16 chunks per span and row, 4 rows per pass, 4 passes) and
// fp32 rows (T = float: 32 chunks, 2 rows per pass, 8 passes; rows 2 apart lie 8 L bytes apart again).
template <class T>
struct LineGeom {
  static constexpr int kChunks = 8 * (int)sizeof(T);    // 16-byte chunks of one row in a span
  static constexpr int kRowBytes = 16 * kChunks;         // of the LDS image
  static constexpr int kRowsPerPass = 64 / kChunks;
  static constexpr int kPasses = kChan / kRowsPerPass;
  static constexpr int kStepsShift = sizeof(T) == 2 ? 3 : 2;  // log2 of the steps in a chunk
};

__device__ __forceinline__ int chunks_into_line(const void* p) {
  return (int)((reinterpret_cast<uintptr_t>(p) >> 4) & 7);
}

// `rows` = the start of channel row 0 of the span's (batch, head) row; `first_wave` = first wavefront of the workgroup
template <class T>
__device__ __forceinline__ LinePlace line_place(const T* rows, long L, int sp, int lane, bool first_wave) {
  typedef LineGeom<T> G;
  LinePlace p;
  p.c = G::kChunks * sp + (lane & (G::kChunks - 1)) - chunks_into_line(rows + (long)(lane / G::kChunks) * L);
  p.own = p.c >= G::kChunks * sp;
  p.here = p.c >= 0 && p.c < (int)(L >> G::kStepsShift) && (p.own || !first_wave);
  return p;
}

// Lanes without a chunk read the span's first one (always there) and drop it, as in slab16_global_to_regs.
template <bool kStream, class T>
__device__ __forceinline__ void line_global_to_regs(const T* rows, long L, int sp, const LinePlace& p, int lane,
                                                    uint4 (&q)[LineGeom<T>::kPasses]) {
  typedef LineGeom<T> G;
  const T* src = rows + (long)(lane / G::kChunks) * L + ((long)(p.here ? p.c : G::kChunks * sp) << G::kStepsShift);
#pragma unroll
  for (int it = 0; it < G::kPasses; ++it) q[it] = load16<kStream>(src + (long)(it * G::kRowsPerPass) * L);
#pragma unroll
  for (int it = 0; it < G::kPasses; ++it) q[it] = p.here ? q[it] : zero4();
}

// Chunks of the wavefront's own image are always written (zeros past the row's end, which the arithmetic
// relies on); chunks of the image before it only when they exist. `stride` = bytes between two wavefronts' images.
template <class T>
__device__ __forceinline__ void line_regs_to_lds(unsigned char* img, int stride, const LinePlace& p, int lane,
                                                 const uint4 (&q)[LineGeom<T>::kPasses]) {
  typedef LineGeom<T> G;
  if (p.own || p.here) {
    unsigned char* dst = img - (p.own ? 0 : stride);
#pragma unroll
    for (int it = 0; it < G::kPasses; ++it)
      *reinterpret_cast<uint4*>(dst + swz<G::kRowBytes>(it * G::kRowsPerPass + lane / G::kChunks, p.c & (G::kChunks - 1))) = q[it];
  }
}

template <bool kStream, class T>
__device__ __forceinline__ void line_lds_to_global(const unsigned char* img, int stride, T* rows, long L,
                                                   const LinePlace& p, int lane) {
  typedef LineGeom<T> G;
  if (p.here) {
    const unsigned char* src = img - (p.own ? 0 : stride);
#pragma unroll
    for (int it = 0; it < G::kPasses; ++it) {
      const int r = it * G::kRowsPerPass + lane / G::kChunks;
      const uint4 v = *reinterpret_cast<const uint4*>(src + swz<G::kRowBytes>(r, p.c & (G::kChunks - 1)));
      store16<kStream>(rows + (long)r * L + ((long)p.c << G::kStepsShift), v);
    }
  }
}

// The tail: the last m chunks of each row of the wavefront's own image. Lane l takes row l / 4 and, in pass u,
// the chunk (l % 4) + 4 u of that row's tail. Tails are the one place where two workgroups touch the same line, so
// they use plain (cached) accesses: measured 2-3 % of the whole launch against streaming ones. The loads sit in a
// real branch: a lane without a chunk must not ask for some other line instead (a tail is 16 lines per instruction
// as it is, twice what a pass over the span's own lines touches; unconditional loads cost 8 % of the launch).
template <class T>
__device__ __forceinline__ void line_tail_global_to_regs(const T* rows, long L, int sp, int lane, uint4 (&q)[2]) {
  typedef LineGeom<T> G;
  const T* row = rows + (long)(lane >> 2) * L;
  const int m = chunks_into_line(row);
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const int i = (lane & 3) + 4 * u, c = G::kChunks * (sp + 1) - m + i;
    q[u] = zero4();
    if (i < m && c < (int)(L >> G::kStepsShift)) q[u] = load16<false>(row + ((long)c << G::kStepsShift));
  }
}

template <class T>
__device__ __forceinline__ void line_tail_regs_to_lds(unsigned char* img, const T* rows, long L, int lane,
                                                      const uint4 (&q)[2]) {
  typedef LineGeom<T> G;
  const int m = chunks_into_line(rows + (long)(lane >> 2) * L);
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const int i = (lane & 3) + 4 * u;
    if (i < m) *reinterpret_cast<uint4*>(img + swz<G::kRowBytes>(lane >> 2, G::kChunks - m + i)) = q[u];
  }
}

template <class T>
__device__ __forceinline__ void line_tail_lds_to_global(const unsigned char* img, T* rows, long L, int sp, int lane) {
  typedef LineGeom<T> G;
  T* row = rows + (long)(lane >> 2) * L;
  const int m = chunks_into_line(row);
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const int i = (lane & 3) + 4 * u, c = G::kChunks * (sp + 1) - m + i;
    if (i < m && c < (int)(L >> G::kStepsShift)) {
      const uint4 v = *reinterpret_cast<const uint4*>(img + swz<G::kRowBytes>(lane >> 2, G::kChunks - m + i));
      store16<false>(row + ((long)c << G::kStepsShift), v);
    }
  }
}

// ---- rows that do not fill whole spans ---------------------------------------------------------
// A wavefront works on a [16 channel x 128 step] image. With spans cut per row, a row of L <= 64 steps fills at
// most half of one (a launch at L = 64 / 32 / 16 moved 0.63 / 0.39 / 0.21 of the peak rate) and the last span of
// a row of 192 steps is half empty. The kFlat instances of the kernels cut spans from the block sequence of the
// whole tensor instead: span s is blocks [8 s, 8 s + 8) of all rows' blocks in order, so only the tensor's very
// last span can be short. The coefficients and dA of a span are 128 consecutive values (their rows follow each
// other in memory); x, dy, y and dx come from one slab per row the span touches, side by side in the image. The
// arithmetic is unchanged except that no carry crosses the steps where a new row starts.
struct PackLane {
  long off;  // of the lane's chunk in pass 0, in elements from the slab of the span's first row
  bool ok;   // the chunk exists
};

// `nb` = blocks in a row, `b0` = which block of its row the span's first block is, `nvalid` = steps in the span
template <class T>
__device__ __forceinline__ PackLane flat_lane(int lane, int L, int nb, int b0, int nvalid) {
  typedef LineGeom<T> G;
  constexpr int kPerBlockShift = 4 - G::kStepsShift;  // log2 of the chunks in a block
  const int lp = lane & (G::kChunks - 1), lr = lane / G::kChunks;
  const int blk = lp >> kPerBlockShift, part = lp & ((1 << kPerBlockShift) - 1);
  const int q = (b0 + blk) / nb, b = b0 + blk - q * nb;  // rows after the span's first one, block inside that row
  PackLane p;
  p.ok = kTile * blk < nvalid;
  p.off = p.ok ? (long)(q * kChan + lr) * L + kTile * b + (part << G::kStepsShift)
               : (long)lr * L + kTile * b0;  // else the span's first chunk, which is always there
  return p;
}

template <bool kStream, class T>
__device__ __forceinline__ void pack_global_to_regs(const T* first, long L, const PackLane& p,
                                                    uint4 (&q)[LineGeom<T>::kPasses]) {
  typedef LineGeom<T> G;
#pragma unroll
  for (int it = 0; it < G::kPasses; ++it) q[it] = load16<kStream>(first + p.off + (long)(it * G::kRowsPerPass) * L);
#pragma unroll
  for (int it = 0; it < G::kPasses; ++it) q[it] = p.ok ? q[it] : zero4();
}

template <bool kStream, class T>
__device__ __forceinline__ void pack_lds_to_global(const unsigned char* img, T* first, long L, const PackLane& p,
                                                   int lane) {
  typedef LineGeom<T> G;
#pragma unroll
  for (int it = 0; it < G::kPasses; ++it) {
    const uint4 v = *reinterpret_cast<const uint4*>(
        img + swz<G::kRowBytes>(it * G::kRowsPerPass + lane / G::kChunks, lane & (G::kChunks - 1)));
    if (p.ok) store16<kStream>(first + p.off + (long)(it * G::kRowsPerPass) * L, v);
  }
}

// ---- rows of any length and alignment (prompt prefill) --------------------------------------
// The same slab movement for rows whose start is only element-aligned (L not a multiple of 8) and
// whose last elements may stop anywhere. Under-aligned 16-byte accesses are served by the hardware
// but measured 4x slower than aligned ones, so this path moves aligned 32-bit words instead: one
// wave instruction covers one channel row of the span (64 lanes x 4 bytes = 128 steps). A row that
// starts on an odd element is read as the aligned words around it and shifted by 16 bits in
// registers; every word that is read contains at least one element of the row, so nothing outside
// the row's own 4-byte blocks is touched, and stores never write an element that is not the row's.
__device__ __forceinline__ uint4 load16_plain_unaligned(const uint16_t* p) { return load16_plain_unaligned_fwd(p); }

// Where the 16 channel rows of a slab start, which decides how much of the work below is needed:
//   kRowsOnWords    every row starts on a 32-bit word (L even, word-aligned tensors)
//   kRowsAlternate  row r starts on a word for even r and on an odd element for odd r (L odd, word-aligned
//                   tensors): known when the code is generated, so even rows need no shifting at all
//   kRowsAnywhere   found out per row at run time (tensors that start on an odd element)
enum RowStarts : int { kRowsOnWords = 0, kRowsAlternate = 1, kRowsAnywhere = 2 };

template <int kRows>
__device__ __forceinline__ bool row_starts_odd(const uint16_t* row, int r) {  // wave-uniform
  if constexpr (kRows == kRowsOnWords) return false;
  else if constexpr (kRows == kRowsAlternate) return (r & 1) != 0;
  else return ((reinterpret_cast<uintptr_t>(row) >> 1) & 1) != 0;
}

// Step 1, all loads, no dependent work between them (so that a slab's 16 loads -- and those of the
// other slabs -- are in flight together): q[r] = the aligned word `lane` of channel row r, i.e.
// elements (2*lane, 2*lane+1) of the span if the row starts on a word and (2*lane-1, 2*lane) if it
// starts on an odd element. `edge` (lanes 0..15, lane = row) is word 64 of the row, which only rows on
// an odd element need.
template <int kRows>
__device__ __forceinline__ void slab16_global_to_regs_ragged(const uint16_t* slab, long L, int nvalid, int lane,
                                                             uint32_t (&q)[16], uint32_t& edge) {
  // (pointer arithmetic, not an integer round trip: the compiler must keep seeing global memory)
  auto words_of = [&](int r, bool odd, int& last) {
    const uint16_t* row = slab + (long)r * L;
    last = odd ? (nvalid >> 1) : ((nvalid - 1) >> 1);  // last word that holds an element of the row
    return reinterpret_cast<const uint32_t*>(row - (odd ? 1 : 0));
  };
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    int last;
    const uint32_t* words = words_of(r, row_starts_odd<kRows>(slab + (long)r * L, r), last);
    q[r] = __builtin_nontemporal_load(words + min(lane, last));
  }
  edge = 0u;
  // word 64 exists only for a row on an odd element whose span is full (its step 127 sits there): one gather,
  // lane i for row i (kRowsAnywhere) or for the i-th odd row (kRowsAlternate)
  if (kRows != kRowsOnWords && nvalid == kSpan) {  // wave-uniform
    constexpr int kEdgeLanes = kRows == kRowsAlternate ? 8 : 16;
    if (lane < kEdgeLanes) {
      int last;
      const int r = kRows == kRowsAlternate ? 2 * lane + 1 : lane;
      const bool odd = kRows == kRowsAlternate ? true : row_starts_odd<kRowsAnywhere>(slab + (long)r * L, r);
      const uint32_t* words = words_of(r, odd, last);
      edge = words[min(64, last)];
    }
  }
}

// Step 2, in registers: shift the rows that start on an odd element by 16 bits (the upper neighbour
// word comes from the next lane, for lane 63 from `edge`), and zero what lies beyond the row's end.
template <int kRows>
__device__ __forceinline__ void slab16_regs_realign(const uint16_t* slab, long L, int nvalid, int lane,
                                                    uint32_t (&q)[16], uint32_t edge) {
  const int e = lane << 1;
  const uint32_t keep = e + 1 < nvalid ? 0xffffffffu : (e < nvalid ? 0x0000ffffu : 0u);
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    uint32_t w = q[r];
    if (kRows == kRowsAnywhere || (kRows == kRowsAlternate && (r & 1))) {
      const bool odd = row_starts_odd<kRows>(slab + (long)r * L, r);
      // the word held by lane + 1: a whole-wavefront DPP shift (wave_shl:1), no LDS traffic
      const uint32_t up = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)w, 0x130, 0xF, 0xF, false);
      const uint32_t w64 = (uint32_t)__builtin_amdgcn_readlane((int)edge, kRows == kRowsAlternate ? (r >> 1) : r);
      const uint32_t w1 = lane == 63 ? w64 : up;
      w = odd ? (w >> 16) | (w1 << 16) : w;
    }
    q[r] = w & keep;
  }
}

__device__ __forceinline__ void slab16_regs_to_lds_ragged(unsigned char* img, int lane, const uint32_t (&q)[16]) {
#pragma unroll
  for (int r = 0; r < 16; ++r)
    *reinterpret_cast<uint32_t*>(img + swz<256>(r, lane >> 2) + ((lane & 3) << 2)) = q[r];
}

// Image -> global. Whole aligned words first (for a row on an odd element, memory word i holds the
// high half of lane i-1's image word and the low half of lane i's); the one or two elements per row
// that no whole word covers are then written by lanes 0..31 acting as per-row workers.
// `chained` (wave-uniform; kRowsAlternate only): every row ends where the next one starts (the slab is the whole
// of its rows, nvalid == L). The word that holds a row's last element and the next row's first one is then this
// wavefront's alone and lane 0 of the odd row writes it whole: no 2-byte stores are left (each of them costs a
// 32-byte memory transaction: +27 % bytes written at L = 127).
template <int kRows>
__device__ __forceinline__ void slab16_lds_to_global_ragged(const unsigned char* img, uint16_t* slab, long L,
                                                            int nvalid, int lane, bool chained = false) {
  const int e = lane << 1;
  auto image_word = [&](int r, int i) {
    return *reinterpret_cast<const uint32_t*>(img + swz<256>(r, i >> 2) + ((i & 3) << 2));
  };
  const bool link = kRows == kRowsAlternate && chained;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    uint16_t* row = slab + (long)r * L;
    const bool odd = row_starts_odd<kRows>(row, r);  // wave-uniform
    const uint32_t w = image_word(r, lane);
    uint32_t mw = w;
    bool whole = e + 1 < nvalid;  // row on a word: lane covers (e, e+1)
    if (kRows == kRowsAnywhere || (kRows == kRowsAlternate && (r & 1))) {
      // on an odd element: lane covers (e-1, e); lane 0 has no whole word unless the rows are chained, in
      // which case its lower half is the previous row's last element (an even index, L being odd)
      uint32_t below = image_word(r, (lane + 63) & 63);
      if (kRows == kRowsAlternate && r > 0) {
        const uint32_t prev_last = image_word(r - 1, (nvalid - 1) >> 1);
        below = (link && lane == 0) ? (prev_last << 16) : below;
      }
      mw = odd ? (below >> 16) | (w << 16) : w;
      whole = odd ? ((lane > 0 || link) && e < nvalid) : whole;
    }
    if (whole) __builtin_nontemporal_store(mw, reinterpret_cast<uint32_t*>(row + e - (odd ? 1 : 0)));
  }
  if (lane < 32 && !link) {
    const int r = lane & 15;
    uint16_t* row = slab + (long)r * L;
    const bool odd = kRows == kRowsAlternate ? (r & 1) != 0 : row_starts_odd<kRowsAnywhere>(row, r);
    // lanes 0..15: first element of a row on an odd element; lanes 16..31: the last element when no
    // whole word reaches it (even count on an odd start, odd count on a word start)
    const bool first = lane < 16;
    const int t = first ? 0 : nvalid - 1;
    const bool need = first ? (odd && nvalid > 0) : (nvalid > 0 && ((nvalid & 1) != (odd ? 1 : 0)) && !(odd && nvalid == 1));
    if (need) {
      const uint32_t w = image_word(r, t >> 1);
      row[t] = (uint16_t)(t & 1 ? w >> 16 : w);
    }
  }
}

// Same for a [16 x 128] slab of fp32 (512 B per row, 32 chunks of 4 steps).
// Lane l of pass `it` handles channel row 2*it + l/32, chunk l%32.
template <bool kStream>
__device__ __forceinline__ void slab32_global_to_regs(const float* slab, long L, int nvalid, int lane,
                                                      uint4 (&q)[8]) {
  const int lr = lane >> 5, lp = lane & 31;
  const bool ok = (lp << 2) < nvalid;
  const float* src = slab + (long)lr * L + (ok ? (lp << 2) : 0);  // see slab16_global_to_regs
#pragma unroll
  for (int it = 0; it < 8; ++it) q[it] = load16<kStream>(src + (long)(it * 2) * L);
#pragma unroll
  for (int it = 0; it < 8; ++it) q[it] = ok ? q[it] : zero4();
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
  const bool ok = (lane << 1) < nvalid;  // unconditional load, as in slab16_global_to_regs
  const typename C::pair_t w = C::load_pair(arow + (ok ? (lane << 1) : 0));
  return ok ? w : C::zero_pair();
}

// rows of any length: element-aligned address, and the last pair may hold a single coefficient
template <class C>
__device__ __forceinline__ typename C::pair_t coeff_global_to_reg_ragged(const typename C::elem* arow, int nvalid,
                                                                          int lane) {
  const int n = nvalid - (lane << 1);
  return n > 0 ? C::load_pair_ragged(arow + (lane << 1), n) : C::zero_pair();
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

// Spans cut from the tensor's block sequence (see flat_lane): `sp` is which block of its row the span starts with
__device__ __forceinline__ SpanCoord flat_coord(long span, int nb, long total_blocks) {
  SpanCoord c;
  const long first = span * (kSpan / kTile);
  c.row = first / nb;
  c.sp = (int)(first - c.row * nb);
  c.s0 = c.sp * kTile;
  c.nvalid = (int)min((long)(kSpan / kTile), total_blocks - first) * kTile;
  return c;
}

// Workgroup index -> first span. Workgroups are dealt round-robin to the 8 XCDs, each with its own L2. With
// kRemap an XCD instead gets runs of SPEAR_BTP_XCD_GROUP neighbouring workgroups (windows of 8 such runs sweep
// the tensor, so the chip as a whole still walks memory front to back): the workgroup that reads a halo and the
// one that streams the same lines then run on the same L2 close in time, and the halo's 128-byte lines are
// fetched once. Measured on rows of several spans (B=16 H=64 L=8192 / B=64 H=128 L=2048), against plain
// round-robin: runs of 32 gain 1.3 % / 3.6 % in forward and 1.5 % / 1.6 % in backward; runs of 2-8 gain nothing,
// runs of 128 and more lose again in backward, and one contiguous eighth of the tensor per XCD (group 0) gains
// 1.8 % / 0.5 % in forward and loses 2 % in backward. On rows of one span nothing is shared: runs of 32 or 128
// change nothing there (+-0.3 %) and runs of 8 lose 1 %, so those keep the plain order.
#ifndef SPEAR_BTP_XCD_REMAP  // 0: never, 1: kernels on rows of several spans, 2: every kernel
#define SPEAR_BTP_XCD_REMAP 1
#endif
#ifndef SPEAR_BTP_XCD_GROUP  // 0: one contiguous eighth per XCD; G > 0: runs of G neighbouring workgroups per XCD
#define SPEAR_BTP_XCD_GROUP 32
#endif
template <bool kRemap = (SPEAR_BTP_XCD_REMAP == 2)>
__device__ __forceinline__ long first_span_of_workgroup(int waves = kWaves) {
  if constexpr (kRemap) {
    const unsigned n = gridDim.x, b = blockIdx.x;
    unsigned mapped = b;
    if constexpr (SPEAR_BTP_XCD_GROUP > 0) {
      constexpr unsigned kWin = 8u * SPEAR_BTP_XCD_GROUP;
      const unsigned win = b / kWin, in = b - win * kWin;
      if ((win + 1) * kWin <= n) mapped = win * kWin + (in & 7u) * SPEAR_BTP_XCD_GROUP + (in >> 3);
    } else {
      const unsigned per = n >> 3;
      if (b < (per << 3)) mapped = (b & 7u) * per + (b >> 3);
    }
    return (long)mapped * waves;
  } else {
    return (long)blockIdx.x * waves;
  }
}

// How the rows of a launch are cut into spans and moved:
//   kMovePlain  per row, a span's own 256 bytes of each channel row (rows of whole spans: the benchmark shapes; rows
//               of 65..127 steps, whose slabs are one contiguous run each)
//   kMoveLines  per row, whole cache lines (rows of several spans that do not end on a 128-byte line)
//   kMoveFlat   from the tensor's block sequence (rows that leave a span partly empty); Grid::stream then says
//               that no row straddles two spans (L = 16, 32, 64)
// A row of L steps fills L / (128 ceil(L / 128)) of its spans. Flat spans have no empty lanes but move rows the
// plain way: 0.80 of peak on rows of whole lines (L % 64 == 0), 0.75 when the rows lie 64 bytes off the lines
// (L % 64 == 32) and 0.65-0.69 when they lie 32 bytes off. Whole lines keep the per-row cut and reach 0.72-0.78
// on rows that fill their spans well. Measured over 23 lengths from 144 to 1168 at 8 Mi (token, head) units, whole
// lines win from the fill percentages below on (SPEAR_BTP_LINES_MIN_FILL, and ..._HALF for L % 64 == 32), within 3 %.
// Below a span, rows of at most 64 steps go flat (0.73-0.82 against 0.21-0.63) and longer ones stay plain
// (0.73-0.78 against 0.67-0.76 flat).
#ifndef SPEAR_BTP_LINES_MIN_FILL
#define SPEAR_BTP_LINES_MIN_FILL 65
#endif
#ifndef SPEAR_BTP_LINES_MIN_FILL_HALF
#define SPEAR_BTP_LINES_MIN_FILL_HALF 80
#endif
enum Movement : int { kMovePlain = 0, kMoveLines = 1, kMoveFlat = 2 };

inline Movement movement_for(int L) {
  if (L <= 0 || L % kSpan == 0) return kMovePlain;
  if (L < kSpan) return SPEAR_BTP_FLAT_SPANS && 2 * L <= kSpan ? kMoveFlat : kMovePlain;
  const int spans = (L + kSpan - 1) / kSpan;
  const bool off_lines = L % 64 != 0 && SPEAR_BTP_WHOLE_LINES;
  const long min_fill = L % 64 == 32 ? SPEAR_BTP_LINES_MIN_FILL_HALF : SPEAR_BTP_LINES_MIN_FILL;
  if (off_lines && 100L * L >= min_fill * spans * kSpan) return kMoveLines;
  return SPEAR_BTP_FLAT_SPANS ? kMoveFlat : (off_lines ? kMoveLines : kMovePlain);
}

struct Grid {
  int spans_per_row;
  long total_spans;
  bool stream;     // kStreamIn of the kernels
  bool lines;      // rows of several spans that do not end on a 128-byte line: kLines of the kernels that have it
  bool flat;       // spans cut from the tensor's block sequence (kFlat of the kernels that have it); then
                   // spans_per_row holds the blocks in a row and total_spans the blocks in the tensor
  int waves;       // wavefronts per workgroup
  unsigned blocks;
};

// Rows that fit one span are read exactly once and can be streamed; longer rows are re-read by
// neighbouring spans' halo loads, so their lines should stay in L2. `waves_long` is the workgroup
// size (in wavefronts) the calling kernel family uses for those longer rows.
inline Grid make_grid(long rows, int L, int waves_long = kWaves, int waves_short = kWaves) {
  Grid g;
  g.spans_per_row = (L + kSpan - 1) / kSpan;
  g.total_spans = rows * g.spans_per_row;
  g.stream = g.spans_per_row == 1;  // template argument kStreamIn of the kernels: rows of a single span
  g.lines = movement_for(L) == kMoveLines;
  g.flat = false;
  g.waves = g.stream ? waves_short : waves_long;
  g.blocks = (unsigned)((g.total_spans + g.waves - 1) / g.waves);
  return g;
}

inline bool stream_inputs(const Grid& g) { return g.stream; }

// The grid of the kFlat instances for the same rows.
inline Grid flat_grid(long rows, int L, int waves_long = kWaves, int waves_short = kWaves) {
  Grid g;
  g.spans_per_row = L / kTile;
  g.total_spans = rows * g.spans_per_row;
  g.stream = (kSpan / kTile) % g.spans_per_row == 0;  // no row straddles two spans
  g.lines = false;
  g.flat = true;
  g.waves = g.stream ? waves_short : waves_long;
  const long spans = (g.total_spans + kSpan / kTile - 1) / (kSpan / kTile);
  g.blocks = (unsigned)((spans + g.waves - 1) / g.waves);
  return g;
}

// Whether a kernel instance reads its slabs with non-temporal loads, from the knob above and from
// whether its rows are single spans (the kernels' template argument).
constexpr bool nt_loads(bool single_span) {
  return SPEAR_BTP_STREAM_LOADS == 1 || (SPEAR_BTP_STREAM_LOADS == 2 && single_span);
}

}  // namespace spear_btp
