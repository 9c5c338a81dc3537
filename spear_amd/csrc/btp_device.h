// Device-side building blocks shared by the gfx950 BTP kernels: element packing, wavefront-level
// LDS synchronisation, DPP lane exchanges and the 16-lane transposing reduction.
//
// Roles they take over from the reference's helpers (paths relative to the reference repository):
//   PackedType / pack_and_convert      csrc/btp/btp-backwards.cu:145-162  -> Elt<...>::pack2
//   warp_prefix_sum / warp_suffix_sum  csrc/btp/btp-backwards.cu:113-142  -> not needed: decay
//                                      products are carried by in-lane recurrences
//   safe_multiply (0*Inf -> 0)         csrc/btp/btp_common.h:23-33        -> not needed: nothing
//                                      here takes log or reciprocal of a coefficient
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace spear_btp {

constexpr int kTile = 16;   // time steps per block (reference: BL / BLK)
constexpr int kChan = 16;   // channels per head   (reference: DH)
constexpr int kSpan = 128;  // time steps one wavefront owns per pass: 8 blocks, 256 B per bf16 row
#ifndef SPEAR_BTP_WAVES_PER_WG
#define SPEAR_BTP_WAVES_PER_WG 4
#endif
constexpr int kWaves = SPEAR_BTP_WAVES_PER_WG;  // wavefronts per workgroup; each works on its own span
#ifndef SPEAR_BTP_WAVES_PER_WG_LONG
#define SPEAR_BTP_WAVES_PER_WG_LONG 8
#endif
// Rows of several spans, backward recurrence kernel: neighbouring spans of a workgroup hand their
// carries over through LDS, so a larger workgroup means fewer halo reads (measured: -3 %).
constexpr int kWavesLong = SPEAR_BTP_WAVES_PER_WG_LONG;

// Coefficients at or below this are treated as exactly zero, as in the reference kernels
// (csrc/btp/btp-forward.cu:179, csrc/btp/btp-backwards.cu:280-286); this also maps negative
// (out-of-domain) inputs to zero.
constexpr float kCoeffFloor = 1e-9f;

typedef float floatx2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 halfx2_t __attribute__((ext_vector_type(2)));

// ---- element traits: two 16-bit storage values per 32-bit word, low half first -------------
struct Bf16 {
  static __device__ __forceinline__ float lo(uint32_t w) { return __uint_as_float(w << 16); }
  static __device__ __forceinline__ float hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }
  // round-to-nearest-even; on gfx950 this is a single v_cvt_pk_bf16_f32
  static __device__ __forceinline__ uint32_t pack2(float a, float b) {
    floatx2_t f = {a, b};
    bf16x2_t h = __builtin_convertvector(f, bf16x2_t);
    return __builtin_bit_cast(uint32_t, h);
  }
};

struct Fp16 {
  static __device__ __forceinline__ float lo(uint32_t w) {
    return (float)__builtin_bit_cast(halfx2_t, w)[0];
  }
  static __device__ __forceinline__ float hi(uint32_t w) {
    return (float)__builtin_bit_cast(halfx2_t, w)[1];
  }
  // Round-to-nearest-even of the fp32 values. The empty asm keeps the conversion apart from the arithmetic before it:
  // folded into a mixed-precision FMA (v_fma_mixlo_f16) the value would be rounded once from the exact sum, which
  // differs from the rounded fp32 result where that lies exactly between two fp16 values, and the compiler folds
  // in some kernel instances and not in others.
  static __device__ __forceinline__ uint32_t pack2(float a, float b) {
    asm("" : "+v"(a), "+v"(b));
    halfx2_t h = {(_Float16)a, (_Float16)b};
    return __builtin_bit_cast(uint32_t, h);
  }
};

template <class E>
__device__ __forceinline__ float clamp_coeff(float a) {
  return a > kCoeffFloor ? a : 0.0f;
}

template <class E>
__device__ __forceinline__ void unpack8(const uint4& q, float* out) {
  out[0] = E::lo(q.x); out[1] = E::hi(q.x);
  out[2] = E::lo(q.y); out[3] = E::hi(q.y);
  out[4] = E::lo(q.z); out[5] = E::hi(q.z);
  out[6] = E::lo(q.w); out[7] = E::hi(q.w);
}

template <class E>
__device__ __forceinline__ uint4 pack8(const float* v) {
  uint4 q;
  q.x = E::pack2(v[0], v[1]);
  q.y = E::pack2(v[2], v[3]);
  q.z = E::pack2(v[4], v[5]);
  q.w = E::pack2(v[6], v[7]);
  return q;
}

// ---- wavefront-private LDS hand-over --------------------------------------------------------
// A wavefront's DS instructions execute in program order, so data written by one lane is visible
// to a later read by another lane of the same wavefront without an s_barrier. The fences keep
// the compiler from moving LDS accesses across the hand-over point.
__device__ __forceinline__ void wave_lds_handover() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// ---- lane exchanges -------------------------------------------------------------------------
// Value of `v` held by lane (lane + delta) mod 64.
__device__ __forceinline__ float lane_rotate(float v, int lane, int delta) {
  return __int_as_float(__builtin_amdgcn_ds_bpermute(((lane + delta) & 63) << 2, __float_as_int(v)));
}

// Value of `v` held by the lane whose index differs in bit `Bit` (within a row of 16 lanes).
template <int Bit>
__device__ __forceinline__ float row_xor(float v) {
  const int s = __float_as_int(v);
  if constexpr (Bit == 8) {
    return __int_as_float(__builtin_amdgcn_mov_dpp(s, 0x128 /* row_ror:8 */, 0xF, 0xF, true));
  } else if constexpr (Bit == 4) {
    // lanes 4..7, 12..15 take from lane-4; lanes 0..3, 8..11 take from lane+4
    int t = __builtin_amdgcn_update_dpp(0, s, 0x114 /* row_shr:4 */, 0xF, 0xA, false);
    t = __builtin_amdgcn_update_dpp(t, s, 0x104 /* row_shl:4 */, 0xF, 0x5, false);
    return __int_as_float(t);
  } else if constexpr (Bit == 2) {
    return __int_as_float(__builtin_amdgcn_mov_dpp(s, 0x4E /* quad_perm:[2,3,0,1] */, 0xF, 0xF, true));
  } else {
    static_assert(Bit == 1, "row_xor: Bit must be 8, 4, 2 or 1");
    return __int_as_float(__builtin_amdgcn_mov_dpp(s, 0xB1 /* quad_perm:[1,0,3,2] */, 0xF, 0xF, true));
  }
}

// Each lane of a 16-lane row holds e[0..15]. Returns, in the lane with index d within its row,
// sum over the row's 16 lanes of e[d]: a reduction over lanes and a transpose in one butterfly
// (8 + 4 + 2 + 1 exchanges instead of 16 full reductions).
__device__ __forceinline__ float row_transpose_reduce(const float (&e)[16], int d) {
  float f8[8], f4[4], f2[2];
  const bool b8 = d & 8, b4 = d & 4, b2 = d & 2, b1 = d & 1;
#pragma unroll
  for (int t = 0; t < 8; ++t) {
    const float keep = b8 ? e[t + 8] : e[t];
    const float send = b8 ? e[t] : e[t + 8];
    f8[t] = keep + row_xor<8>(send);
  }
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const float keep = b4 ? f8[t + 4] : f8[t];
    const float send = b4 ? f8[t] : f8[t + 4];
    f4[t] = keep + row_xor<4>(send);
  }
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    const float keep = b2 ? f4[t + 2] : f4[t];
    const float send = b2 ? f4[t] : f4[t + 2];
    f2[t] = keep + row_xor<2>(send);
  }
  const float keep = b1 ? f2[1] : f2[0];
  const float send = b1 ? f2[0] : f2[1];
  return keep + row_xor<1>(send);
}

}  // namespace spear_btp
