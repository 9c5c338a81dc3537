// MFMA tile kernel for the Block Two-Pass operator on gfx950 (MI355X), bf16 and fp16: the formulation the
// reference uses on sm90 -- materialise the block's decay matrix, multiply it with the activation
// tile on the matrix cores (csrc/btp/btp-forward.cu:214-274, WarpMma in csrc/btp/btp_common.h:35-45)
// -- rebuilt around v_mfma_f32_16x16x32_bf16 / _f16. Selected with SPEAR_BTP_PATH_MFMA; the default path
// is the exact-fp32 recurrence (btp_scan.hip), which is at least as fast (both are HBM-bound) and
// does not round the decay matrix to bf16.
//
// One MFMA per 16-step block i covers BOTH passes of the reference algorithm. With K = 32 running
// over the previous block's 16 steps and the block's own 16 steps,
//     Y_i [16 steps x 16 channels] = [ C_i | L_i ] [16 x 32]  *  [ X_{i-1} ; X_i ] [32 x 16]
//     L_i[r][c] = prod_{j=c+1..r} a_j  (c <= r, else 0)          block-local pass
//     C_i[r][c] = (prod_{j=0..r} a_j) (prod_{j=c+1..15} a^{prev}_j)  one-hop carry, rank 1
// i.e. entry(r, t') = prod_{j=t'+1..r} a_j over the concatenated coefficient sequence, t' = -16..15.
// The carry never exists as a separate vector (the reference ships it between warps through shared
// memory / DSMEM, btp-forward.cu:287-424).
//
// Operand layouts of v_mfma_f32_16x16x32_bf16 (lane = 16 q + n):
//     A: lane holds row m = n, k = 8q..8q+7        -> decay entries, built in registers
//     B: lane holds column n,  k = 8q..8q+7        -> x[channel n][8 consecutive steps]: one 16-byte
//                                                    chunk of the swizzled LDS image, no shuffling
//     D: lane holds column n,  rows 4q..4q+3       -> y[channel n][4 consecutive steps]: one 8-byte
//                                                    (bf16) or 16-byte (fp32) LDS write
// A lane's 8 decay entries are one row segment; they are produced right to left by a running
// product, entry(r, t'-1) = entry(r, t') * a_t', started from a per-row prefix product that comes
// from a 3-step DPP scan inside 8-lane halves plus two v_readlane broadcasts.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "btp_device.h"
#include "btp_launch.h"
#include "btp_staging.h"

namespace spear_btp {

namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float floatx4_t __attribute__((ext_vector_type(4)));

// v from lane (n - Shift) of the same 16-lane row; lanes without a source get `fill`.
template <int Shift>
__device__ __forceinline__ float row_shift_right(float v, float fill) {
  return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(fill), __float_as_int(v), 0x110 + Shift, 0xF, 0xF,
                                                    false));
}

// W[n] = prod of a over the lanes of n's 8-lane half up to and including n (n = lane % 16).
__device__ __forceinline__ float half_row_prefix_product(float a_n, int n) {
  const int n8 = n & 7;
  float w = a_n;
  float t = row_shift_right<1>(w, 1.0f);
  w = (n8 >= 1) ? w * t : w;
  t = row_shift_right<2>(w, 1.0f);
  w = (n8 >= 2) ? w * t : w;
  t = row_shift_right<4>(w, 1.0f);
  w = (n8 >= 4) ? w * t : w;
  return w;
}

__device__ __forceinline__ float lane_broadcast(float v, int src_lane) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), src_lane));
}

typedef _Float16 halfx8_t __attribute__((ext_vector_type(8)));

// One 16x16x32 matrix instruction on eight 16-bit elements per lane and operand (raw bits), fp32 accumulate.
template <class E>
__device__ __forceinline__ floatx4_t mfma_16x16x32(uint4 a, uint4 b, floatx4_t acc) {
  if constexpr (std::is_same<E, Bf16>::value)
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), acc,
                                                   0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(halfx8_t, a), __builtin_bit_cast(halfx8_t, b), acc,
                                                  0, 0, 0);
}

template <class E, class OutT, bool kStreamIn>
__global__ __launch_bounds__(64 * kWaves) void btp_fwd_mfma_kernel(const uint16_t* __restrict__ coeff,
                                                                   const uint16_t* __restrict__ x,
                                                                   OutT* __restrict__ y, int L, int spans_per_row,
                                                                   long total_spans, int k) {
  constexpr bool kOutF32 = std::is_same<OutT, float>::value;
  constexpr bool kStreamOut = SPEAR_BTP_STREAM_STORES == 1;
  constexpr int kOutBytes = kOutF32 ? 8192 : 4096;
  // per wavefront: x image | x halo (16 rows x 32 B) | output image | coefficients (16 halo + 128)
  constexpr int kWaveBytes = 4096 + 512 + kOutBytes + (kTile + kSpan) * 4;
  __shared__ __align__(16) unsigned char lds[kWaves][kWaveBytes];

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const long span = first_span_of_workgroup() + wave;
  if (span >= total_spans) return;
  const SpanCoord sc = span_coord(span, spans_per_row, L);

  unsigned char* img_x = lds[wave];
  unsigned char* halo_x = img_x + 4096;
  unsigned char* img_y = halo_x + 512;
  float* a_ext = reinterpret_cast<float*>(img_y + kOutBytes);  // a_ext[16 + t] = a at span step t

  const uint16_t* xslab = x + (sc.row * kChan) * (long)L + sc.s0;
  const uint16_t* arow = coeff + sc.row * (long)L + sc.s0;
  const int q = lane >> 4, n = lane & 15;

  // ---- global -> LDS
  uint4 xin[4];
  slab16_global_to_regs<kStreamIn>(xslab, L, sc.nvalid, lane, xin);
  const uint32_t ain = coeff_global_to_reg<LinCoeff<E>>(arow, sc.nvalid, lane);
  const bool halo = (k == 2) && (sc.sp > 0);  // wave-uniform
  uint4 hx = zero4();
  uint32_t ha = 0u;
  if (halo) {
    if (lane < 32) hx = *reinterpret_cast<const uint4*>(xslab + (long)(lane >> 1) * L - kTile + ((lane & 1) << 3));
    if (lane < 8) ha = *reinterpret_cast<const uint32_t*>(arow - kTile + (lane << 1));
  }
  slab16_regs_to_lds(img_x, lane, xin);
  if (lane < 32) *reinterpret_cast<uint4*>(halo_x + (lane >> 1) * 32 + ((lane & 1) << 4)) = hx;
  {
    float2 f;
    f.x = clamp_coeff<E>(E::lo(ain));
    f.y = clamp_coeff<E>(E::hi(ain));
    *reinterpret_cast<float2*>(a_ext + kTile + (lane << 1)) = f;
    if (lane < 8) {
      f.x = clamp_coeff<E>(E::lo(ha));
      f.y = clamp_coeff<E>(E::hi(ha));
      *reinterpret_cast<float2*>(a_ext + (lane << 1)) = f;
    }
  }
  wave_lds_handover();

  // product of the last 8 coefficients of the block before the span (only meaningful with a halo)
  float g_prev = lane_broadcast(half_row_prefix_product(a_ext[n], n), 15);

#pragma unroll
  for (int i = 0; i < kSpan / kTile; ++i) {
    // per-row prefix products of this block (identical in the four lane groups)
    const float w = half_row_prefix_product(a_ext[kTile + kTile * i + n], n);
    const float s7 = lane_broadcast(w, 7), s15 = lane_broadcast(w, 15);
    const float p = (n >= 8) ? w * s7 : w;  // prod_{j=0..n} a_j

    // start value = entry(n, 8q-9), the lane's rightmost column; 1 where the row is still masked
    const bool cross = (k == 2) && (i > 0 || halo);
    float val;
    if (q == 0) val = cross ? g_prev * p : 0.0f;
    else if (q == 1) val = cross ? p : 0.0f;
    else if (q == 2) val = (n >= 8) ? w : 1.0f;
    else val = 1.0f;

    const float4 a_lo = *reinterpret_cast<const float4*>(a_ext + kTile * i + 8 * q);
    const float4 a_hi = *reinterpret_cast<const float4*>(a_ext + kTile * i + 8 * q + 4);
    const float av[8] = {a_lo.x, a_lo.y, a_lo.z, a_lo.w, a_hi.x, a_hi.y, a_hi.z, a_hi.w};
    float e[8];
#pragma unroll
    for (int jj = 7; jj >= 0; --jj) {
      const bool above = (8 * q - 16 + jj) > n;  // column is later than the row: structural zero
      e[jj] = above ? 0.0f : val;
      val *= above ? 1.0f : av[jj];
    }
    const uint4 A = pack8<E>(e);

    // B: steps 16(i-1) + 8q .. +7 of channel n
    const int cidx = 2 * i - 2 + q;
    uint4 braw;
    if (i == 0) {
      braw = (q < 2) ? *reinterpret_cast<const uint4*>(halo_x + n * 32 + (q << 4))
                     : *reinterpret_cast<const uint4*>(img_x + swz<256>(n, cidx));
    } else {
      braw = *reinterpret_cast<const uint4*>(img_x + swz<256>(n, cidx));
    }
    floatx4_t acc = {0.0f, 0.0f, 0.0f, 0.0f};
    acc = mfma_16x16x32<E>(A, braw, acc);

    // D: y[channel n][16 i + 4 q .. + 3]
    if constexpr (kOutF32) {
      *reinterpret_cast<float4*>(img_y + swz<512>(n, 4 * i + q)) = make_float4(acc[0], acc[1], acc[2], acc[3]);
    } else {
      uint2 o;
      o.x = E::pack2(acc[0], acc[1]);
      o.y = E::pack2(acc[2], acc[3]);
      *reinterpret_cast<uint2*>(img_y + swz<256>(n, 2 * i + (q >> 1)) + ((q & 1) << 3)) = o;
    }
    g_prev = s15;
  }

  wave_lds_handover();
  if constexpr (kOutF32) {
    slab32_lds_to_global<kStreamOut>(img_y, reinterpret_cast<float*>(y) + (sc.row * kChan) * (long)L + sc.s0, L,
                                     sc.nvalid, lane);
  } else {
    slab16_lds_to_global<kStreamOut>(img_y, reinterpret_cast<uint16_t*>(y) + (sc.row * kChan) * (long)L + sc.s0, L,
                                     sc.nvalid, lane);
  }
}

template <class E, class OutT, bool kStreamIn>
void launch_fwd_mfma(const FwdArgs& p, const Grid& g, hipStream_t s) {
  hipLaunchKernelGGL((btp_fwd_mfma_kernel<E, OutT, kStreamIn>), dim3(g.blocks), dim3(64 * kWaves), 0, s,
                     static_cast<const uint16_t*>(p.coeff), static_cast<const uint16_t*>(p.x),
                     static_cast<OutT*>(p.y), p.L, g.spans_per_row, g.total_spans, p.k);
}

}  // namespace

hipError_t mfma_forward(const FwdArgs& p, hipStream_t s) {
  const Grid g = make_grid((long)p.B * p.H, p.L);
  const bool st = stream_inputs(g);
  auto by_out = [&](auto e) {
    using E = decltype(e);
    if (p.out_dtype == kF32) {
      if (st) launch_fwd_mfma<E, float, true>(p, g, s);
      else launch_fwd_mfma<E, float, false>(p, g, s);
    } else {
      if (st) launch_fwd_mfma<E, uint16_t, true>(p, g, s);
      else launch_fwd_mfma<E, uint16_t, false>(p, g, s);
    }
  };
  if (p.in_dtype == kBf16) by_out(Bf16{});
  else by_out(Fp16{});
  return hipGetLastError();
}

}  // namespace spear_btp
