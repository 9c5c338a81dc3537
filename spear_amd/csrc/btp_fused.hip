// Fused Phalanx mixing kernel for gfx950 (MI355X), forward: everything the layer does between its
// input projections and its output projection, in the projections' own [B, L, features] layout.
//
//     A = sigmoid(a_logit)            [B, L, H]          decay per head and step
//     X = sigmoid(b_logit) * v        [B, L, H*16]       gated input (b, c may have fewer, shared heads)
//     h = btp(A, X)   (k = 2)                            one-hop block recurrence over time
//     out = h * c + v                 [B, L, H*16]
//
// In the reference these are separate PyTorch ops around the BTP kernel
// (spear/nn/phalanx/swr.py:166-221 for the gates, :311-327 for `y * C + V`, the permute and the
// `.contiguous()` transposes hidden in spear/ops/btp/interface.py:186-187): about twenty passes
// over [B, L, H*16]-sized tensors. Here each operand is read once and the result written once.
//
// Layout and work split. Features are the contiguous axis, time is strided, so a lane owns
// features and walks through time: one wavefront owns 64 features (4 heads) of one batch row and
// advances 32 steps (two 16-step blocks) per iteration. Lane (j, p) = (lane / 32, lane % 32) owns
// the feature pair p (4 bytes) of block 2s + j. A wave-level load or store therefore touches two
// full 128-byte lines (steps t and t + 16 of the same 64 features); there is no LDS staging of the
// big operands at all. A word's register is refilled with the next iteration's word as soon as it
// has been consumed, which keeps up to 12 KiB per wavefront in flight.
//
// Per block a lane runs the same two fp32 recurrences as the stand-alone forward kernel: a
// zero-started one whose terminal value is the carry for the next block, and one started from the
// incoming carry that produces the outputs. The carry crosses between the two lane halves with one
// ds_bpermute per feature (block 2s -> 2s+1 inside an iteration, block 2s+1 -> 2s+2 across
// iterations), so a row of any length is processed without halo re-reads.
// sigmoid(a_logit) is computed once per (step, head) by 32 lanes and handed to the others through a
// 512-byte LDS tile.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "btp_device.h"
#include "btp_launch.h"

namespace spear_btp {

namespace {

__device__ __forceinline__ float fast_sigmoid(float z) {
  return __builtin_amdgcn_rcpf(1.0f + __expf(-z));
}

constexpr int kFusedSteps = 32;  // time steps per iteration: two blocks, one per lane half

template <class E>
__global__ __launch_bounds__(64 * kWaves) void phalanx_mix_fwd_kernel(
    const uint16_t* __restrict__ a_logit, const uint16_t* __restrict__ b_logit, const uint16_t* __restrict__ c_in,
    const uint16_t* __restrict__ v_in, uint16_t* __restrict__ out, int L, int H, int kv_groups, long total_waves) {
  __shared__ __align__(16) float a_tile[kWaves][4 * kFusedSteps];  // [head in quad][step] decay, fp32

  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const long w = (long)blockIdx.x * kWaves + wave;
  if (w >= total_waves) return;
  const int quads = H >> 2;
  const long brow = w / quads;
  const int hq = (int)(w - brow * quads);

  const int j = lane >> 5, p = lane & 31;
  const int head_local = p >> 3;
  const int head = 4 * hq + head_local;
  const int d0 = (p & 7) << 1;
  const int F = H * kChan;
  const int Fkv = (H / kv_groups) * kChan;
  // Buffer addressing: a wave-uniform resource per operand (base of this batch row), a wave-uniform
  // SGPR offset for the time step and one constant per-lane byte offset for (feature pair, lane
  // half). No per-access vector address arithmetic is left.
  const int v_stride = 2 * F, kv_stride = 2 * Fkv;  // bytes per time step
  constexpr int kRsrcFlags = 0x00020000;            // raw 32-bit buffer, gfx9 encoding
  const __amdgpu_buffer_rsrc_t rv =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(v_in + brow * L * F), 0, L * v_stride, kRsrcFlags);
  const __amdgpu_buffer_rsrc_t ro = __builtin_amdgcn_make_buffer_rsrc(out + brow * L * F, 0, L * v_stride, kRsrcFlags);
  const __amdgpu_buffer_rsrc_t rb =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(b_logit + brow * L * Fkv), 0, L * kv_stride, kRsrcFlags);
  const __amdgpu_buffer_rsrc_t rc =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(c_in + brow * L * Fkv), 0, L * kv_stride, kRsrcFlags);
  const uint16_t* arow = a_logit + brow * L * H + 4 * hq;
  const int v_feat = 2 * (head * kChan + d0), kv_feat = 2 * ((head / kv_groups) * kChan + d0);
  const int v_lane = v_feat + 16 * j * v_stride, kv_lane = kv_feat + 16 * j * kv_stride;
  float* at = a_tile[wave];
  constexpr int kNt = 2;  // non-temporal: every word is touched once

  auto gate_row = [&](int t0) -> uint2 {
    const int t = min(t0 + (lane & (kFusedSteps - 1)), L - 1);  // clamped: rows past the end are never used
    return *reinterpret_cast<const uint2*>(arow + (long)t * H);
  };

  // Rolling buffers: slot r always holds the words of step r of the lane's current block; as soon
  // as a word has been consumed, the same slot is refilled with the next iteration's word.
  // All loads are in bounds by construction: where a lane's block does not exist (odd number of
  // blocks: the upper lane half in the last iteration; and the refill after the last iteration)
  // it re-reads rows that do exist, and what it computes from them is never stored and never
  // reaches a lane whose block exists.
  uint32_t bw[16], cw[16], vw[16];
  {
    const bool upper = kTile < L;
    const int ov = upper ? v_lane : v_feat, okv = upper ? kv_lane : kv_feat;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      bw[r] = __builtin_amdgcn_raw_buffer_load_b32(rb, okv, r * kv_stride, kNt);
      vw[r] = __builtin_amdgcn_raw_buffer_load_b32(rv, ov, r * v_stride, kNt);
      cw[r] = __builtin_amdgcn_raw_buffer_load_b32(rc, okv, r * kv_stride, kNt);
    }
  }
  uint2 araw = gate_row(0);
  float saved0 = 0.0f, saved1 = 0.0f;  // terminal local state of the block before block 2s (lanes j = 0)

  for (int t0 = 0; t0 < L; t0 += kFusedSteps) {
    const bool ok = t0 + 16 * j < L;  // this lane's block exists
    // rows the refills come from (wave-uniform), and whether the upper lane half has a block there
    const int tn = (t0 + kFusedSteps < L) ? t0 + kFusedSteps : t0;
    const bool upper = tn + kTile < L;
    const int nv = upper ? v_lane : v_feat, nkv = upper ? kv_lane : kv_feat;

    // decay of the 32 steps x 4 heads of this iteration: lane t computes row t
    if (lane < kFusedSteps) {
      at[0 * kFusedSteps + lane] = clamp_coeff<E>(fast_sigmoid(E::lo(araw.x)));
      at[1 * kFusedSteps + lane] = clamp_coeff<E>(fast_sigmoid(E::hi(araw.x)));
      at[2 * kFusedSteps + lane] = clamp_coeff<E>(fast_sigmoid(E::lo(araw.y)));
      at[3 * kFusedSteps + lane] = clamp_coeff<E>(fast_sigmoid(E::hi(araw.y)));
    }
    araw = gate_row(t0 + kFusedSteps);
    wave_lds_handover();
    float a[16];
#pragma unroll
    for (int c4 = 0; c4 < 4; ++c4) {
      const float4 q = *reinterpret_cast<const float4*>(at + head_local * kFusedSteps + 16 * j + 4 * c4);
      a[4 * c4 + 0] = q.x; a[4 * c4 + 1] = q.y; a[4 * c4 + 2] = q.z; a[4 * c4 + 3] = q.w;
    }
    wave_lds_handover();  // the tile may be overwritten by the next iteration from here on

    // pass 1: gated inputs and the zero-started recurrence (its terminal value is the next carry)
    float x0[16], x1[16];
    float l0 = 0.0f, l1 = 0.0f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      x0[r] = fast_sigmoid(E::lo(bw[r])) * E::lo(vw[r]);
      x1[r] = fast_sigmoid(E::hi(bw[r])) * E::hi(vw[r]);
      bw[r] = __builtin_amdgcn_raw_buffer_load_b32(rb, nkv, (tn + r) * kv_stride, kNt);
      l0 = fmaf(a[r], l0, x0[r]);
      l1 = fmaf(a[r], l1, x1[r]);
    }
    // carries: lanes j = 1 take this iteration's block 2s terminal from lanes j = 0; lanes j = 0 use
    // the terminal of block 2s - 1 kept from the previous iteration and keep block 2s + 1's for the next
    const float r0 = lane_rotate(l0, lane, 32), r1 = lane_rotate(l1, lane, 32);
    float y0 = j ? r0 : saved0, y1 = j ? r1 : saved1;
    saved0 = r0;
    saved1 = r1;

    // pass 2: the carry-started recurrence, the output mix, and the refill of c / v.
    // A lane without a block stores at an offset beyond the resource, which the buffer unit drops.
    const int so = ok ? v_lane : 0x7ffffff0;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      y0 = fmaf(a[r], y0, x0[r]);
      y1 = fmaf(a[r], y1, x1[r]);
      const uint32_t ow = E::pack2(fmaf(y0, E::lo(cw[r]), E::lo(vw[r])), fmaf(y1, E::hi(cw[r]), E::hi(vw[r])));
      cw[r] = __builtin_amdgcn_raw_buffer_load_b32(rc, nkv, (tn + r) * kv_stride, kNt);
      vw[r] = __builtin_amdgcn_raw_buffer_load_b32(rv, nv, (tn + r) * v_stride, kNt);
      __builtin_amdgcn_raw_buffer_store_b32(ow, ro, so, (t0 + r) * v_stride, kNt);
    }
  }
}

}  // namespace

hipError_t fused_mix_forward(const MixArgs& p, hipStream_t s) {
  const long total = (long)p.B * (p.H / 4);
  const unsigned blocks = (unsigned)((total + kWaves - 1) / kWaves);
  if (p.dtype == kBf16) {
    hipLaunchKernelGGL((phalanx_mix_fwd_kernel<Bf16>), dim3(blocks), dim3(64 * kWaves), 0, s,
                       static_cast<const uint16_t*>(p.a_logit), static_cast<const uint16_t*>(p.b_logit),
                       static_cast<const uint16_t*>(p.c), static_cast<const uint16_t*>(p.v),
                       static_cast<uint16_t*>(p.out), p.L, p.H, p.kv_groups, total);
  } else {
    hipLaunchKernelGGL((phalanx_mix_fwd_kernel<Fp16>), dim3(blocks), dim3(64 * kWaves), 0, s,
                       static_cast<const uint16_t*>(p.a_logit), static_cast<const uint16_t*>(p.b_logit),
                       static_cast<const uint16_t*>(p.c), static_cast<const uint16_t*>(p.v),
                       static_cast<uint16_t*>(p.out), p.L, p.H, p.kv_groups, total);
  }
  return hipGetLastError();
}

}  // namespace spear_btp
