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
// features and walks through time: one wavefront owns 128 features (8 heads) of one batch row,
// lane p the feature pair p (4 bytes), and advances one 16-step block per iteration. A wave-level
// load or store is one contiguous 256-byte run, and the four wavefronts of a workgroup cover 512
// consecutive features of the same time step, so a workgroup walks whole 1-KiB rows; there is no
// LDS staging of the big operands at all. Two register sets alternate: the next block's 48 words per
// lane are requested before the current block is processed (12 KiB per wavefront in flight). Addressing
// uses buffer instructions: a wave-uniform resource per operand, an SGPR offset for the time step
// and one constant per-lane byte offset, so no per-access vector address arithmetic is left.
//
// Per block a lane runs the same two fp32 recurrences as the stand-alone forward kernel: a
// zero-started one whose terminal value is the carry for the next block, and one started from the
// incoming carry that produces the outputs. Because a lane walks through time, the carry simply
// stays in the lane's registers: a row of any length is processed without halo re-reads.
// sigmoid(a_logit) is computed once per (step, head) -- two per lane -- and handed to the lanes
// that need it through a 640-byte LDS tile.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdlib.h>

#include "btp_device.h"
#include "btp_launch.h"

namespace spear_btp {

namespace {

__device__ __forceinline__ float fast_sigmoid(float z) {
  return __builtin_amdgcn_rcpf(1.0f + __expf(-z));
}

constexpr int kHeadsPerWave = 8;
constexpr int kGateRow = 20;  // floats per head in the decay tile: 16 steps + 4 of padding (bank spread)

template <class E>
__global__ __launch_bounds__(64 * kWaves) void phalanx_mix_fwd_kernel(
    const uint16_t* __restrict__ a_logit, const uint16_t* __restrict__ b_logit, const uint16_t* __restrict__ c_in,
    const uint16_t* __restrict__ v_in, uint16_t* __restrict__ out, int L, int H, int kv_groups, int chunk_steps,
    int chunks, long total_waves) {
  __shared__ __align__(16) float a_tile[kWaves][kHeadsPerWave * kGateRow];  // [head][step] decay, fp32

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const long w = (long)blockIdx.x * kWaves + wave;
  if (w >= total_waves) return;
  // wavefront -> (batch row, time chunk, group of 8 heads); heads vary fastest so that the four
  // wavefronts of a workgroup read neighbouring features of the same time steps
  const int octs = (H + kHeadsPerWave - 1) / kHeadsPerWave;
  const long bc = w / octs;
  const int ho = (int)(w - bc * octs) * kHeadsPerWave;  // first head of this wavefront
  const long brow = bc / chunks;
  const int t_begin = (int)(bc - brow * chunks) * chunk_steps;
  const int t_end = min(L, t_begin + chunk_steps);
  // A chunk that does not start the row first runs the block before it without storing, only to
  // obtain that block's terminal state (the carry is one hop, so one block of run-in is exact).
  const int t_first = max(t_begin - kTile, 0);

  // H is a multiple of 4: the last wavefront of a row may own only 4 real heads. Lanes of heads
  // that do not exist read a head that does and store nowhere.
  const int head_local = lane >> 3;
  const bool real = ho + head_local < H;
  const int head = real ? ho + head_local : H - 1;
  const int d0 = (lane & 7) << 1;
  const int F = H * kChan;
  const int Fkv = (H / kv_groups) * kChan;
  const int v_stride = 2 * F, kv_stride = 2 * Fkv;  // bytes per time step
  constexpr int kRsrcFlags = 0x00020000;            // raw 32-bit buffer, gfx9 encoding
  const __amdgpu_buffer_rsrc_t rv =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(v_in + brow * L * F), 0, L * v_stride, kRsrcFlags);
  const __amdgpu_buffer_rsrc_t ro = __builtin_amdgcn_make_buffer_rsrc(out + brow * L * F, 0, L * v_stride, kRsrcFlags);
  const __amdgpu_buffer_rsrc_t rb =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(b_logit + brow * L * Fkv), 0, L * kv_stride, kRsrcFlags);
  const __amdgpu_buffer_rsrc_t rc =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(c_in + brow * L * Fkv), 0, L * kv_stride, kRsrcFlags);
  const __amdgpu_buffer_rsrc_t ra =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(a_logit + brow * L * H), 0, L * H * 2, kRsrcFlags);
  const int v_lane = 2 * (head * kChan + d0), kv_lane = 2 * ((head / kv_groups) * kChan + d0);
  // A lane without a head stores at an offset beyond the resource, which the buffer unit drops.
  const int o_lane = real ? v_lane : 0x7ffffff0;
  // gate logits: lane (hg, t) = (lane / 16, lane % 16) converts heads ho + 2 hg, + 1 of step t
  const int gt = lane & 15, ghead = min(ho + 2 * (lane >> 4), H - 2);
  const int a_lane = 2 * (gt * H + ghead);
  float* at = a_tile[wave];
#ifndef SPEAR_FUSED_LD_AUX
#define SPEAR_FUSED_LD_AUX 2
#endif
#ifndef SPEAR_FUSED_ST_AUX
#define SPEAR_FUSED_ST_AUX 2
#endif
  constexpr int kNt = SPEAR_FUSED_LD_AUX;  // non-temporal: every word is touched once
  constexpr int kNtS = SPEAR_FUSED_ST_AUX;

  // Two register sets of one block each (16 steps x {b, c, v} words per lane): while one block is
  // being processed the next one is already in flight, so a wait only ever concerns loads that
  // were issued a whole block earlier and never the younger stores.
  struct Words {
    uint32_t b[16], c[16], v[16];
  };
  auto issue = [&](Words& wd, int t) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      wd.b[r] = __builtin_amdgcn_raw_buffer_load_b32(rb, kv_lane, (t + r) * kv_stride, kNt);
      wd.v[r] = __builtin_amdgcn_raw_buffer_load_b32(rv, v_lane, (t + r) * v_stride, kNt);
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) wd.c[r] = __builtin_amdgcn_raw_buffer_load_b32(rc, kv_lane, (t + r) * kv_stride, kNt);
  };
  auto issue_gate = [&](int t) -> uint32_t { return __builtin_amdgcn_raw_buffer_load_b32(ra, a_lane, t * H * 2, 0); };

  float carry0 = 0.0f, carry1 = 0.0f;  // terminal local state of the previous block

  auto process = [&](const Words& wd, uint32_t araw, int t0) {
    const int o_off = (t0 >= t_begin) ? o_lane : 0x7ffffff0;  // run-in block: store nowhere
    at[(2 * (lane >> 4)) * kGateRow + gt] = clamp_coeff<E>(fast_sigmoid(E::lo(araw)));
    at[(2 * (lane >> 4) + 1) * kGateRow + gt] = clamp_coeff<E>(fast_sigmoid(E::hi(araw)));
    wave_lds_handover();
    float a[16];
#pragma unroll
    for (int c4 = 0; c4 < 4; ++c4) {
      const float4 q = *reinterpret_cast<const float4*>(at + head_local * kGateRow + 4 * c4);
      a[4 * c4 + 0] = q.x; a[4 * c4 + 1] = q.y; a[4 * c4 + 2] = q.z; a[4 * c4 + 3] = q.w;
    }
    wave_lds_handover();  // the tile may be overwritten by the next block from here on

    // pass 1: gated inputs and the zero-started recurrence (its terminal value is the next carry)
    float x0[16], x1[16];
    float l0 = 0.0f, l1 = 0.0f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      x0[r] = fast_sigmoid(E::lo(wd.b[r])) * E::lo(wd.v[r]);
      x1[r] = fast_sigmoid(E::hi(wd.b[r])) * E::hi(wd.v[r]);
      l0 = fmaf(a[r], l0, x0[r]);
      l1 = fmaf(a[r], l1, x1[r]);
    }
    // pass 2: the carry-started recurrence and the output mix
    float y0 = carry0, y1 = carry1;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      y0 = fmaf(a[r], y0, x0[r]);
      y1 = fmaf(a[r], y1, x1[r]);
      const uint32_t ow =
          E::pack2(fmaf(y0, E::lo(wd.c[r]), E::lo(wd.v[r])), fmaf(y1, E::hi(wd.c[r]), E::hi(wd.v[r])));
      __builtin_amdgcn_raw_buffer_store_b32(ow, ro, o_off, (t0 + r) * v_stride, kNtS);
    }
    carry0 = l0;
    carry1 = l1;
  };

  Words w0, w1;
  issue(w0, t_first);
  uint32_t g0 = issue_gate(t_first), g1 = 0u;
  for (int t0 = t_first; t0 < t_end; t0 += 2 * kTile) {
    // the scheduling barriers keep the look-ahead loads in front of the arithmetic (left alone,
    // the scheduler sinks them next to their uses to save registers, which serialises the two)
    const bool more1 = t0 + kTile < t_end, more2 = t0 + 2 * kTile < t_end;  // wave-uniform
    if (more1) {
      issue(w1, t0 + kTile);
      g1 = issue_gate(t0 + kTile);
    }
    __builtin_amdgcn_sched_barrier(0);
    process(w0, g0, t0);
    if (more1) {
      __builtin_amdgcn_sched_barrier(0);
      if (more2) {
        issue(w0, t0 + 2 * kTile);
        g0 = issue_gate(t0 + 2 * kTile);
      }
      __builtin_amdgcn_sched_barrier(0);
      process(w1, g1, t0 + kTile);
    }
    __builtin_amdgcn_sched_barrier(0);
  }
}

}  // namespace

hipError_t fused_mix_forward(const MixArgs& p, hipStream_t s) {
  // Rows are cut into time chunks when batch x heads alone would leave the GPU underfilled. A chunk
  // costs one extra block of reads (its run-in), so chunks are at least 8 blocks long.
  const long per_row = (p.H + 7) / 8;
  const int nb = p.L / kTile;
  const char* env = getenv("SPEAR_BTP_FUSED_WAVES");  // tuning override
  const long want_waves = env ? atol(env) : 1024;  // one wavefront per SIMD: longer runs beat more waves (measured)
  long chunks = (want_waves + p.B * per_row - 1) / (p.B * per_row);
  chunks = chunks < 1 ? 1 : chunks;
  if (chunks > nb / 8) chunks = nb / 8 > 0 ? nb / 8 : 1;
  const int chunk_blocks = (int)((nb + chunks - 1) / chunks);
  chunks = (nb + chunk_blocks - 1) / chunk_blocks;
  const int chunk_steps = chunk_blocks * kTile;
  const long total = (long)p.B * chunks * per_row;
  const unsigned blocks = (unsigned)((total + kWaves - 1) / kWaves);
  if (p.dtype == kBf16) {
    hipLaunchKernelGGL((phalanx_mix_fwd_kernel<Bf16>), dim3(blocks), dim3(64 * kWaves), 0, s,
                       static_cast<const uint16_t*>(p.a_logit), static_cast<const uint16_t*>(p.b_logit),
                       static_cast<const uint16_t*>(p.c), static_cast<const uint16_t*>(p.v),
                       static_cast<uint16_t*>(p.out), p.L, p.H, p.kv_groups, chunk_steps, (int)chunks, total);
  } else {
    hipLaunchKernelGGL((phalanx_mix_fwd_kernel<Fp16>), dim3(blocks), dim3(64 * kWaves), 0, s,
                       static_cast<const uint16_t*>(p.a_logit), static_cast<const uint16_t*>(p.b_logit),
                       static_cast<const uint16_t*>(p.c), static_cast<const uint16_t*>(p.v),
                       static_cast<uint16_t*>(p.out), p.L, p.H, p.kv_groups, chunk_steps, (int)chunks, total);
  }
  return hipGetLastError();
}

}  // namespace spear_btp
