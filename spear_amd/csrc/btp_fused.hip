// Fused Phalanx mixing kernels for gfx950 (MI355X): everything the layer does between its input
// projections and its output projection, in the projections' own [B, L, features] layout.
//
//     A = sigmoid(a_logit)            [B, L, H]          decay per head and step
//     X = sigmoid(b_logit) * v        [B, L, H*16]       gated input (b, c may have fewer, shared heads)
//     h = btp(A, X)   (k = 2)                            one-hop block recurrence over time
//     out = h * c + v                 [B, L, H*16]
//
// In the reference these are separate PyTorch ops around the BTP kernel
// (spear/nn/phalanx/swr.py:166-221 for the gates, :311-327 for `y * C + V`, the permute and the
// `.contiguous()` transposes hidden in spear/ops/btp/interface.py:186-187): about twenty passes
// over [B, L, H*16]-sized tensors. Here each operand is read once and each result written once, forward
// (phalanx_mix_fwd_tile_kernel) and backward (phalanx_mix_bwd_tile_kernel).
//
// Layout and work split. Features are the contiguous axis, time is strided, so a lane owns a feature
// pair (4 bytes) of up to 8 consecutive heads' 128 features and a wavefront owns ONE 16-step block of
// them: a wave-level load or store is one contiguous 256-byte run per time step, addressed through
// buffer instructions (a wave-uniform resource per operand, an SGPR offset for the time step, one constant
// per-lane byte offset). A wavefront runs no loop over time: every load is issued at the start, every store
// at the end, and a workgroup (4 or 8 wavefronts = consecutive blocks of the same features of one batch row)
// lives for a few microseconds. The one-hop structure makes blocks independent up to quantities that are
// local to a block (the terminal value of its zero-started recurrence; in backward also a_0 R_0 of its
// zero-started reverse recurrence): every wavefront computes its own block's, leaves them in LDS for its
// neighbours behind the kernel's single barrier, and the first / last block of a workgroup recompute the
// neighbour's from two operands of the block beyond the edge. There is no LDS staging of the big operands.
// sigmoid(a_logit) is computed once per (step, head) -- two per lane -- and handed to the lanes that need
// it through a 640-byte LDS tile.
//
// Copy loops with these kernels' traffic are why the split looks like this: wavefronts that walk through
// time with two register sets reach 0.65 of the HBM peak whatever the chunking, short-lived tiles 0.71-0.74
// (reads and writes do not overlap on the memory bus, so what counts is how quickly a wavefront turns from
// its read phase to its write phase and makes room for the next one). An earlier pair of kernels whose
// wavefronts walked through time gave the same results and was slower at every shape measured (forward
// 92-96 against 86-87 us, backward 185-196 against 163 us at B=1024 L=128 H=32).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <mutex>
#include <type_traits>

#include "../../include/spear_btp.h"
#include "btp_device.h"
#include "btp_launch.h"

// Device memory owned by the library, for the one entry point that must not allocate
// (fused_mix_backward_bias below): the per-(batch row, time tile) partial column sums of the fused
// backward kernel park here between that kernel and the kernel that finishes the sums. Every GPU the
// library runs on holds its own copy until the process ends. In host code the name stands for the
// symbol, not for a device address: the address is looked up once per device and only that pointer
// is handed to kernels.
static __device__ __align__(256) float scratch[SPEAR_MIX_BIAS_SCRATCH_FLOATS];

namespace spear_btp {

namespace {

// Value of `v` held by lane ^ mask (any mask; goes through the LDS crossbar, no memory access).
__device__ __forceinline__ float lane_xor(float v, int lane, int mask) {
  return __int_as_float(__builtin_amdgcn_ds_bpermute((lane ^ mask) << 2, __float_as_int(v)));
}

__device__ __forceinline__ float fast_sigmoid(float z) {
  return __builtin_amdgcn_rcpf(1.0f + __expf(-z));
}

// The kernels come in two operand conventions (kQkv):
//   false  layer form:  a = sigmoid(a_logit), a_logit 16-bit;  input gate G = sigmoid(b_logit)
//   true   q/k/v/gate form:  a = exp(gate), gate fp32 log-decay [B, L, H];  the b operand is k itself
//          (G = k), the c operand is q:   out = q * btp(exp(gate), k * v) + v
// Everything else (layout, work split, recurrences) is shared.
struct GateWords {
  uint32_t lo, hi;  // layer form: lo = two 16-bit logits; q/k/v form: two fp32 log-decays
};

template <class E, bool kQkv>
__device__ __forceinline__ float2 decay_pair(GateWords w) {
  if constexpr (kQkv) {
    const float a0 = __expf(__uint_as_float(w.lo)), a1 = __expf(__uint_as_float(w.hi));
    return make_float2(clamp_coeff<E>(a0), clamp_coeff<E>(a1));
  } else {
    return make_float2(clamp_coeff<E>(fast_sigmoid(E::lo(w.lo))), clamp_coeff<E>(fast_sigmoid(E::hi(w.lo))));
  }
}

template <bool kQkv>
__device__ __forceinline__ float input_gate(float b) {
  if constexpr (kQkv) return b;
  else return fast_sigmoid(b);
}

constexpr int kHeadsPerWave = 8;
constexpr int kGateRow = 20;  // floats per head in the decay tile: 16 steps + 4 of padding (bank spread)
constexpr int kNowhere = 0x7ffffff0;  // a byte offset beyond every buffer resource: the buffer unit drops the access

typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

// Where the gate values of a wavefront's heads come from. Lane (hg, t) = (lane / 16, lane % 16) converts the
// head pair (first + 2 hg, first + 2 hg + 1) of step t. Heads past the last one are clamped to it (their tile
// rows are read by lanes without a head only). 16-bit logits of a head pair are one aligned 32-bit word when
// the row length H and the wavefront's first head are even; otherwise (`split`, wave-uniform) they are
// fetched as two 16-bit loads.
struct GatePlace {
  int off0, off1;  // byte offsets of the two heads' values inside a [L, H] batch row, step t included
  bool split;
};

template <bool kQkv>
__device__ __forceinline__ GatePlace gate_place(int first, int H, int lane) {
  constexpr int kGateBytes = kQkv ? 4 : 2;
  const int gt = lane & 15, h0 = first + 2 * (lane >> 4);
  GatePlace g;
  g.split = !kQkv && (((H | first) & 1) != 0);
  if (kQkv || g.split) {
    g.off0 = kGateBytes * (gt * H + min(h0, H - 1));
    g.off1 = kGateBytes * (gt * H + min(h0 + 1, H - 1));
  } else {
    g.off0 = kGateBytes * (gt * H + min(h0, H - 2));
    g.off1 = 0;
  }
  return g;
}

// The gate words of the block that starts at step t (ra: the batch row's [L, H] gates).
template <bool kQkv>
__device__ __forceinline__ GateWords load_gate_words(__amdgpu_buffer_rsrc_t ra, const GatePlace& g, int t, int H) {
  constexpr int kGateBytes = kQkv ? 4 : 2;
  GateWords w;
  if constexpr (kQkv) {
    w.lo = __builtin_amdgcn_raw_buffer_load_b32(ra, g.off0, t * H * kGateBytes, 0);
    w.hi = __builtin_amdgcn_raw_buffer_load_b32(ra, g.off1, t * H * kGateBytes, 0);
  } else {
    if (g.split) {
      const uint32_t lo = __builtin_amdgcn_raw_buffer_load_b16(ra, g.off0, t * H * kGateBytes, 0);
      const uint32_t hi = __builtin_amdgcn_raw_buffer_load_b16(ra, g.off1, t * H * kGateBytes, 0);
      w.lo = lo | (hi << 16);
    } else {
      w.lo = __builtin_amdgcn_raw_buffer_load_b32(ra, g.off0, t * H * kGateBytes, 0);
    }
    w.hi = 0u;
  }
  return w;
}


// ==========================================================================================
// Shared by the forward and the backward kernel: which tile a workgroup is.
// ==========================================================================================
// Wavefronts per workgroup and per SIMD of the backward kernel. 4 and 3 (168 registers: nothing spills, 12
// wavefronts per CU) beat 8 and 4 (128 registers, three or four spilled values per lane that show up as 2.5 %
// more HBM writes, 16 wavefronts per CU) by 1 % at B=1024 L=128 H=32, 3 % at B=16 L=8192 H=64 and 5 % at B=64
// L=2048 H=128.
#ifndef SPEAR_FUSED_TILE_WAVES
#define SPEAR_FUSED_TILE_WAVES 4
#endif
constexpr int kTileWaves = SPEAR_FUSED_TILE_WAVES;

// v of the lane `kCtrl` names within the lane's DPP row of 16, or 1.0 where that lane does not exist
template <int kCtrl>
__device__ __forceinline__ float dpp_or_one(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0x3f800000, __float_as_int(v), kCtrl, 0xF, 0xF, false));
}

// For a value held by the 16 lanes of a DPP row (lane t = step t): the product over all OTHER lanes' values.
__device__ __forceinline__ float product_of_the_others(float a) {
  float p = a, q = a;  // inclusive prefix and suffix products (row_shr / row_shl by 1, 2, 4, 8)
  p *= dpp_or_one<0x111>(p); p *= dpp_or_one<0x112>(p); p *= dpp_or_one<0x114>(p); p *= dpp_or_one<0x118>(p);
  q *= dpp_or_one<0x101>(q); q *= dpp_or_one<0x102>(q); q *= dpp_or_one<0x104>(q); q *= dpp_or_one<0x108>(q);
  return dpp_or_one<0x111>(p) * dpp_or_one<0x101>(q);
}

#ifndef SPEAR_FUSED_TILE_XCD_GROUP  // neighbouring 4-wavefront workgroups per XCD; 0: launch order (round-robin)
#define SPEAR_FUSED_TILE_XCD_GROUP 64
#endif
#ifndef SPEAR_FUSED_TILE_WAVES_PER_EU
#define SPEAR_FUSED_TILE_WAVES_PER_EU 3
#endif
// The kWide backward (head groups summed through LDS) at 2 per SIMD: 220-250 registers, nothing spills. At 3 it
// spills 204 bytes per lane and takes 1.8-2.3 times as long (B=1024 L=128 H=32 in groups of 16: 171 -> 301 us).
#ifndef SPEAR_FUSED_WIDE_WAVES_PER_EU
#define SPEAR_FUSED_WIDE_WAVES_PER_EU 2
#endif
// Which tile workgroup this is: two steps, XCD dealing (tile_workgroup) and the order of the tiles (tile_place).
// Launch order deals workgroups round-robin to the 8 XCDs, each with its own L2. An XCD gets runs of
// SPEAR_FUSED_TILE_XCD_GROUP neighbouring workgroups instead (windows of 8 runs sweep the tensors front to back):
// the workgroup that owns an edge block and the neighbour that reads it as its halo then share an L2 close in
// time. Backward with head slots fastest, against plain round-robin (0), runs of 128 four-wavefront workgroups:
// 184 -> 166-167 us at B=1024 L=128 H=32, 371 -> 344 us at B=16 L=8192 H=64, 733 -> 718 us at B=64 L=2048 H=128;
// with the tiles in groups of 8 (below) runs of 64 are best (32: forward -3 % on long rows, 256: -5 to -15 %).
// The tail of the grid that does not fill a window keeps the launch order.
//
// Workgroup -> (batch row, time tile, head slot: which 128 features). Up to SPEAR_FUSED_TILE_TIME_GROUP consecutive
// time tiles of one head slot are neighbours in this order, then come the row's other head slots, then the next
// tiles: the workgroup that streams an edge block and the one that reads it as its halo are dispatched back to
// back on one XCD, while the run as a whole still covers whole feature rows. Measured (forward / backward, us):
//   tiles in groups of   1 (head slots fastest)    2           4           8           16         all (time fastest)
//   B=1024 L=128 H=32    86.9 / 166.4              86.9 / 162  86.9 / 162  86.9 / 162  87 / 162   87.0 / 162.2
//   B=16 L=8192 H=64     178.9 / 344.4             173 / 336   167 / 342   172 / 327   179 / 334  191.5 / 372.4
//   B=64 L=2048 H=128    364.2 / 707               363 / 711   372 / 681   346 / 679   356 / 689  355.8 / 698.6
// A grid padded to whole groups: workgroups of tiles past the row's end only join the barriers.
#ifndef SPEAR_FUSED_TILE_TIME_GROUP
#define SPEAR_FUSED_TILE_TIME_GROUP 8
#endif
struct TilePlace {
  int slot, tile;
  long brow;
};
__device__ __forceinline__ TilePlace tile_place(unsigned wg, int tiles, int slots) {
  const unsigned tg = min((unsigned)SPEAR_FUSED_TILE_TIME_GROUP, (unsigned)tiles);
  const unsigned tgroups = ((unsigned)tiles + tg - 1) / tg;
  const unsigned t_lo = wg % tg, r1 = wg / tg;
  TilePlace p;
  p.slot = (int)(r1 % (unsigned)slots);
  const unsigned r2 = r1 / (unsigned)slots;
  p.tile = (int)((r2 % tgroups) * tg + t_lo);
  p.brow = r2 / tgroups;
  return p;
}

template <int kRun = SPEAR_FUSED_TILE_XCD_GROUP>
__device__ __forceinline__ unsigned tile_workgroup() {
  unsigned wg = blockIdx.x;
  if constexpr (kRun > 0) {
    constexpr unsigned kWin = 8u * kRun;
    const unsigned win = wg / kWin, in = wg - win * kWin;
    if ((win + 1) * kWin <= gridDim.x) wg = win * kWin + (in & 7u) * kRun + (in >> 3);
  }
  return wg;
}

// Which heads a wavefront of the backward kernel owns. A head slot is normally 8 consecutive heads (the last
// slot of a row may hold fewer). The gradients of b and c are sums over the heads that share a kv head; with
// groups of 1, 2, 4 or 8 heads a group lies inside one slot on lanes a power of two apart, and the sum is a few
// DPP / permute exchanges. Every other grouping (kWide) gets slots cut at group borders instead:
//   groups of 3, 5, 6, 7 heads:   a slot = as many whole groups as fit into 8 heads (2, 1, 1, 1)
//   groups of more than 8 heads:  a slot = one kv head; the wavefront works through the group's heads 8 at a
//                                 time (a loop around the whole tile computation) and adds up as it goes
// and the sum over a group goes through LDS, four time steps at a time, in a fixed order.
struct HeadSlot {
  int first, count;        // heads [first, first + count) are this pass's, count <= 8
  int kv_first, kv_count;  // kWide: the kv heads whose groups these are (one, if a group is worked through in passes)
};
template <bool kWide>
__device__ __forceinline__ HeadSlot head_slot(int slot, int pass, int H, int group) {
  HeadSlot s;
  if constexpr (!kWide) {
    s.first = slot * kHeadsPerWave;
    s.count = min(kHeadsPerWave, H - s.first);
    s.kv_first = s.first / group;
    s.kv_count = 0;  // not used
  } else if (group <= kHeadsPerWave) {
    const int per_slot = kHeadsPerWave / group;
    s.kv_first = slot * per_slot;
    s.kv_count = min(per_slot, H / group - s.kv_first);
    s.first = s.kv_first * group;
    s.count = s.kv_count * group;
  } else {
    s.kv_first = slot;
    s.kv_count = 1;
    s.first = slot * group + pass * kHeadsPerWave;
    s.count = min(kHeadsPerWave, group - pass * kHeadsPerWave);
  }
  return s;
}

// ==========================================================================================
// Backward of the fused mixing stage. Inputs a_logit, b_logit, c, v, dout; outputs da_logit, db_logit, dc, dv --
// each big tensor is read or written exactly once. A workgroup is kTileWaves consecutive blocks of one head slot
// of one batch row, one wavefront each.
//
// The one-hop structure makes tiles independent up to two neighbour quantities, both LOCAL to a block:
//   c_out(i)  = terminal value of the zero-started forward recurrence over block i      (carry into block i+1)
//   dC_out(i) = a_0 R_0 of the zero-started reverse recurrence over block i             (gradient carry into block i-1)
// Every wavefront computes both for its own block first and leaves them in LDS; after the workgroup
// barrier its neighbours pick them up. The first and last block of a workgroup have no neighbour inside it:
// those wavefronts read two operands of the block beyond the edge as well (b, v for the forward carry or dout,
// c for the gradient carry; cacheable loads, the neighbouring workgroup reads the same lines at about the
// same time) and run the one recurrence they need on them.
//
// With A = sigmoid(a), G = sigmoid(b), x = G v, g = dout * c (the recurrence's upstream gradient), R the
// zero-started reverse recurrence R_r = g_r + a_{r+1} R_{r+1}, h the state of the carry-started recurrence
// (h_{-1} = c_in, h_r = a_r h_{r-1} + x_r) and dX_r = R_r + (prod_{j>r} a_j) dC, per step
//   dc_r = dout_r h_r ;  dv_r = dout_r + dX_r G_r ;  db_r = dX_r v_r G_r (1 - G_r)
//   dA_r = sum over the head's channels of dX_r h_{r-1}  -  (prod_{j != r} a_j) sum over channels of dC c_in
//   da_r = dA_r A_r (1 - A_r)
// (the second term of dA takes out the two-hop path c_in -> dC that h carries but the operator does not have).
//
// kF32: check mode, the four gradients leave as fp32 (the kernel's own values, not rounded to 16 bits).
// kSums: also leave, per workgroup (batch row, time tile), the sums over the tile's time steps of da_logit, db_logit
// and dc in fp32 (before their rounding to 16 bits): every wavefront sums its block's 16 steps, the workgroup's
// blocks are added in block order behind a second barrier (a fixed order: the same bits in every run), and row
// `batch row * tiles + tile` of the three arrays is written.
// kWide: head groupings other than 1, 2, 4, 8 heads per kv head (head_slot above).
// ==========================================================================================
template <class E, bool kQkv, bool kF32, bool kSums = false, bool kWide = false>
__global__ __launch_bounds__(64 * kTileWaves)
__attribute__((amdgpu_waves_per_eu(kWide ? SPEAR_FUSED_WIDE_WAVES_PER_EU : SPEAR_FUSED_TILE_WAVES_PER_EU)))
void phalanx_mix_bwd_tile_kernel(
    const uint16_t* __restrict__ a_logit, const uint16_t* __restrict__ b_logit, const uint16_t* __restrict__ c_in,
    const uint16_t* __restrict__ v_in, const uint16_t* __restrict__ dout, uint16_t* __restrict__ da_logit,
    uint16_t* __restrict__ db_logit, uint16_t* __restrict__ dc, uint16_t* __restrict__ dv, float* __restrict__ sum_da,
    float* __restrict__ sum_db, float* __restrict__ sum_dc, int ld_da, int ld_db, int ld_dc, int ld_dv, int L, int H,
    int kv_groups, int tiles, int slots) {
  // per wavefront: decay of its block, product of the block's other decays per step, decay of the block beyond the edge
  __shared__ __align__(16) float gate_tiles[kTileWaves][3][kHeadsPerWave * kGateRow];
  __shared__ float2 carry_out[kTileWaves][2][64];  // [0] dC_out, [1] c_out of the wavefront's block, per lane
  __shared__ float block_sums[kSums ? kTileWaves : 1][5][64];  // kSums: db (2), dc (2), da of the wavefront's block
  // kWide: (dc0, dc1, db0, db1) of four time steps per lane, before the sum over a kv head's group
  __shared__ __align__(16) float4 group_terms[kWide ? kTileWaves : 1][4][64];

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const unsigned wg = tile_workgroup();
  constexpr int nb_w = kTileWaves;  // consecutive blocks per workgroup, one per wavefront, all of one head slot
  const TilePlace at = tile_place(wg, tiles, slots);
  const int tile = at.tile, bl = wave;
  const long brow = at.brow;
  const int t0 = (tile * nb_w + bl) * kTile;
  // passes over the heads of a group that is larger than a wavefront's 8 heads (kWide only), same for the workgroup
  const int passes = (kWide && kv_groups > kHeadsPerWave) ? (kv_groups + kHeadsPerWave - 1) / kHeadsPerWave : 1;
  const bool valid = t0 < L;  // wave-uniform; a wavefront without a block only joins the barriers

  const int head_local = lane >> 3;
  const int d0 = (lane & 7) << 1;
  const int F = H * kChan, Fkv = (H / kv_groups) * kChan;
  const int stride = 2 * F, kv_stride = 2 * Fkv;
  constexpr int kRsrcFlags = 0x00020000;
  constexpr int kGateBytes = kQkv ? 4 : 2;
  constexpr int kDaBytes = (kQkv || kF32) ? 4 : 2;
  constexpr int kGradBytes = kF32 ? 4 : 2;
  const long big = brow * L * F, kvbig = brow * L * Fkv, small = brow * L * H;
  auto rsrc = [&](const uint16_t* p, long off, int bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(p + off), 0, bytes, kRsrcFlags);
  };
  const __amdgpu_buffer_rsrc_t rb = rsrc(b_logit, kvbig, L * kv_stride), rc = rsrc(c_in, kvbig, L * kv_stride),
                               rv = rsrc(v_in, big, L * stride), rg = rsrc(dout, big, L * stride),
                               ra = rsrc(a_logit, small * (kGateBytes / 2), L * H * kGateBytes),
                               // the four gradients may sit side by side in one wider buffer: each has its
                               // own elements-per-time-step (ld_*), equal to its width when it is dense
                               rdb = rsrc(db_logit, brow * L * ld_db * (kGradBytes / 2), L * ld_db * kGradBytes),
                               rdc = rsrc(dc, brow * L * ld_dc * (kGradBytes / 2), L * ld_dc * kGradBytes),
                               rdv = rsrc(dv, brow * L * ld_dv * (kGradBytes / 2), L * ld_dv * kGradBytes),
                               rda = rsrc(da_logit, brow * L * ld_da * (kDaBytes / 2), L * ld_da * kDaBytes);
  constexpr int kNt = 2;

  // the block beyond the workgroup's edge that this wavefront has to look at (at most one: nb_w >= 2)
  const bool halo_prev = valid && bl == 0 && t0 > 0;                    // needs c_out of block t0 - 16
  const bool halo_next = valid && bl == nb_w - 1 && t0 + kTile < L;     // needs dC_out of block t0 + 16
  const bool halo = halo_prev || halo_next;
  const int th = halo_prev ? t0 - kTile : t0 + kTile;

  float* ta = gate_tiles[wave][0];
  float* te = gate_tiles[wave][1];
  float* tn = gate_tiles[wave][2];
  const int gt = lane & 15;
  auto write_tile = [&](float* tile_, float x0, float x1) {
    tile_[(2 * (lane >> 4)) * kGateRow + gt] = x0;
    tile_[(2 * (lane >> 4) + 1) * kGateRow + gt] = x1;
  };

  // kWide with passes: the sums over the group so far, for the lane's (step, feature pair) of each quarter block
  float4 group_acc[4];
#pragma unroll
  for (int c4 = 0; c4 < 4; ++c4) group_acc[c4] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);

  for (int pass = 0; pass < passes; ++pass) {
  const HeadSlot hs = head_slot<kWide>(at.slot, pass, H, kv_groups);
  const bool real = head_local < hs.count;
  const int head = hs.first + (real ? head_local : hs.count - 1);  // lanes without a head read one that exists
  const int f_lane = 2 * (head * kChan + d0);
  const int kv_lane = 2 * ((head / kv_groups) * kChan + d0);
  const int o_lane = real ? f_lane * (kGradBytes / 2) : kNowhere;  // and store nowhere
  // groups of 2, 4 or 8 heads: the sums over a group end up in all its lanes; its first head stores them
  const int okv_lane = (!kWide && real && (head % kv_groups) == 0) ? kv_lane * (kGradBytes / 2) : kNowhere;
  const GatePlace gp = gate_place<kQkv>(hs.first, H, lane);
  // da_logit: lane k of a head (k = lane % 8) ends up with steps 2k and 2k+1 of that head
  const int da_lane = real ? kDaBytes * ((2 * (lane & 7)) * ld_da + head) : kNowhere;
  const int da_lane1 = real ? da_lane + kDaBytes * ld_da : kNowhere;

  // ---- every global read, before anything waits
  uint32_t b[16], c[16], v[16], g[16], h0[16], h1[16];
  GateWords araw = {0u, 0u}, haraw = {0u, 0u};
  // Wavefronts at a workgroup edge read the block beyond the edge first and their own b, v only once those 32
  // registers are free again (b and v are not needed before the local forward recurrence); the other
  // wavefronts issue everything at once (with every load up front the kernel is no faster: 168 against 166 us).
  auto load_bv = [&]() {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      b[r] = __builtin_amdgcn_raw_buffer_load_b32(rb, kv_lane, (t0 + r) * kv_stride, kNt);
      v[r] = __builtin_amdgcn_raw_buffer_load_b32(rv, f_lane, (t0 + r) * stride, kNt);
    }
  };
  if (valid) {
  araw = load_gate_words<kQkv>(ra, gp, t0, H);
  if (halo) haraw = load_gate_words<kQkv>(ra, gp, th, H);
  if (halo_prev) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      h0[r] = __builtin_amdgcn_raw_buffer_load_b32(rb, kv_lane, (th + r) * kv_stride, 0);
      h1[r] = __builtin_amdgcn_raw_buffer_load_b32(rv, f_lane, (th + r) * stride, 0);
    }
  } else if (halo_next) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      h0[r] = __builtin_amdgcn_raw_buffer_load_b32(rg, f_lane, (th + r) * stride, 0);
      h1[r] = __builtin_amdgcn_raw_buffer_load_b32(rc, kv_lane, (th + r) * kv_stride, 0);
    }
  }
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    g[r] = __builtin_amdgcn_raw_buffer_load_b32(rg, f_lane, (t0 + r) * stride, kNt);
    c[r] = __builtin_amdgcn_raw_buffer_load_b32(rc, kv_lane, (t0 + r) * kv_stride, kNt);
  }
  if (!halo) load_bv();
  }
  __builtin_amdgcn_sched_barrier(0);

  float cin0 = 0.0f, cin1 = 0.0f, dC0 = 0.0f, dC1 = 0.0f;
  float R[32];  // local reverse states, later dX, channel pair interleaved: R[2 r], R[2 r + 1]
  if (valid) {
    const float2 a01 = decay_pair<E, kQkv>(araw);
    write_tile(ta, a01.x, a01.y);
    write_tile(te, product_of_the_others(a01.x), product_of_the_others(a01.y));
    if (halo) {
      const float2 n01 = decay_pair<E, kQkv>(haraw);
      write_tile(tn, n01.x, n01.y);
    }
    wave_lds_handover();

    // ---- the block beyond the edge first, so that its 32 registers are free again before R is formed
    if (halo_prev) {
#pragma unroll
      for (int c4 = 0; c4 < 4; ++c4) {
        const float4 q = *reinterpret_cast<const float4*>(tn + head_local * kGateRow + 4 * c4);
        const float a4[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int r = 4 * c4 + i;
          cin0 = fmaf(a4[i], cin0, input_gate<kQkv>(E::lo(h0[r])) * E::lo(h1[r]));
          cin1 = fmaf(a4[i], cin1, input_gate<kQkv>(E::hi(h0[r])) * E::hi(h1[r]));
        }
        asm volatile("" ::: "memory");
      }
    } else if (halo_next) {
      float r0 = 0.0f, r1 = 0.0f, up = 0.0f;
#pragma unroll
      for (int c4 = 3; c4 >= 0; --c4) {
        const float4 q = *reinterpret_cast<const float4*>(tn + head_local * kGateRow + 4 * c4);
        const float a4[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (int i = 3; i >= 0; --i) {
          const int r = 4 * c4 + i;
          r0 = fmaf(up, r0, E::lo(h0[r]) * E::lo(h1[r]));
          r1 = fmaf(up, r1, E::hi(h0[r]) * E::hi(h1[r]));
          up = a4[i];
        }
        asm volatile("" ::: "memory");
      }
      dC0 = up * r0;
      dC1 = up * r1;
    }
    __builtin_amdgcn_sched_barrier(0);
    if (halo) load_bv();
    __builtin_amdgcn_sched_barrier(0);

    // Decays are read from the LDS tile four steps at a time, next to their use (a broadcast read for the 8
    // lanes of a head), rather than held in 16 registers through every pass; the compiler barriers keep the
    // reads where they are written.
    // ---- local reverse recurrence (upstream gradient of the recurrence: dout * c)
    {
      float r0 = 0.0f, r1 = 0.0f, up = 0.0f;  // up: decay of the step after the current one
#pragma unroll
      for (int c4 = 3; c4 >= 0; --c4) {
        const float4 q = *reinterpret_cast<const float4*>(ta + head_local * kGateRow + 4 * c4);
        const float a4[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (int i = 3; i >= 0; --i) {
          const int r = 4 * c4 + i;
          r0 = fmaf(up, r0, E::lo(g[r]) * E::lo(c[r]));
          r1 = fmaf(up, r1, E::hi(g[r]) * E::hi(c[r]));
          R[2 * r] = r0;
          R[2 * r + 1] = r1;
          up = a4[i];
        }
        asm volatile("" ::: "memory");
      }
      carry_out[wave][0][lane] = make_float2(up * r0, up * r1);
    }
    // ---- local forward recurrence: only its terminal value is needed here
    {
      float l0 = 0.0f, l1 = 0.0f;
#pragma unroll
      for (int c4 = 0; c4 < 4; ++c4) {
        const float4 q = *reinterpret_cast<const float4*>(ta + head_local * kGateRow + 4 * c4);
        const float a4[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int r = 4 * c4 + i;
          l0 = fmaf(a4[i], l0, input_gate<kQkv>(E::lo(b[r])) * E::lo(v[r]));
          l1 = fmaf(a4[i], l1, input_gate<kQkv>(E::hi(b[r])) * E::hi(v[r]));
        }
        asm volatile("" ::: "memory");
      }
      carry_out[wave][1][lane] = make_float2(l0, l1);
    }
  }
  __syncthreads();  // the workgroup barrier of the carries; wavefronts without a block arrive here directly
  if (!valid) {
    if constexpr (kSums) __syncthreads();  // the barrier of the sums counts every wavefront of the workgroup
    if (passes > 1) __syncthreads();
    continue;
  }

  if (bl > 0) {  // the block before this one belongs to the wavefront before this one
    const float2 q = carry_out[wave - 1][1][lane];
    cin0 = q.x;
    cin1 = q.y;
  }
  if (bl < nb_w - 1 && t0 + kTile < L) {
    const float2 q = carry_out[wave + 1][0][lane];
    dC0 = q.x;
    dC1 = q.y;
  }

  // dX_r = R_r + (prod_{j > r} a_j) dC, in place
  {
    float q0 = dC0, q1 = dC1;
#pragma unroll
    for (int c4 = 3; c4 >= 0; --c4) {
      const float4 q = *reinterpret_cast<const float4*>(ta + head_local * kGateRow + 4 * c4);
      const float a4[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
      for (int i = 3; i >= 0; --i) {
        const int r = 4 * c4 + i;
        R[2 * r] += q0;
        R[2 * r + 1] += q1;
        q0 *= a4[i];
        q1 *= a4[i];
      }
      asm volatile("" ::: "memory");
    }
  }

  // kWide: this lane's share of the sums over a group. Per quarter block (4 steps) the wavefront has 4 steps x 8
  // feature pairs x kv_count results; lane = (kv head, feature pair, step) adds the group's heads in head order.
  const int w_step = lane & 3, w_pair = (lane >> 2) & 7, w_kv = lane >> 5;
  const bool w_owner = kWide && w_kv < hs.kv_count;
  const int w_heads = kv_groups <= kHeadsPerWave ? kv_groups : hs.count;  // heads of the group in this pass
  const int w_src = (w_kv * w_heads) * 8 + w_pair;                        // the lane of the group's first head
  const bool w_store = w_owner && pass == passes - 1;
  const int w_col = kGradBytes * ((hs.kv_first + w_kv) * kChan + 2 * w_pair);
  const int w_dc = w_store ? w_col + w_step * kGradBytes * ld_dc : kNowhere;
  const int w_db = w_store ? w_col + w_step * kGradBytes * ld_db : kNowhere;

  // ---- forward pass: state, gradients, per-step partial sums of dA
  float e[16];
  float acc_b0 = 0.0f, acc_b1 = 0.0f, acc_c0 = 0.0f, acc_c1 = 0.0f;  // kSums only
  float hs0 = cin0, hs1 = cin1;  // h_{r-1}
#pragma unroll
  for (int c4 = 0; c4 < 4; ++c4) {
    const float4 qa = *reinterpret_cast<const float4*>(ta + head_local * kGateRow + 4 * c4);
    const float a4[4] = {qa.x, qa.y, qa.z, qa.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int r = 4 * c4 + i;
      const float G0 = input_gate<kQkv>(E::lo(b[r])), G1 = input_gate<kQkv>(E::hi(b[r]));
      const float v0 = E::lo(v[r]), v1 = E::hi(v[r]);
      const float go0 = E::lo(g[r]), go1 = E::hi(g[r]);
      const float dX0 = R[2 * r], dX1 = R[2 * r + 1];
      e[r] = fmaf(dX0, hs0, dX1 * hs1);
      hs0 = fmaf(a4[i], hs0, G0 * v0);
      hs1 = fmaf(a4[i], hs1, G1 * v1);
      float dc0 = go0 * hs0, dc1 = go1 * hs1;
      float db0 = dX0 * v0, db1 = dX1 * v1;  // dX * v: the gradient of k in the q/k/v form
      if constexpr (!kQkv) {
        db0 *= G0 * (1.0f - G0);
        db1 *= G1 * (1.0f - G1);
      }
      const float dv0 = fmaf(dX0, G0, go0), dv1 = fmaf(dX1, G1, go1);
      if constexpr (kWide) {
        group_terms[wave][i][lane] = real ? make_float4(dc0, dc1, db0, db1) : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        if constexpr (kF32) {
          const u32x2_t wdv = {__float_as_uint(dv0), __float_as_uint(dv1)};
          __builtin_amdgcn_raw_buffer_store_b64(wdv, rdv, o_lane, (t0 + r) * 4 * ld_dv, kNt);
        } else {
          __builtin_amdgcn_raw_buffer_store_b32(E::pack2(dv0, dv1), rdv, o_lane, (t0 + r) * 2 * ld_dv, kNt);
        }
      } else {
        if (kv_groups > 1) {  // wave-uniform: sum over the heads that share this kv head
          dc0 += row_xor<8>(dc0); dc1 += row_xor<8>(dc1); db0 += row_xor<8>(db0); db1 += row_xor<8>(db1);
          if (kv_groups > 2) {
            dc0 += lane_xor(dc0, lane, 16); dc1 += lane_xor(dc1, lane, 16);
            db0 += lane_xor(db0, lane, 16); db1 += lane_xor(db1, lane, 16);
          }
          if (kv_groups > 4) {
            dc0 += lane_xor(dc0, lane, 32); dc1 += lane_xor(dc1, lane, 32);
            db0 += lane_xor(db0, lane, 32); db1 += lane_xor(db1, lane, 32);
          }
        }
        if constexpr (kSums) {
          acc_b0 += db0; acc_b1 += db1; acc_c0 += dc0; acc_c1 += dc1;
        }
        if constexpr (kF32) {
          const u32x2_t wdc = {__float_as_uint(dc0), __float_as_uint(dc1)}, wdv = {__float_as_uint(dv0), __float_as_uint(dv1)},
                        wdb = {__float_as_uint(db0), __float_as_uint(db1)};
          __builtin_amdgcn_raw_buffer_store_b64(wdc, rdc, okv_lane, (t0 + r) * 4 * ld_dc, kNt);
          __builtin_amdgcn_raw_buffer_store_b64(wdv, rdv, o_lane, (t0 + r) * 4 * ld_dv, kNt);
          __builtin_amdgcn_raw_buffer_store_b64(wdb, rdb, okv_lane, (t0 + r) * 4 * ld_db, kNt);
        } else {
          __builtin_amdgcn_raw_buffer_store_b32(E::pack2(dc0, dc1), rdc, okv_lane, (t0 + r) * 2 * ld_dc, kNt);
          __builtin_amdgcn_raw_buffer_store_b32(E::pack2(dv0, dv1), rdv, o_lane, (t0 + r) * 2 * ld_dv, kNt);
          __builtin_amdgcn_raw_buffer_store_b32(E::pack2(db0, db1), rdb, okv_lane, (t0 + r) * 2 * ld_db, kNt);
        }
      }
    }
    if constexpr (kWide) {
      wave_lds_handover();
      float4 sum = group_acc[c4];
      if (w_owner) {
        for (int j = 0; j < w_heads; ++j) {  // head order: the same bits in every run
          const float4 t = group_terms[wave][w_step][w_src + 8 * j];
          sum.x += t.x; sum.y += t.y; sum.z += t.z; sum.w += t.w;
        }
      }
      group_acc[c4] = sum;
      if constexpr (kSums) {  // the owner's four steps are the lanes of a quad
        float4 q = sum;
        q.x += row_xor<1>(q.x); q.y += row_xor<1>(q.y); q.z += row_xor<1>(q.z); q.w += row_xor<1>(q.w);
        q.x += row_xor<2>(q.x); q.y += row_xor<2>(q.y); q.z += row_xor<2>(q.z); q.w += row_xor<2>(q.w);
        acc_c0 += q.x; acc_c1 += q.y; acc_b0 += q.z; acc_b1 += q.w;
      }
      const int row = t0 + 4 * c4;
      if constexpr (kF32) {
        const u32x2_t wdc = {__float_as_uint(sum.x), __float_as_uint(sum.y)}, wdb = {__float_as_uint(sum.z), __float_as_uint(sum.w)};
        __builtin_amdgcn_raw_buffer_store_b64(wdc, rdc, w_dc, row * 4 * ld_dc, kNt);
        __builtin_amdgcn_raw_buffer_store_b64(wdb, rdb, w_db, row * 4 * ld_db, kNt);
      } else {
        __builtin_amdgcn_raw_buffer_store_b32(E::pack2(sum.x, sum.y), rdc, w_dc, row * 2 * ld_dc, kNt);
        __builtin_amdgcn_raw_buffer_store_b32(E::pack2(sum.z, sum.w), rdb, w_db, row * 2 * ld_db, kNt);
      }
      wave_lds_handover();  // the terms may be overwritten by the next quarter block from here on
    }
    asm volatile("" ::: "memory");
  }

  // ---- dA: sum over the 8 lanes (16 channels) of the head, transposing: lane k keeps steps 2k, 2k+1
  const int kk = lane & 7;
  float f8[8], f4[4];
  {
    const bool hi = kk & 4;
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      const float keep = hi ? e[t + 8] : e[t], send = hi ? e[t] : e[t + 8];
      f8[t] = keep + row_xor<4>(send);
    }
  }
  {
    const bool hi = kk & 2;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const float keep = hi ? f8[t + 4] : f8[t], send = hi ? f8[t] : f8[t + 4];
      f4[t] = keep + row_xor<2>(send);
    }
  }
  float s0, s1;
  {
    const bool hi = kk & 1;
    const float k0 = hi ? f4[2] : f4[0], n0 = hi ? f4[0] : f4[2];
    const float k1 = hi ? f4[3] : f4[1], n1 = hi ? f4[1] : f4[3];
    s0 = k0 + row_xor<1>(n0);
    s1 = k1 + row_xor<1>(n1);
  }
  // the two-hop path c_in -> dC, summed over the head's channels
  float two_hop = fmaf(dC0, cin0, dC1 * cin1);
  two_hop += row_xor<1>(two_hop);
  two_hop += row_xor<2>(two_hop);
  two_hop += row_xor<4>(two_hop);
  const float2 aa = *reinterpret_cast<const float2*>(ta + head_local * kGateRow + 2 * kk);
  const float2 ee = *reinterpret_cast<const float2*>(te + head_local * kGateRow + 2 * kk);
  s0 = fmaf(-ee.x, two_hop, s0);
  s1 = fmaf(-ee.y, two_hop, s1);
  // d/d a_logit = dA a (1 - a);  d/d gate = dA a  (gate = log a)
  const float da0 = kQkv ? s0 * aa.x : s0 * aa.x * (1.0f - aa.x), da1 = kQkv ? s1 * aa.y : s1 * aa.y * (1.0f - aa.y);
  if constexpr (kDaBytes == 4) {
    __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(da0), rda, da_lane, t0 * ld_da * 4, 0);
    __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(da1), rda, da_lane1, t0 * ld_da * 4, 0);
  } else {
    const uint32_t dap = E::pack2(da0, da1);
    __builtin_amdgcn_raw_buffer_store_b16((unsigned short)(dap & 0xffffu), rda, da_lane, t0 * ld_da * 2, 0);
    __builtin_amdgcn_raw_buffer_store_b16((unsigned short)(dap >> 16), rda, da_lane1, t0 * ld_da * 2, 0);
  }

  if constexpr (kSums) {
    float acc_a = da0 + da1;  // lane k of a head holds steps 2k, 2k+1
    acc_a += row_xor<1>(acc_a);
    acc_a += row_xor<2>(acc_a);
    acc_a += row_xor<4>(acc_a);  // now every lane of the head has the block's sum
    block_sums[wave][0][lane] = acc_b0;
    block_sums[wave][1][lane] = acc_b1;
    block_sums[wave][2][lane] = acc_c0;
    block_sums[wave][3][lane] = acc_c1;
    block_sums[wave][4][lane] = acc_a;
    __syncthreads();
    if (bl == 0) {  // the first block's wavefront adds the tile's blocks, in block order
      float t[5] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
      for (int j = 0; j < nb_w && t0 + j * kTile < L; ++j) {
#pragma unroll
        for (int q = 0; q < 5; ++q) t[q] += block_sums[j][q][lane];
      }
      const long row = brow * tiles + tile;
      if (real && (lane & 7) == 0) sum_da[row * H + head] = t[4];
      if constexpr (kWide) {  // every lane of an owner's quad has the sums of its (kv head, feature pair)
        if (w_store && w_step == 0) {
          const long col = row * Fkv + (hs.kv_first + w_kv) * kChan + 2 * w_pair;
          *reinterpret_cast<float2*>(sum_dc + col) = make_float2(t[2], t[3]);
          *reinterpret_cast<float2*>(sum_db + col) = make_float2(t[0], t[1]);
        }
      } else if (real && (head % kv_groups) == 0) {  // the group's sum is in every lane of the group
        const long col = row * Fkv + (head / kv_groups) * kChan + d0;
        *reinterpret_cast<float2*>(sum_db + col) = make_float2(t[0], t[1]);
        *reinterpret_cast<float2*>(sum_dc + col) = make_float2(t[2], t[3]);
      }
    }
  }
  if (passes > 1) __syncthreads();  // carry_out and block_sums are written again by the next pass
  }  // passes
}


// ==========================================================================================
// Forward of the fused mixing stage: the work split of the backward above (one wavefront per 16-step block of
// 128 features, no loop, one workgroup barrier, workgroups dealt to the XCDs in runs of neighbours). Per block a
// lane runs two fp32 recurrences over its feature pair: a zero-started one whose terminal value is the carry for
// the next block, and one started from the incoming carry that produces the outputs. A block needs one neighbour
// quantity, the terminal value of the zero-started recurrence over the block before it: every wavefront computes
// its own block's and leaves it in LDS for the next wavefront; the first block of a workgroup reads b and v of
// the block before the edge (cacheable loads: the neighbouring workgroup streams the same lines on the same L2)
// and runs that recurrence itself. A kv head shared by several heads is resolved by indexing (head h reads b, c of
// kv head h / group), for any group size. The wavefront of a row's last block also stores the streaming state for
// decoding after this prompt, when asked.
// kW wavefronts per workgroup, one head slot x kW consecutive blocks (2 head slots x kW / 2 blocks measured
// slower at every shape): 4 or 8. Microseconds for 4 / 8, B L H:
//   1024 128 32: 87.3 / 91.5    256 512 32: 89.8 / 86.0    16 8192 32: 89.4 / 87.1
//   512 128 64: 91.6 / 90.2     16 8192 64: 167.5 / 170.6  64 2048 128: 336.1 / 338.3
//   256 128 128: 87.7 / 90.1    4096 128 8: 92.9 / 88.1    1024 128 48: 132.9 / 125.3
// ==========================================================================================
template <class E, int kW, bool kQkv, bool kF32>
__global__ __launch_bounds__(64 * kW) __attribute__((amdgpu_waves_per_eu(SPEAR_FUSED_TILE_WAVES_PER_EU)))
void phalanx_mix_fwd_tile_kernel(const uint16_t* __restrict__ a_logit, const uint16_t* __restrict__ b_logit,
                                 const uint16_t* __restrict__ c_in, const uint16_t* __restrict__ v_in,
                                 uint16_t* __restrict__ out, float* __restrict__ c_prev_tail, int L, int H,
                                 int kv_groups, int tiles) {
  __shared__ __align__(16) float gate_tiles[kW][2][kHeadsPerWave * kGateRow];  // own block, block before the edge
  __shared__ float2 carry_out[kW][64];  // terminal local state of the wavefront's block, per lane

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const unsigned wg = tile_workgroup<SPEAR_FUSED_TILE_XCD_GROUP * 4 / kW>();
  constexpr int nb_w = kW;  // consecutive blocks per workgroup, one per wavefront, all of one head slot
  const TilePlace at = tile_place(wg, tiles, (H + kHeadsPerWave - 1) / kHeadsPerWave);
  const int tile = at.tile, bl = wave;
  const long brow = at.brow;
  const int ho = at.slot * kHeadsPerWave;
  const int t0 = (tile * nb_w + bl) * kTile;
  const bool valid = t0 < L;  // wave-uniform; a wavefront without a block only joins the barrier

  // The last slot of a row may hold fewer than 8 heads. Lanes of heads that do not exist read a head that
  // does and store nowhere.
  const int head_local = lane >> 3;
  const bool real = ho + head_local < H;
  const int head = real ? ho + head_local : H - 1;
  const int d0 = (lane & 7) << 1;
  const int F = H * kChan, Fkv = (H / kv_groups) * kChan;
  const int stride = 2 * F, kv_stride = 2 * Fkv;
  constexpr int kRsrcFlags = 0x00020000;
  constexpr int kGateBytes = kQkv ? 4 : 2;
  constexpr int kOutScale = kF32 ? 2 : 1;
  const long big = brow * L * F, kvbig = brow * L * Fkv, small = brow * L * H;
  auto rsrc = [&](const uint16_t* p, long off, int bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(p + off), 0, bytes, kRsrcFlags);
  };
  const __amdgpu_buffer_rsrc_t rb = rsrc(b_logit, kvbig, L * kv_stride), rc = rsrc(c_in, kvbig, L * kv_stride),
                               rv = rsrc(v_in, big, L * stride),
                               ra = rsrc(a_logit, small * (kGateBytes / 2), L * H * kGateBytes),
                               ro = rsrc(out, big * kOutScale, L * stride * kOutScale);
  const int f_lane = 2 * (head * kChan + d0);
  const int kv_lane = 2 * ((head / kv_groups) * kChan + d0);
  const int o_lane = real ? f_lane * kOutScale : kNowhere;
  const int gt = lane & 15;
  const GatePlace gp = gate_place<kQkv>(ho, H, lane);
  constexpr int kNt = 2;

  const bool halo = valid && bl == 0 && t0 > 0;  // needs the terminal local state of block t0 - 16
  const int th = t0 - kTile;

  // ---- every global read, before anything waits
  uint32_t b[16], c[16], v[16], hb[16], hv[16];
  GateWords araw = {0u, 0u}, haraw = {0u, 0u};
  if (valid) {
    araw = load_gate_words<kQkv>(ra, gp, t0, H);
    if (halo) {
      haraw = load_gate_words<kQkv>(ra, gp, th, H);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        hb[r] = __builtin_amdgcn_raw_buffer_load_b32(rb, kv_lane, (th + r) * kv_stride, 0);
        hv[r] = __builtin_amdgcn_raw_buffer_load_b32(rv, f_lane, (th + r) * stride, 0);
      }
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      b[r] = __builtin_amdgcn_raw_buffer_load_b32(rb, kv_lane, (t0 + r) * kv_stride, kNt);
      v[r] = __builtin_amdgcn_raw_buffer_load_b32(rv, f_lane, (t0 + r) * stride, kNt);
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) c[r] = __builtin_amdgcn_raw_buffer_load_b32(rc, kv_lane, (t0 + r) * kv_stride, kNt);
  }
  __builtin_amdgcn_sched_barrier(0);

  float* ta = gate_tiles[wave][0];
  float* tn = gate_tiles[wave][1];
  auto write_tile = [&](float* tile_, float x0, float x1) {
    tile_[(2 * (lane >> 4)) * kGateRow + gt] = x0;
    tile_[(2 * (lane >> 4) + 1) * kGateRow + gt] = x1;
  };
  auto read_decays = [&](const float* tile_, float (&a)[16]) {
#pragma unroll
    for (int c4 = 0; c4 < 4; ++c4) {
      const float4 q = *reinterpret_cast<const float4*>(tile_ + head_local * kGateRow + 4 * c4);
      a[4 * c4 + 0] = q.x; a[4 * c4 + 1] = q.y; a[4 * c4 + 2] = q.z; a[4 * c4 + 3] = q.w;
    }
  };

  float a[16], x0[16], x1[16];
  float cin0 = 0.0f, cin1 = 0.0f;
  if (valid) {
    const float2 a01 = decay_pair<E, kQkv>(araw);
    write_tile(ta, a01.x, a01.y);
    if (halo) {
      const float2 n01 = decay_pair<E, kQkv>(haraw);
      write_tile(tn, n01.x, n01.y);
    }
    wave_lds_handover();
    if (halo) {  // the zero-started recurrence over the block before the edge
      float an[16];
      read_decays(tn, an);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        cin0 = fmaf(an[r], cin0, input_gate<kQkv>(E::lo(hb[r])) * E::lo(hv[r]));
        cin1 = fmaf(an[r], cin1, input_gate<kQkv>(E::hi(hb[r])) * E::hi(hv[r]));
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    read_decays(ta, a);
    // gated inputs and the zero-started recurrence: its terminal value is the next block's carry
    float l0 = 0.0f, l1 = 0.0f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      x0[r] = input_gate<kQkv>(E::lo(b[r])) * E::lo(v[r]);
      x1[r] = input_gate<kQkv>(E::hi(b[r])) * E::hi(v[r]);
      l0 = fmaf(a[r], l0, x0[r]);
      l1 = fmaf(a[r], l1, x1[r]);
    }
    carry_out[wave][lane] = make_float2(l0, l1);
    // Hand-over for token-by-token decoding after this prompt: the terminal local state of the row's last block is
    // what the next block's steps need as c_prev (the block-local state restarts at 0 and the gate product at 1).
    if (c_prev_tail != nullptr && t0 + kTile == L && real)
      *reinterpret_cast<float2*>(c_prev_tail + (brow * H + head) * kChan + d0) = make_float2(l0, l1);
  }
  __syncthreads();  // the kernel's only workgroup barrier; wavefronts without a block arrive here directly
  if (!valid) return;

  if (bl > 0) {  // the block before this one belongs to the wavefront before this one
    const float2 q = carry_out[wave - 1][lane];
    cin0 = q.x;
    cin1 = q.y;
  }
  // the carry-started recurrence and the output mix
  float y0 = cin0, y1 = cin1;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    y0 = fmaf(a[r], y0, x0[r]);
    y1 = fmaf(a[r], y1, x1[r]);
    const float o0 = fmaf(y0, E::lo(c[r]), E::lo(v[r])), o1 = fmaf(y1, E::hi(c[r]), E::hi(v[r]));
    if constexpr (kF32) {
      const u32x2_t ow = {__float_as_uint(o0), __float_as_uint(o1)};
      __builtin_amdgcn_raw_buffer_store_b64(ow, ro, o_lane, (t0 + r) * stride * 2, kNt);
    } else {
      __builtin_amdgcn_raw_buffer_store_b32(E::pack2(o0, o1), ro, o_lane, (t0 + r) * stride, kNt);
    }
  }
}


// ==========================================================================================
// One decode token of the mixing stage in the layer's own layout: the projections' outputs for ONE time step,
// [B, features], and the streaming state of every (batch row, head). It is step_jagged of the reference
// (spear/nn/phalanx/inference.py:178-278) with the gates of the layer (spear/nn/phalanx/swr.py:196-221) applied
// in the same pass and the kv-head sharing resolved by indexing:
//   A = sigmoid(a_logit), G = sigmoid(b_logit);   h = A h + G v;   r = A r;   out = (h + r c_prev) c + v
//   a token that completes a block:  c_prev = h, h = 0, r = 1
// A thread owns 8 consecutive features (16-byte accesses); the two threads of a head sit in neighbouring lanes,
// so the head's scalar r is read by both before one of them writes it back (in-place state).
// kAdvance: the kernel also moves pos[b] to the next token's position. That needs every thread of a batch row to
// have read pos[b] before one of them writes it, which holds when a row's 2 H threads lie inside one wavefront
// (2 H divides 64: the stored value depends on the loaded one, so the wavefront's load has returned for all its
// lanes before the store is issued); otherwise a second kernel does it.
// ==========================================================================================
template <class E, bool kAdvance>
__global__ __launch_bounds__(256) void phalanx_mix_step_kernel(
    const uint16_t* __restrict__ a_logit, const uint16_t* __restrict__ b_logit, const uint16_t* __restrict__ c_in,
    const uint16_t* __restrict__ v_in, uint16_t* __restrict__ out, float* __restrict__ h, float* __restrict__ r,
    float* __restrict__ c_prev, int* __restrict__ pos, int boundary_all, int block_len, long total, int H,
    int kv_groups) {
  const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const int per_row = 2 * H;  // 8-feature pieces per batch row
  const long brow = idx / per_row;
  const int piece = (int)(idx - brow * per_row);
  const int head = piece >> 1, half = piece & 1;
  const long kv_piece = brow * (2 * (H / kv_groups)) + 2 * (head / kv_groups) + half;
  const int at = pos != nullptr ? pos[brow] : 0;
  const bool boundary = pos != nullptr ? (at == block_len - 1) : (boundary_all != 0);

  const uint32_t aw = a_logit[brow * H + head];
  const float a = clamp_coeff<E>(fast_sigmoid(E::lo(aw)));
  const float r_new = a * r[brow * H + head];
  float bf[8], cf[8], vf[8], hf[8], pf[8], of[8];
  unpack8<E>(*reinterpret_cast<const uint4*>(b_logit + kv_piece * 8), bf);
  unpack8<E>(*reinterpret_cast<const uint4*>(c_in + kv_piece * 8), cf);
  unpack8<E>(*reinterpret_cast<const uint4*>(v_in + idx * 8), vf);
  const float4 h0 = *reinterpret_cast<const float4*>(h + idx * 8), h1 = *reinterpret_cast<const float4*>(h + idx * 8 + 4);
  const float4 p0 = *reinterpret_cast<const float4*>(c_prev + idx * 8), p1 = *reinterpret_cast<const float4*>(c_prev + idx * 8 + 4);
  hf[0] = h0.x; hf[1] = h0.y; hf[2] = h0.z; hf[3] = h0.w; hf[4] = h1.x; hf[5] = h1.y; hf[6] = h1.z; hf[7] = h1.w;
  pf[0] = p0.x; pf[1] = p0.y; pf[2] = p0.z; pf[3] = p0.w; pf[4] = p1.x; pf[5] = p1.y; pf[6] = p1.z; pf[7] = p1.w;
#pragma unroll
  for (int q = 0; q < 8; ++q) {
    hf[q] = fmaf(a, hf[q], fast_sigmoid(bf[q]) * vf[q]);
    of[q] = fmaf(fmaf(r_new, pf[q], hf[q]), cf[q], vf[q]);
  }
  *reinterpret_cast<uint4*>(out + idx * 8) = pack8<E>(of);
  if (boundary) {
    *reinterpret_cast<float4*>(c_prev + idx * 8) = make_float4(hf[0], hf[1], hf[2], hf[3]);
    *reinterpret_cast<float4*>(c_prev + idx * 8 + 4) = make_float4(hf[4], hf[5], hf[6], hf[7]);
#pragma unroll
    for (int q = 0; q < 8; ++q) hf[q] = 0.0f;
  }
  *reinterpret_cast<float4*>(h + idx * 8) = make_float4(hf[0], hf[1], hf[2], hf[3]);
  *reinterpret_cast<float4*>(h + idx * 8 + 4) = make_float4(hf[4], hf[5], hf[6], hf[7]);
  if (half == 0) r[brow * H + head] = boundary ? 1.0f : r_new;
  if constexpr (kAdvance) {
    if (piece == 0) pos[brow] = boundary ? 0 : at + 1;
  }
}

// pos[b] <- position of the next token inside its block
__global__ __launch_bounds__(256) void advance_block_positions_kernel(int* __restrict__ pos, int B, int block_len) {
  const int b = blockIdx.x * blockDim.x + threadIdx.x;
  if (b >= B) return;
  const int next = pos[b] + 1;
  pos[b] = next >= block_len ? 0 : next;
}



// Tile geometry shared by the two kernels: a workgroup is `waves` consecutive blocks of one head slot.
struct TileGrid {
  int tiles;  // time tiles per row: one workgroup each per head slot
  long wgs;
};
TileGrid tile_grid(long B, int slots, int L, int waves) {
  const int nb = L / kTile;
  TileGrid g;
  g.tiles = (nb + waves - 1) / waves;
  const int tg = g.tiles < SPEAR_FUSED_TILE_TIME_GROUP ? g.tiles : SPEAR_FUSED_TILE_TIME_GROUP;  // tile_place()
  g.wgs = B * (long)((g.tiles + tg - 1) / tg) * tg * slots;
  return g;
}

// Workgroups of 8 wavefronts on rows of one head slot and on long rows of up to 32 heads, of 4 otherwise
// (table at the forward kernel).
bool forward_takes_eight_waves(int H, int L) { return H < 16 || (L >= 512 && H <= 32); }

template <class E, int kW, bool kQkv, bool kF32 = false>
void launch_mix_fwd_tile(const MixArgs& p, hipStream_t s) {
  const TileGrid g = tile_grid(p.B, (p.H + kHeadsPerWave - 1) / kHeadsPerWave, p.L, kW);
  hipLaunchKernelGGL((phalanx_mix_fwd_tile_kernel<E, kW, kQkv, kF32>), dim3((unsigned)g.wgs), dim3(64 * kW), 0, s,
                     static_cast<const uint16_t*>(p.a_logit), static_cast<const uint16_t*>(p.b_logit),
                     static_cast<const uint16_t*>(p.c), static_cast<const uint16_t*>(p.v), static_cast<uint16_t*>(p.out),
                     p.c_prev_tail, p.L, p.H, p.kv_groups, g.tiles);
}

// Groups of 1, 2, 4, 8 heads per kv head are summed inside a wavefront's 8 heads; the others take slots cut at
// group borders (head_slot).
bool wide_grouping(int kv_groups) { return kv_groups != 1 && kv_groups != 2 && kv_groups != 4 && kv_groups != 8; }

int backward_slots(int H, int kv_groups) {
  if (!wide_grouping(kv_groups)) return (H + kHeadsPerWave - 1) / kHeadsPerWave;
  const int kv_heads = H / kv_groups;
  if (kv_groups > kHeadsPerWave) return kv_heads;
  const int per_slot = kHeadsPerWave / kv_groups;
  return (kv_heads + per_slot - 1) / per_slot;
}

template <class E, bool kQkv, bool kF32, bool kSums, bool kWide>
void launch_mix_bwd_tile(const MixBwdArgs& p, hipStream_t s) {
  const int slots = backward_slots(p.H, p.kv_groups);
  const TileGrid g = tile_grid(p.B, slots, p.L, kTileWaves);
  auto u = [](const void* q) { return static_cast<const uint16_t*>(q); };
  auto w = [](void* q) { return static_cast<uint16_t*>(q); };
  const int Fkv = (p.H / p.kv_groups) * kChan;
  hipLaunchKernelGGL((phalanx_mix_bwd_tile_kernel<E, kQkv, kF32, kSums, kWide>), dim3((unsigned)g.wgs),
                     dim3(64 * kTileWaves), 0, s, u(p.a_logit), u(p.b_logit), u(p.c), u(p.v), u(p.dout), w(p.da_logit),
                     w(p.db_logit), w(p.dc), w(p.dv), p.sum_da, p.sum_db, p.sum_dc, p.ld_da ? p.ld_da : p.H,
                     p.ld_db ? p.ld_db : Fkv, p.ld_dc ? p.ld_dc : Fkv, p.ld_dv ? p.ld_dv : p.H * kChan, p.L, p.H,
                     p.kv_groups, g.tiles, slots);
}

}  // namespace

long fused_mix_workgroups(long B, int H, int kv_groups, int L, bool backward) {
  if (B <= 0 || H <= 0 || L <= 0 || kv_groups <= 0) return 0;
  if (backward) return tile_grid(B, backward_slots(H, kv_groups), L, kTileWaves).wgs;
  return tile_grid(B, (H + kHeadsPerWave - 1) / kHeadsPerWave, L, forward_takes_eight_waves(H, L) ? 8 : 4).wgs;
}

hipError_t fused_mix_forward(const MixArgs& p, hipStream_t s) {
  const bool eight = forward_takes_eight_waves(p.H, p.L);
  auto by_form = [&](auto e, auto q) {
    using E = decltype(e);
    if (p.f32_out) launch_mix_fwd_tile<E, 4, decltype(q)::value, true>(p, s);  // check mode: one instance per form
    else if (eight) launch_mix_fwd_tile<E, 8, decltype(q)::value>(p, s);
    else launch_mix_fwd_tile<E, 4, decltype(q)::value>(p, s);
  };
  if (p.dtype == kBf16) {
    if (p.qkv) by_form(Bf16{}, std::true_type{});
    else by_form(Bf16{}, std::false_type{});
  } else {
    if (p.qkv) by_form(Fp16{}, std::true_type{});
    else by_form(Fp16{}, std::false_type{});
  }
  return hipGetLastError();
}

long fused_mix_backward_sum_rows(long B, int H, int L) {
  if (B <= 0 || H <= 0 || L <= 0) return 0;
  return B * ((L / kTile + kTileWaves - 1) / kTileWaves);
}

hipError_t fused_mix_backward(const MixBwdArgs& p, hipStream_t s) {
  const bool sums = p.sum_da != nullptr;
  if (sums && (p.qkv || p.f32_grads)) return hipErrorInvalidValue;  // the caller has checked: layer form, 16-bit results
  const bool wide = wide_grouping(p.kv_groups);
  auto by_options = [&](auto e, auto wd) {
    using E = decltype(e);
    constexpr bool kWide = decltype(wd)::value;
    if (sums) launch_mix_bwd_tile<E, false, false, true, kWide>(p, s);
    else if (p.f32_grads && p.qkv) launch_mix_bwd_tile<E, true, true, false, kWide>(p, s);
    else if (p.f32_grads) launch_mix_bwd_tile<E, false, true, false, kWide>(p, s);
    else if (p.qkv) launch_mix_bwd_tile<E, true, false, false, kWide>(p, s);
    else launch_mix_bwd_tile<E, false, false, false, kWide>(p, s);
  };
  if (p.dtype == kBf16) {
    if (wide) by_options(Bf16{}, std::true_type{});
    else by_options(Bf16{}, std::false_type{});
  } else {
    if (wide) by_options(Fp16{}, std::true_type{});
    else by_options(Fp16{}, std::false_type{});
  }
  return hipGetLastError();
}

namespace {

// Finishes the column sums: out[col] = sum over `rows` of part[row * cols + col], for three arrays at once
// (blockIdx.y picks one). A workgroup owns 64 columns; its 16 wavefronts each add up every 16th row (a
// wave-level load is one contiguous 256-byte run of a row), then the 16 partial results meet in LDS. The
// order of the additions is fixed, so equal inputs give equal bits.
constexpr int kSumWaves = 16;
struct SumJob {
  const float* part;
  float* out;
  int cols;
};
__global__ __launch_bounds__(64 * kSumWaves) void finish_column_sums_kernel(SumJob j0, SumJob j1, SumJob j2, long rows) {
  __shared__ float partial[kSumWaves][64];
  const SumJob job = blockIdx.y == 0 ? j0 : (blockIdx.y == 1 ? j1 : j2);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int col = blockIdx.x * 64 + lane;
  const bool live = col < job.cols;  // whole workgroups beyond the array's width fall through to the barrier
  float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
  if (live) {
    const float* p = job.part + col;
    long r = wave;
    for (; r + 3 * kSumWaves < rows; r += 4 * kSumWaves) {
#pragma unroll
      for (int u = 0; u < 4; ++u) acc[u] += p[(r + u * kSumWaves) * job.cols];
    }
    for (; r < rows; r += kSumWaves) acc[0] += p[r * job.cols];
  }
  partial[wave][lane] = (acc[0] + acc[1]) + (acc[2] + acc[3]);
  __syncthreads();
  if (wave == 0 && live) {
    float total = 0.0f;
#pragma unroll
    for (int w = 0; w < kSumWaves; ++w) total += partial[w][lane];
    job.out[col] = total;
  }
}

// Device address of `scratch` on the current device, looked up until it succeeds once per device. A failed
// lookup (a first call that arrives while its stream is being captured, say) is reported and not remembered:
// the next call on that device tries again.
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
float* g_scratch_ptr[kMaxDevices] = {};

hipError_t scratch_of_current_device(float** out) {
  int dev = -1;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) return err;
  if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
  std::lock_guard<std::mutex> hold(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* p = nullptr;
    err = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (err != hipSuccess) return err;
    if (p == nullptr) return hipErrorInvalidSymbol;
    g_scratch_ptr[dev] = static_cast<float*>(p);
  }
  *out = g_scratch_ptr[dev];
  return hipSuccess;
}

}  // namespace

hipError_t fused_mix_step(const MixStepArgs& p, hipStream_t s) {
  const long total = (long)p.B * p.H * 2;
  const unsigned blocks = (unsigned)((total + 255) / 256);
  auto u = [](const void* q) { return static_cast<const uint16_t*>(q); };
  // a batch row's 2 H threads inside one wavefront: the step kernel advances the positions itself
  const bool advance_inside = p.pos != nullptr && 64 % (2 * p.H) == 0;
  auto launch = [&](auto e, auto adv) {
    hipLaunchKernelGGL((phalanx_mix_step_kernel<decltype(e), decltype(adv)::value>), dim3(blocks), dim3(256), 0, s,
                       u(p.a_logit), u(p.b_logit), u(p.c), u(p.v), static_cast<uint16_t*>(p.out), p.h, p.r, p.c_prev, p.pos,
                       p.boundary, p.block_len, total, p.H, p.kv_groups);
  };
  if (p.dtype == kBf16) {
    if (advance_inside) launch(Bf16{}, std::true_type{});
    else launch(Bf16{}, std::false_type{});
  } else {
    if (advance_inside) launch(Fp16{}, std::true_type{});
    else launch(Fp16{}, std::false_type{});
  }
  if (hipError_t err = hipGetLastError(); err != hipSuccess) return err;
  if (p.pos != nullptr && !advance_inside) {  // stream order puts this after every read of pos above
    hipLaunchKernelGGL(advance_block_positions_kernel, dim3((unsigned)((p.B + 255) / 256)), dim3(256), 0, s, p.pos, p.B, p.block_len);
    return hipGetLastError();
  }
  return hipSuccess;
}

long fused_mix_backward_bias_scratch_floats(long B, int H, int kv_groups, int L) {
  if (B <= 0 || H <= 0 || L <= 0 || kv_groups <= 0) return 0;
  const long Fkv = (long)(H / kv_groups) * kChan;
  return fused_mix_backward_sum_rows(B, H, L) * (H + 2 * Fkv);
}

hipError_t fused_mix_backward_bias(const MixBwdArgs& p, float* bias_da, float* bias_db, float* bias_dc, hipStream_t s) {
  if (p.qkv) return hipErrorInvalidValue;
  const long rows = fused_mix_backward_sum_rows(p.B, p.H, p.L);
  const long Fkv = (long)(p.H / p.kv_groups) * kChan;
  if (rows * (p.H + 2 * Fkv) > (long)SPEAR_MIX_BIAS_SCRATCH_FLOATS) return hipErrorInvalidValue;  // the caller has checked
  float* base = nullptr;
  if (hipError_t err = scratch_of_current_device(&base); err != hipSuccess) return err;
  // Nothing has to be cleared: the backward kernel writes every element of the three partial-sum arrays
  // of this shape, and the finishing kernel reads only those.
  MixBwdArgs q = p;
  q.sum_da = base;
  q.sum_db = base + rows * p.H;
  q.sum_dc = q.sum_db + rows * Fkv;
  if (hipError_t err = fused_mix_backward(q, s); err != hipSuccess) return err;
  const SumJob ja{q.sum_da, bias_da, p.H}, jb{q.sum_db, bias_db, (int)Fkv}, jc{q.sum_dc, bias_dc, (int)Fkv};
  const unsigned gx = (unsigned)((Fkv + 63) / 64);  // H <= Fkv * kv_groups / 16: the gate array is never the widest
  const unsigned gxa = (unsigned)((p.H + 63) / 64);
  hipLaunchKernelGGL(finish_column_sums_kernel, dim3(gx > gxa ? gx : gxa, 3), dim3(64 * kSumWaves), 0, s, ja, jb, jc, rows);
  return hipGetLastError();
}

}  // namespace spear_btp
