// Host-side argument blocks and launcher entry points shared by the C ABI and the kernel files.
// They stand where the reference has its templated launchers
// (csrc/btp/btp-forward.cu:462-527, csrc/btp/btp-backwards.cu:811-884).
#pragma once

#include <hip/hip_runtime.h>

namespace spear_btp {

// Must match SPEAR_BTP_BF16 / _F16 / _F32 of the public header.
enum Dtype : int { kBf16 = 0, kF16 = 1, kF32 = 2 };

struct FwdArgs {
  const void* coeff;  // 16-bit linear-space decay, or fp32 log-space gate when log_gate is set
  const void* x;
  void* y;
  float* checkpoint;  // nullptr: do not store the carry checkpoint
  int B, H, L, k;
  int in_dtype, out_dtype;
  bool log_gate = false;
};

struct BwdArgs {
  const void* coeff;
  const void* x;
  const void* dy;
  void* dx;
  float* dA;  // d/d coeff, or d/d gate when log_gate is set
  int B, H, L, k;
  int in_dtype, dy_dtype;
  bool log_gate = false;
  bool dx_f32 = false;  // check mode: dx is fp32 [B, H, 16, L] (the kernel's fp32 values, not rounded to in_dtype)
};

// Exact-fp32 recurrence kernels (btp_scan.hip).
hipError_t scan_forward(const FwdArgs& p, hipStream_t s);
hipError_t scan_backward(const BwdArgs& p, hipStream_t s);

// MFMA tile kernels (btp_mfma.hip), bf16 or fp16 inputs; the forward stores no checkpoint, the backward has
// neither log-space gates nor the fp32-dx check mode and takes dy in the inputs' type only.
hipError_t mfma_forward(const FwdArgs& p, hipStream_t s);
hipError_t mfma_backward(const BwdArgs& p, hipStream_t s);

// Fused layer-layout forward (btp_fused.hip): all operands [B, L, features], 16-bit.
struct MixArgs {
  const void* a_logit;  // [B, L, H]
  const void* b_logit;  // [B, L, (H / kv_groups) * 16]
  const void* c;        // [B, L, (H / kv_groups) * 16]
  const void* v;        // [B, L, H * 16]
  void* out;            // [B, L, H * 16]
  int B, L, H, kv_groups;
  int dtype;
  // q/k/v/gate form: a_logit is an fp32 log-decay gate (a = exp(gate)), b_logit is k (used as it is), c is q
  bool qkv = false;
  bool f32_out = false;  // check mode: `out` is fp32
  // null, or fp32 [B, H, 16]: receives the terminal local state of every row's last block (the c_prev of the
  // streaming state after this prompt)
  float* c_prev_tail = nullptr;
};
hipError_t fused_mix_forward(const MixArgs& p, hipStream_t s);
// Workgroups the forward / backward kernel launches for a shape (must fit a 31-bit grid).
long fused_mix_workgroups(long B, int H, int kv_groups, int L, bool backward);

// Fused layer-layout backward (btp_fused.hip); kv_groups = H / kv_heads, any positive integer.
struct MixBwdArgs {
  const void *a_logit, *b_logit, *c, *v, *dout;  // [B,L,H], [B,L,Hkv*16] x 2, [B,L,H*16] x 2
  void *da_logit, *db_logit, *dc, *dv;           // same shapes as the inputs they belong to
  int B, L, H, kv_groups;
  int dtype;
  // all three null, or fp32 [fused_mix_backward_sum_rows(B, H, L), H | Hkv*16 | Hkv*16]: sums over the time steps of
  // one (batch row, time tile) per row
  float *sum_da = nullptr, *sum_db = nullptr, *sum_dc = nullptr;
  // elements per time step of each gradient tensor; 0 = dense (its own width)
  int ld_da = 0, ld_db = 0, ld_dc = 0, ld_dv = 0;
  bool qkv = false;  // as in MixArgs; da_logit is then the fp32 gradient of the gate
  bool f32_grads = false;  // check mode: da_logit, db_logit, dc, dv are fp32
};
hipError_t fused_mix_backward(const MixBwdArgs& p, hipStream_t s);
long fused_mix_backward_sum_rows(long B, int H, int L);
// The same backward with the column sums finished inside the library: the per-tile partial sums go through
// a static device array instead of caller memory, and bias_da [H], bias_db / bias_dc [(H / kv_groups) * 16]
// receive the sums over batch and time. Allocates nothing. `p.sum_*` are ignored.
hipError_t fused_mix_backward_bias(const MixBwdArgs& p, float* bias_da, float* bias_db, float* bias_dc, hipStream_t s);
long fused_mix_backward_bias_scratch_floats(long B, int H, int kv_groups, int L);

// One decode token of the mixing stage in the layer's layout (btp_fused.hip): 16-bit [B, features] operands,
// fp32 state updated in place. pos: null, or the position inside its block of every batch row's token (device
// int32 [B]), which decides the block boundary per row and is advanced by the call; else `boundary` decides.
struct MixStepArgs {
  const void *a_logit, *b_logit, *c, *v;  // [B, H], [B, Hkv*16] x 2, [B, H*16]
  void* out;                              // [B, H*16]
  float *h, *r, *c_prev;                  // [B, H, 16], [B, H], [B, H, 16]
  int* pos;
  int boundary, block_len;
  int B, H, kv_groups;
  int dtype;
};
hipError_t fused_mix_step(const MixStepArgs& p, hipStream_t s);

// Streaming form (btp_jagged.hip). Tensors [B, H, D, L] / [B, H, L]; state vectors [B, H, D] / [B, H].
struct JagPrefillArgs {
  const void *a, *x, *c, *v;  // c and v both null: no "* C + V" epilogue
  const void* carry_init;     // null, or the carry into the first block, [B, H, D] in state_dtype
  void* y;
  void *h_tail, *r_tail, *c_prev_tail;  // all null: no state wanted
  int B, H, D, L, block_len;
  int a_dtype, x_dtype, state_dtype, r_dtype;
  bool log_a;    // a holds log(a_t)
  bool aligned;  // every tensor pointer is 16-byte aligned (the tiled kernel needs it)
};
bool jagged_prefill_is_tiled(const JagPrefillArgs& p);
hipError_t jagged_prefill(const JagPrefillArgs& p, hipStream_t s);

struct JagStepArgs {
  const void *a_t, *x_t, *c_t, *v_t;  // c_t and v_t both null: y_t without "* C + V"
  void* y_t;
  const void *h_in, *r_in, *c_prev_in;
  void *h_out, *r_out, *c_prev_out;  // may alias the inputs; c_prev_out is written only at a block boundary
  int B, H, D;
  int boundary;  // this token completes a block: snapshot the carry, reset the local state
  int a_dtype, x_dtype, state_dtype, r_dtype;
  int log_a, log_r;  // a_t holds log(a_t); the r buffers hold log(r)
  float tiny;        // lower clamp of a_t before the logarithm (log_r only)
  bool aligned;      // every tensor pointer is 16-byte aligned (the 8-channel kernel needs it)
};
hipError_t jagged_step(const JagStepArgs& p, hipStream_t s);

// ---- measurement aids (btp_probe.hip), not part of the operator -------------------------------------------
// Records / clears the calling thread's error string (btp_capi.hip) for entry points that live in other files.
int report_error(int code, const char* fmt, ...);
void clear_error();

// Plain copy kernel used for bandwidth / counter calibration.
hipError_t device_copy(const void* src, void* dst, unsigned long long bytes, hipStream_t s);

// Slab-shaped non-temporal copy (b == nullptr) or two-input combine, for measuring what the memory
// system gives the operator's access pattern.
hipError_t stream_probe(const void* a, const void* b, void* dst, unsigned long long bytes, hipStream_t s);
// The same traffic in other launch shapes (0 = the one above, 1..4 see stream_probe_shape_kernel).
hipError_t stream_probe_shape(const void* a, const void* b, void* dst, unsigned long long bytes, int shape, hipStream_t s);
// The probe with the fused kernels' stream counts: (n_src, n_dst) = (3, 1) or (4, 3); `compute` adds a compute phase.
hipError_t stream_probe_mix(const void* const* src, int n_src, void* const* dst, int n_dst, unsigned long long bytes,
                            bool compute, hipStream_t s);

}  // namespace spear_btp
