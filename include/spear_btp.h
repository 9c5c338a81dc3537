/*
 * spear_btp.h -- C ABI of the MI355X (gfx950) Block Two-Pass kernels.
 *
 * This is the drop-in boundary for SPEAR's native BTP extension. The reference binds two
 * functions from its CUDA extension module `spear._btp`:
 *
 *     forward (coeff, x, y, checkpoint, k, wpb)               csrc/btp/_bindings.cu:76-150, 241
 *     backward(coeff, x, dy, checkpoint, dx, dA, k, wpb)      csrc/btp/_bindings.cu:152-229, 242
 *
 * which unpack torch tensors and call the launchers
 *
 *     sss::launch_block_two_pass<T, O, WPB>                   csrc/btp/btp-forward.cu:462-527
 *     sss::launch_btp_backward <T, O, 16, WPB>                csrc/btp/btp-backwards.cu:811-884
 *
 * The entry points below take exactly what those launchers take -- raw device pointers, B, H, L,
 * k and a stream -- plus dtype tags in place of the template parameters. No torch types appear.
 * `wpb` (warps per block) is an sm90 launch-shape knob with no meaning on CDNA4; the host shim
 * validates it for compatibility and does not pass it down.
 *
 * Tensor layouts (all dense, row-major, caller-allocated; spear/ops/btp/interface.py:136-144,155-158):
 *     coeff       [B, H, L]          in_dtype   linear-space decay a_t in (0, 1]
 *     x, dx       [B, H, 16, L]      in_dtype   time is the contiguous axis
 *     y           [B, H, 16, L]      out_dtype  (in_dtype or fp32)
 *     dy          [B, H, 16, L]      dy_dtype   (in_dtype or fp32)
 *     checkpoint  [B, H, L/16, 16]   fp32       slot i-1 = local terminal state of block i-1
 *     dA          [B, H, L]          fp32       every element is written (no accumulation)
 *
 * Requirements: L is a positive multiple of 16; every pointer is 16-byte aligned; k is 1 or 2.
 * Calls are asynchronous on `stream` (a hipStream_t passed as void*, NULL = default stream),
 * allocate nothing, keep no state besides a thread-local error string, and are re-entrant.
 *
 * Return value: 0 on success, a negative SPEAR_BTP_E* code otherwise; spear_btp_last_error()
 * then describes the failure. B*H == 0 or L == 0 is a successful no-op, as in the reference
 * launchers (btp-forward.cu:466, btp-backwards.cu:815).
 */
#ifndef SPEAR_BTP_H_
#define SPEAR_BTP_H_

#ifdef __cplusplus
extern "C" {
#endif

/* element types (template parameters ElementT / ElementO of the reference launchers) */
#define SPEAR_BTP_BF16 0
#define SPEAR_BTP_F16 1
#define SPEAR_BTP_F32 2

/* flags */
#define SPEAR_BTP_WRITE_CHECKPOINT 0x1u /* forward: also store the carry checkpoint            */
#define SPEAR_BTP_PATH_MFMA 0x2u        /* forward and backward: use the MFMA tile kernels (decay matrices built   */
                                        /* per block and multiplied on the matrix cores, the reference's            */
                                        /* formulation; each entry goes in as two 16-bit pieces, so fp32 results    */
                                        /* keep the 1e-4 bound) instead of the fp32 recurrences; the backward then  */
                                        /* takes dy in in_dtype only (SPEAR_BTP_EINVAL for an fp32 dy, which the    */
                                        /* 16-bit operands of the matrix instruction cannot hold) and has no        */
                                        /* SPEAR_BTP_DX_F32                                                          */

#define SPEAR_BTP_DX_F32 0x10u          /* backward: check mode, `dx` is fp32 [B, H, 16, L] and receives the    */
                                        /* kernel's fp32 values instead of their rounding to in_dtype           */

/* error codes */
#define SPEAR_BTP_EINVAL (-1)  /* bad shape, dtype, k, flag or alignment                       */
#define SPEAR_BTP_ENULL (-2)   /* a required pointer is NULL                                   */
#define SPEAR_BTP_ELAUNCH (-3) /* the HIP runtime rejected the launch                          */

/* Replaces spear._btp.forward -> sss::launch_block_two_pass (csrc/btp/_bindings.cu:76-150,
 * csrc/btp/btp-forward.cu:462-527).  `checkpoint` may be NULL unless SPEAR_BTP_WRITE_CHECKPOINT
 * is set. */
int spear_btp_forward(const void* coeff, const void* x, void* y, float* checkpoint, int B, int H,
                      int L, int k, int in_dtype, int out_dtype, unsigned flags, void* stream);

/* Replaces spear._btp.backward -> sss::launch_btp_backward (csrc/btp/_bindings.cu:152-229,
 * csrc/btp/btp-backwards.cu:811-884).  `checkpoint` is accepted for signature compatibility and
 * never read: the carries are recomputed from `coeff` and `x`. The reference fixes dx.dtype == x.dtype
 * (_bindings.cu:52-54), which stays the default; SPEAR_BTP_DX_F32 is the fp32 check mode (arithmetic is fp32
 * either way, the flag only drops the final rounding so that dx can be compared at fp32 tolerances). */
int spear_btp_backward(const void* coeff, const void* x, const void* dy, const float* checkpoint,
                       void* dx, float* dA, int B, int H, int L, int k, int in_dtype, int dy_dtype,
                       unsigned flags, void* stream);

/* Log-space gate variants. They have no counterpart function in the reference, whose op takes
 * the decay already exponentiated and rounded to 16 bits (spear/ops/btp/interface.py:164-188);
 * they serve callers that hold the gate in log space -- the Phalanx layer's -softplus(.) of a
 * logit (spear/nn/phalanx/swr.py:216), or the fp32 log-decay gates of the benchmark
 * configurations -- and want a_t = exp(g_t) formed in fp32 inside the kernel (a 16-bit a_t cannot
 * represent 1 - 1e-4). Same tensors and rules as above except:
 *     gate   [B, H, L] fp32   log-space decay g_t <= 0 (a_t = exp(g_t); exp(g_t) <= 1e-9 counts as 0)
 *     dgate  [B, H, L] fp32   gradient w.r.t. g_t (= a_t * dL/da_t), every element written
 * SPEAR_BTP_PATH_MFMA is not available for these. */
int spear_btp_forward_loggate(const float* gate, const void* x, void* y, float* checkpoint, int B, int H,
                              int L, int k, int x_dtype, int out_dtype, unsigned flags, void* stream);
int spear_btp_backward_loggate(const float* gate, const void* x, const void* dy, void* dx, float* dgate,
                               int B, int H, int L, int k, int x_dtype, int dy_dtype, unsigned flags,
                               void* stream);

/* Fused forward of the Phalanx mixing stage in the layer's own layout. No single counterpart in the
 * reference: it stands for the chain  sigmoid / gate product (spear/nn/phalanx/swr.py:216-219),
 * the transposing .contiguous() copies (spear/ops/btp/interface.py:186-187), the BTP forward, and
 * `y * C + V` with the permute back (swr.py:320-323), for callers that have the projection outputs
 * in [B, L, features] layout (time strided, features contiguous), all in `dtype` (bf16 / fp16):
 *     a_logit [B, L, H]            b_logit, c [B, L, kv_heads * 16]        v, out [B, L, H * 16]
 *     out = btp(sigmoid(a_logit), sigmoid(b_logit) * v) * c + v      (k = 2, fp32 arithmetic)
 * Head h reads b / c of kv head h / (H / kv_heads). Requirements: L % 16 == 0, H % kv_heads == 0 (any H >= 1, any
 * number of heads per kv head, as spear/nn/phalanx/swr.py:37-38 accepts them), 16-byte aligned pointers. */
int spear_phalanx_mix_forward(const void* a_logit, const void* b_logit, const void* c, const void* v, void* out,
                              int B, int L, int H, int kv_heads, int dtype, unsigned flags, void* stream);

/* Flag for spear_phalanx_mix_forward / _backward / _backward_ex: the q/k/v/gate convention of the same
 * kernels, for callers that hold the operands of linear attention rather than the layer's logits:
 *     a_logit  is an fp32 log-decay gate [B, L, H]:       a = exp(gate), formed in fp32 (no 16-bit rounding
 *              of the decay, so gates next to 0 stay distinct from 0)
 *     b_logit  is k [B, L, kv_heads * 16], used as it is (no sigmoid);   c is q;   v is v
 *     out = q * btp(exp(gate), k * v) + v      in the layout [B, L, H, 16]
 * In the backward, da_logit is the fp32 gradient of the gate (dA * a), db_logit = dk, dc = dq, dv = dv.
 * This is the composition written out at spear/nn/phalanx/swr.py:196-221, 311-327 with the two sigmoids
 * left to the caller; the reference has no single function for it. */
#define SPEAR_MIX_QKV_GATE 0x1u

/* Flag for the same three entry points: fp32 check mode. The kernels compute in fp32 either way; with this
 * flag the results are stored as fp32 instead of being rounded to `dtype`, so that they can be held to fp32
 * tolerances: forward `out`; backward `da_logit`, `db_logit`, `dc`, `dv` (row strides then count fp32
 * elements). Inputs keep their types. Not combinable with the column sums of _backward_ex. */
#define SPEAR_MIX_F32_RESULTS 0x2u

/* Backward of spear_phalanx_mix_forward: reads a_logit, b_logit, c, v and the upstream gradient
 * dout [B, L, H * 16]; writes da_logit [B, L, H], db_logit and dc [B, L, kv_heads * 16] (summed over
 * the heads sharing a kv head) and dv [B, L, H * 16] -- every element, no accumulation, all in
 * `dtype`. Any number of heads per kv head: groups of 1, 2, 4 or 8 heads are summed inside a wavefront (the fast
 * path), every other group size through LDS in a fixed order (groups of more than 8 heads are worked through 8
 * heads at a time). It stands for the autograd chain through the ops listed at spear_phalanx_mix_forward; no
 * single counterpart in the reference. */
int spear_phalanx_mix_backward(const void* a_logit, const void* b_logit, const void* c, const void* v,
                               const void* dout, void* da_logit, void* db_logit, void* dc, void* dv, int B, int L,
                               int H, int kv_heads, int dtype, unsigned flags, void* stream);

/* The same backward with two options.
 * (1) Row strides for the outputs: ld_da, ld_db, ld_dc, ld_dv are the elements per time step of the four
 * gradient tensors, 0 meaning dense (the tensor's own width). With strides the four can be column blocks of
 * one [B, L, ld] buffer (all four ld equal, the pointers offset into its first row), which is then the
 * gradient of the four projections' concatenated output: one GEMM each for the input and the weight gradient
 * instead of four. A stride is a number of elements not below the tensor's width, even for db_logit, dc and dv;
 * elements between the blocks are not touched.
 * (2) It leaves the column sums of da_logit, db_logit and dc -- the bias
 * gradients of the projections that produced a_logit, b_logit and c (spear/nn/phalanx/swr.py:157-163 gives
 * proj_a, proj_b and proj_c a bias) -- so that the caller does not read the three gradients again to
 * sum them. The kernel cannot finish the sums without a second pass, so it leaves partial sums in fp32:
 *     sum_da [sum_rows, H],  sum_db [sum_rows, kv_heads * 16],  sum_dc [sum_rows, kv_heads * 16]
 * where row r sums the time steps of one (batch row, tile of 64 time steps) and the caller adds the rows up.
 * sum_rows must equal spear_phalanx_mix_backward_sum_rows(B, L, H) = B * ceil(L / 64). Every element of the
 * three arrays is written; the sums are taken before the gradients are rounded to `dtype`. All three NULL: no
 * sums. With neither option it is exactly spear_phalanx_mix_backward. */
long long spear_phalanx_mix_backward_sum_rows(int B, int L, int H);
int spear_phalanx_mix_backward_ex(const void* a_logit, const void* b_logit, const void* c, const void* v,
                                  const void* dout, void* da_logit, void* db_logit, void* dc, void* dv, int ld_da,
                                  int ld_db, int ld_dc, int ld_dv, float* sum_da, float* sum_db, float* sum_dc,
                                  long long sum_rows, int B, int L, int H, int kv_heads, int dtype, unsigned flags,
                                  void* stream);

/* The same backward for callers that cannot allocate device memory -- code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc -- and therefore cannot bring the partial-sum arrays of
 * spear_phalanx_mix_backward_ex. It has no counterpart in the reference. The partial column sums pass through
 * a device array the library holds statically (SPEAR_MIX_BIAS_SCRATCH_FLOATS floats = 16 MiB on every GPU the
 * library is used on, until the process ends), a second kernel finishes them, and the caller receives the
 * finished bias gradients of proj_a, proj_b and proj_c (spear/nn/phalanx/swr.py:157-163):
 *     bias_da [H],  bias_db [kv_heads * 16],  bias_dc [kv_heads * 16]      fp32, sums over batch and time,
 * taken before the gradients are rounded to `dtype`; all three are required and 16-byte aligned. Everything
 * else is as in spear_phalanx_mix_backward_ex (layer form only, no SPEAR_MIX_QKV_GATE). The call makes no
 * hipMalloc / hipFree and no allocating library call. Limit:
 *     spear_phalanx_mix_backward_sum_rows(B, L, H) * (H + 2 * kv_heads * 16) <= SPEAR_MIX_BIAS_SCRATCH_FLOATS
 * (B = 1024, L = 128, H = kv_heads = 32 needs 2,162,688), otherwise SPEAR_BTP_EINVAL. All calls on one GPU
 * share that GPU's array: calls that overlap in time on one GPU (two streams, two threads) race, so
 * serialise them. Nothing in the array has to be cleared between calls -- each call overwrites all it later
 * reads. The array's address is looked up on the first call on each device; make that first call outside
 * stream capture. */
#define SPEAR_MIX_BIAS_SCRATCH_FLOATS 4194304
int spear_phalanx_mix_backward_bias(const void* a_logit, const void* b_logit, const void* c, const void* v,
                                    const void* dout, void* da_logit, void* db_logit, void* dc, void* dv, int ld_da,
                                    int ld_db, int ld_dc, int ld_dv, float* bias_da, float* bias_db, float* bias_dc,
                                    int B, int L, int H, int kv_heads, int dtype, unsigned flags, void* stream);

/* spear_phalanx_mix_forward for a prompt that token-by-token decoding will continue: the same kernel also leaves
 * the part of the streaming state that depends on the prompt,
 *     c_prev_tail [B, H, 16] fp32   terminal local state of every row's last block
 * (after a whole number of blocks the block-local state is 0 and the gate product 1, so this is all of it).
 * It stands for what parallel_jagged returns beside Y (spear/nn/phalanx/inference.py:327-357) when the layer's gates
 * are applied in the same pass; layer form only. */
int spear_phalanx_mix_prefill(const void* a_logit, const void* b_logit, const void* c, const void* v, void* out,
                              float* c_prev_tail, int B, int L, int H, int kv_heads, int dtype, unsigned flags,
                              void* stream);

/* One decode token of the mixing stage in the layer's own layout: the four projections' outputs for one time step,
 * [B, features] in `dtype`, and the fp32 streaming state, updated in place. It stands for step_jagged
 * (spear/nn/phalanx/inference.py:178-278) fed by the layer's gates (spear/nn/phalanx/swr.py:196-221): the reference
 * has no single function for it (its step takes A_t, X_t, C_t, V_t already gated, expanded over kv heads and
 * reshaped to [B, H, D]).
 *     a_logit [B, H]     b_logit, c [B, kv_heads * 16]     v, out [B, H * 16]
 *     h, c_prev [B, H, 16] fp32     r [B, H] fp32           (zero state: h = 0, r = 1, c_prev = 0)
 *     A = sigmoid(a_logit);  h = A h + sigmoid(b_logit) v;  r = A r;  out = (h + r c_prev) c + v
 *     a token that completes a block:  c_prev = h, h = 0, r = 1
 * Which tokens complete a block: with `pos` (device int32 [B], the position of each batch row's token inside its
 * block, 0 .. block_len-1) every row decides for itself (pos[b] == block_len - 1) and the call advances pos by one
 * step (wrapping to 0), so that one captured HIP graph serves every token and batch rows may be at different
 * positions; with pos == NULL the host decides for all rows through `boundary`. Calls on one state must not
 * overlap. Nothing is allocated; with `pos` the call launches one kernel when 2 * H divides 64 (a batch row's
 * threads then share a wavefront and advance the position themselves), two otherwise. Alignment: b_logit, c, v, out, h and
 * c_prev 16 bytes; a_logit 2 and r 4 bytes (one token's row of a [tokens, B, H] tensor can be passed as it lies). */
int spear_phalanx_mix_step(const void* a_logit, const void* b_logit, const void* c, const void* v, void* out, float* h,
                           float* r, float* c_prev, int* pos, int boundary, int block_len, int B, int H, int kv_heads,
                           int dtype, unsigned flags, void* stream);

/* ---- streaming form: prompt prefill with state hand-over, and the one-token decode step --------
 * They replace the PyTorch loops of spear/nn/phalanx/inference.py. Tensors are dense, row-major:
 *     a         [B, H, L]      a_dtype (x_dtype or fp32)   a_t, or log(a_t) with SPEAR_JAGGED_LOG_A
 *     x, c, v   [B, H, D, L]   x_dtype (bf16 / fp16 / fp32)
 *     y         [B, H, D, L]   x_dtype
 *     h, c_prev [B, H, D]      state_dtype (x_dtype or fp32)
 *     r         [B, H]         r_dtype (any of the three)
 * Arithmetic is fp32 whatever the storage types. */
#define SPEAR_JAGGED_LOG_A 0x4u /* a / a_t hold log(a_t)                                         */
#define SPEAR_JAGGED_LOG_R 0x8u /* step: the r buffers hold log(r)                               */

/* Replaces parallel_jagged (spear/nn/phalanx/inference.py:281-360) and, with c = v = NULL and no state
 * pointers, jagged_band_infer_sequential (inference.py:36-92; `carry_init`, [B, H, D] in state_dtype or
 * NULL, is the carry into the first block):
 *     y_t = (h_loc_t + r_t * c_prev) * c_t + v_t      h_loc, r: block-local scan and gate product
 * and writes the state after step L-1 as the reference assembles it (inference.py:327-357): h_tail the
 * block-local state, r_tail the in-block gate product (1 when L ends a block), c_prev_tail the terminal
 * local state of the last completed block. The three state pointers are given together or all NULL.
 * Any L >= 0, D > 0, block_len > 0, pointers aligned to their element size. 16-bit tensors with D = 16,
 * block_len = 16 and a in x_dtype (a_t or log a_t) or fp32 log(a_t) run the tiled kernel (HBM-bound; rows
 * whose length is not a multiple of 8 or that are not 16-byte aligned are realigned in registers, at
 * 0.5-0.65 of peak instead of 0.75); everything else (fp32 tensors, other D / block_len, fp32 linear a_t)
 * runs an element-granular kernel. */
int spear_jagged_prefill(const void* a, const void* x, const void* c, const void* v, const void* carry_init, void* y,
                         void* h_tail, void* r_tail, void* c_prev_tail, int B, int H, int D, int L, int block_len,
                         int a_dtype, int x_dtype, int state_dtype, int r_dtype, unsigned flags, void* stream);

/* Replaces step_jagged (spear/nn/phalanx/inference.py:178-278) and, with c_t = v_t = NULL,
 * JaggedBandState.step (inference.py:121-140). One token for every (batch, head):
 *     h = a_t * h_in + x_t;   r = a_t * r_in   (or exp(r_in + log max(a_t, tiny)) with SPEAR_JAGGED_LOG_R)
 *     y_t = (h + r * c_prev_in) * c_t + v_t
 * `boundary` != 0 says this token completes a block: then c_prev_out = h, h_out = 0, r_out = 1 (log: 0);
 * otherwise h_out = h, r_out = r (log: log r) and c_prev_out is not written (may be NULL). a_t [B, H] in
 * a_dtype; x_t, c_t, v_t, y_t [B, H, D] in x_dtype. Each output state buffer may be the same memory as
 * its input (in-place update); calls on one state must not overlap. */
int spear_jagged_step(const void* a_t, const void* x_t, const void* c_t, const void* v_t, void* y_t, const void* h_in,
                      const void* r_in, const void* c_prev_in, void* h_out, void* r_out, void* c_prev_out, int B, int H,
                      int D, int boundary, int a_dtype, int x_dtype, int state_dtype, int r_dtype, unsigned flags,
                      float tiny, void* stream);

/* Message for the last failing call on this thread ("" if none).  The reference prints launch
 * failures and carries on (csrc/btp/btp-forward.cu:501-520); here they are reported. */
const char* spear_btp_last_error(void);

/* ABI version of this header: bumped whenever a signature above changes. */
int spear_btp_abi_version(void);

#ifdef __cplusplus
}
#endif
#endif /* SPEAR_BTP_H_ */
