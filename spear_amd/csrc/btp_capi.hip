// C ABI of the BTP library: argument validation, error reporting, dispatch to the kernel
// launchers. Validation mirrors what the reference's binding checks before launching
// (csrc/btp/_bindings.cu:19-60) for the properties that are visible at this level (k, dtypes),
// and adds the ones the reference leaves unchecked (L % 16, alignment, NULL pointers).
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#include "../../include/spear_btp.h"
#include "btp_launch.h"

namespace {

thread_local char g_error[256] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

}  // namespace

namespace spear_btp {

// Error reporting for the entry points that live in other files (btp_probe.hip).
int report_error(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}
void clear_error() { g_error[0] = '\0'; }

}  // namespace spear_btp

namespace {

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

bool dtype_ok(int d) { return d == SPEAR_BTP_BF16 || d == SPEAR_BTP_F16 || d == SPEAR_BTP_F32; }

int check_common(const char* who, int B, int H, int L, int k, int in_dtype, int io_dtype, const char* io_name,
                 unsigned flags, unsigned allowed_flags) {
  if (B < 0 || H < 0 || L < 0) return fail(SPEAR_BTP_EINVAL, "%s: negative dimension (B=%d H=%d L=%d)", who, B, H, L);
  if (L % 16 != 0) return fail(SPEAR_BTP_EINVAL, "%s: Length L must be multiple of 16 (got %d)", who, L);
  if (k != 1 && k != 2) return fail(SPEAR_BTP_EINVAL, "%s: k must be 1 or 2.", who);
  if (in_dtype != SPEAR_BTP_BF16 && in_dtype != SPEAR_BTP_F16)
    return fail(SPEAR_BTP_EINVAL, "%s: coeff must be float16 or bfloat16.", who);
  if (io_dtype != SPEAR_BTP_F32 && io_dtype != in_dtype)
    return fail(SPEAR_BTP_EINVAL, "%s: %s must be float32 or match x dtype.", who, io_name);
  if (flags & ~allowed_flags) return fail(SPEAR_BTP_EINVAL, "%s: unknown flag bits 0x%x", who, flags & ~allowed_flags);
  if ((long long)B * H * 16ll * L >= (1ll << 40)) return fail(SPEAR_BTP_EINVAL, "%s: tensor too large", who);
  return 0;
}

}  // namespace

extern "C" {

int spear_btp_abi_version(void) { return 18; }

const char* spear_btp_last_error(void) { return g_error; }

int spear_btp_forward(const void* coeff, const void* x, void* y, float* checkpoint, int B, int H, int L, int k,
                      int in_dtype, int out_dtype, unsigned flags, void* stream) {
  g_error[0] = '\0';
  if (int rc = check_common("spear_btp_forward", B, H, L, k, in_dtype, out_dtype, "y", flags,
                            SPEAR_BTP_WRITE_CHECKPOINT | SPEAR_BTP_PATH_MFMA))
    return rc;
  if ((long long)B * H == 0 || L == 0) return 0;
  const bool want_ckpt = (flags & SPEAR_BTP_WRITE_CHECKPOINT) != 0;
  if (!coeff || !x || !y || (want_ckpt && !checkpoint))
    return fail(SPEAR_BTP_ENULL, "spear_btp_forward: NULL tensor pointer");
  if (!aligned16(coeff) || !aligned16(x) || !aligned16(y) || (want_ckpt && !aligned16(checkpoint)))
    return fail(SPEAR_BTP_EINVAL, "spear_btp_forward: tensor pointers must be 16-byte aligned");
  const bool mfma = (flags & SPEAR_BTP_PATH_MFMA) != 0;
  if (mfma && want_ckpt)
    return fail(SPEAR_BTP_EINVAL, "spear_btp_forward: the MFMA path does not store the carry checkpoint");

  spear_btp::FwdArgs a{coeff, x, y, want_ckpt ? checkpoint : nullptr, B, H, L, k, in_dtype, out_dtype};
  const hipStream_t hs = static_cast<hipStream_t>(stream);
  const hipError_t err = mfma ? spear_btp::mfma_forward(a, hs) : spear_btp::scan_forward(a, hs);
  if (err != hipSuccess) return fail(SPEAR_BTP_ELAUNCH, "spear_btp_forward: launch failed: %s", hipGetErrorString(err));
  return 0;
}

int spear_btp_backward(const void* coeff, const void* x, const void* dy, const float* checkpoint, void* dx, float* dA,
                       int B, int H, int L, int k, int in_dtype, int dy_dtype, unsigned flags, void* stream) {
  (void)checkpoint;  // carries are recomputed from coeff and x
  g_error[0] = '\0';
  if (int rc = check_common("spear_btp_backward", B, H, L, k, in_dtype, dy_dtype, "dy", flags,
                            SPEAR_BTP_PATH_MFMA | SPEAR_BTP_DX_F32))
    return rc;
  if ((long long)B * H == 0 || L == 0) return 0;
  if (!coeff || !x || !dy || !dx || !dA) return fail(SPEAR_BTP_ENULL, "spear_btp_backward: NULL tensor pointer");
  if (!aligned16(coeff) || !aligned16(x) || !aligned16(dy) || !aligned16(dx) || !aligned16(dA))
    return fail(SPEAR_BTP_EINVAL, "spear_btp_backward: tensor pointers must be 16-byte aligned");
  const bool mfma = (flags & SPEAR_BTP_PATH_MFMA) != 0;
  if (mfma && (flags & SPEAR_BTP_DX_F32))
    return fail(SPEAR_BTP_EINVAL, "spear_btp_backward: the MFMA path has no fp32 dx (SPEAR_BTP_DX_F32)");
  if (mfma && dy_dtype == SPEAR_BTP_F32)
    return fail(SPEAR_BTP_EINVAL,
                "spear_btp_backward: the MFMA path takes dy in the inputs' 16-bit type (the matrix instruction's operand "
                "width) and does not round a float32 dy silently; use the default path, or give the forward an output "
                "in the inputs' dtype so that dy arrives in it");

  spear_btp::BwdArgs a{coeff, x, dy, dx, dA, B, H, L, k, in_dtype, dy_dtype, false, (flags & SPEAR_BTP_DX_F32) != 0};
  const hipStream_t hs = static_cast<hipStream_t>(stream);
  const hipError_t err = mfma ? spear_btp::mfma_backward(a, hs) : spear_btp::scan_backward(a, hs);
  if (err != hipSuccess) return fail(SPEAR_BTP_ELAUNCH, "spear_btp_backward: launch failed: %s", hipGetErrorString(err));
  return 0;
}

int spear_btp_forward_loggate(const float* gate, const void* x, void* y, float* checkpoint, int B, int H, int L, int k,
                              int x_dtype, int out_dtype, unsigned flags, void* stream) {
  g_error[0] = '\0';
  if (int rc = check_common("spear_btp_forward_loggate", B, H, L, k, x_dtype, out_dtype, "y", flags,
                            SPEAR_BTP_WRITE_CHECKPOINT))
    return rc;
  if ((long long)B * H == 0 || L == 0) return 0;
  const bool want_ckpt = (flags & SPEAR_BTP_WRITE_CHECKPOINT) != 0;
  if (!gate || !x || !y || (want_ckpt && !checkpoint))
    return fail(SPEAR_BTP_ENULL, "spear_btp_forward_loggate: NULL tensor pointer");
  if (!aligned16(gate) || !aligned16(x) || !aligned16(y) || (want_ckpt && !aligned16(checkpoint)))
    return fail(SPEAR_BTP_EINVAL, "spear_btp_forward_loggate: tensor pointers must be 16-byte aligned");
  spear_btp::FwdArgs a{gate, x, y, want_ckpt ? checkpoint : nullptr, B, H, L, k, x_dtype, out_dtype, true};
  const hipError_t err = spear_btp::scan_forward(a, static_cast<hipStream_t>(stream));
  if (err != hipSuccess)
    return fail(SPEAR_BTP_ELAUNCH, "spear_btp_forward_loggate: launch failed: %s", hipGetErrorString(err));
  return 0;
}

int spear_btp_backward_loggate(const float* gate, const void* x, const void* dy, void* dx, float* dgate, int B, int H,
                               int L, int k, int x_dtype, int dy_dtype, unsigned flags, void* stream) {
  g_error[0] = '\0';
  if (int rc = check_common("spear_btp_backward_loggate", B, H, L, k, x_dtype, dy_dtype, "dy", flags, SPEAR_BTP_DX_F32))
    return rc;
  if ((long long)B * H == 0 || L == 0) return 0;
  if (!gate || !x || !dy || !dx || !dgate)
    return fail(SPEAR_BTP_ENULL, "spear_btp_backward_loggate: NULL tensor pointer");
  if (!aligned16(gate) || !aligned16(x) || !aligned16(dy) || !aligned16(dx) || !aligned16(dgate))
    return fail(SPEAR_BTP_EINVAL, "spear_btp_backward_loggate: tensor pointers must be 16-byte aligned");
  spear_btp::BwdArgs a{gate, x, dy, dx, dgate, B, H, L, k, x_dtype, dy_dtype, true, (flags & SPEAR_BTP_DX_F32) != 0};
  const hipError_t err = spear_btp::scan_backward(a, static_cast<hipStream_t>(stream));
  if (err != hipSuccess)
    return fail(SPEAR_BTP_ELAUNCH, "spear_btp_backward_loggate: launch failed: %s", hipGetErrorString(err));
  return 0;
}

int spear_phalanx_mix_forward(const void* a_logit, const void* b_logit, const void* c, const void* v, void* out, int B,
                              int L, int H, int kv_heads, int dtype, unsigned flags, void* stream) {
  return spear_phalanx_mix_prefill(a_logit, b_logit, c, v, out, nullptr, B, L, H, kv_heads, dtype, flags, stream);
}

int spear_phalanx_mix_prefill(const void* a_logit, const void* b_logit, const void* c, const void* v, void* out,
                              float* c_prev_tail, int B, int L, int H, int kv_heads, int dtype, unsigned flags,
                              void* stream) {
  g_error[0] = '\0';
  const char* who = c_prev_tail ? "spear_phalanx_mix_prefill" : "spear_phalanx_mix_forward";
  if (B < 0 || L < 0 || H < 0) return fail(SPEAR_BTP_EINVAL, "%s: negative dimension (B=%d L=%d H=%d)", who, B, L, H);
  if (L % 16 != 0) return fail(SPEAR_BTP_EINVAL, "%s: Length L must be multiple of 16 (got %d)", who, L);
  if (kv_heads <= 0 || H % kv_heads != 0)
    return fail(SPEAR_BTP_EINVAL, "%s: heads (%d) must be divisible by kv_heads (%d)", who, H, kv_heads);
  if (dtype != SPEAR_BTP_BF16 && dtype != SPEAR_BTP_F16)
    return fail(SPEAR_BTP_EINVAL, "%s: tensors must be float16 or bfloat16.", who);
  const unsigned known = SPEAR_MIX_QKV_GATE | SPEAR_MIX_F32_RESULTS;
  if (flags & ~known) return fail(SPEAR_BTP_EINVAL, "%s: unknown flag bits 0x%x", who, flags & ~known);
  const bool f32 = (flags & SPEAR_MIX_F32_RESULTS) != 0;
  if ((long long)B * L * H * 16ll >= (1ll << 40)) return fail(SPEAR_BTP_EINVAL, "%s: tensor too large", who);
  if ((long long)L * H * (f32 ? 64ll : 32ll) >= (1ll << 31))  // a batch row is addressed through one 32-bit buffer resource
    return fail(SPEAR_BTP_EINVAL, "%s: one batch row (L * H * 16 elements) must stay below 2 GiB", who);
  if ((long long)B * H == 0 || L == 0) return 0;
  if (spear_btp::fused_mix_workgroups(B, H, H / kv_heads, L, false) >= (1ll << 31))
    return fail(SPEAR_BTP_EINVAL, "%s: too many tiles for one launch (B * L / 64 * H / 8 must stay below 2^31)", who);
  if (!a_logit || !b_logit || !c || !v || !out) return fail(SPEAR_BTP_ENULL, "%s: NULL tensor pointer", who);
  if (!aligned16(a_logit) || !aligned16(b_logit) || !aligned16(c) || !aligned16(v) || !aligned16(out))
    return fail(SPEAR_BTP_EINVAL, "%s: tensor pointers must be 16-byte aligned", who);
  if (c_prev_tail && !aligned16(c_prev_tail)) return fail(SPEAR_BTP_EINVAL, "%s: tensor pointers must be 16-byte aligned", who);
  if (c_prev_tail && (flags & SPEAR_MIX_QKV_GATE))
    return fail(SPEAR_BTP_EINVAL, "%s: the hand-over state belongs to the layer form, not SPEAR_MIX_QKV_GATE", who);
  spear_btp::MixArgs a{a_logit, b_logit, c, v, out, B, L, H, H / kv_heads, dtype, (flags & SPEAR_MIX_QKV_GATE) != 0, f32,
                       c_prev_tail};
  const hipError_t err = spear_btp::fused_mix_forward(a, static_cast<hipStream_t>(stream));
  if (err != hipSuccess) return fail(SPEAR_BTP_ELAUNCH, "%s: launch failed: %s", who, hipGetErrorString(err));
  return 0;
}

long long spear_phalanx_mix_backward_sum_rows(int B, int L, int H) {
  if (B <= 0 || L <= 0 || H <= 0 || L % 16 != 0) return 0;
  return spear_btp::fused_mix_backward_sum_rows(B, H, L);
}

int spear_phalanx_mix_backward(const void* a_logit, const void* b_logit, const void* c, const void* v, const void* dout,
                               void* da_logit, void* db_logit, void* dc, void* dv, int B, int L, int H, int kv_heads,
                               int dtype, unsigned flags, void* stream) {
  return spear_phalanx_mix_backward_ex(a_logit, b_logit, c, v, dout, da_logit, db_logit, dc, dv, 0, 0, 0, 0, nullptr,
                                       nullptr, nullptr, 0, B, L, H, kv_heads, dtype, flags, stream);
}

// Checks shared by the fused backward entry points; 1 = nothing to do (empty tensors), 0 = go on.
static int check_mix_backward(const char* who, const void* const (&ptrs)[9], const int (&lds)[4], int B, int L, int H,
                              int kv_heads, int dtype, unsigned flags, unsigned allowed_flags) {
  if (B < 0 || L < 0 || H < 0) return fail(SPEAR_BTP_EINVAL, "%s: negative dimension (B=%d L=%d H=%d)", who, B, L, H);
  if (L % 16 != 0) return fail(SPEAR_BTP_EINVAL, "%s: Length L must be multiple of 16 (got %d)", who, L);
  if (kv_heads <= 0 || H % kv_heads != 0)
    return fail(SPEAR_BTP_EINVAL, "%s: heads (%d) must be divisible by kv_heads (%d)", who, H, kv_heads);
  if (dtype != SPEAR_BTP_BF16 && dtype != SPEAR_BTP_F16)
    return fail(SPEAR_BTP_EINVAL, "%s: tensors must be float16 or bfloat16.", who);
  if (flags & ~allowed_flags) return fail(SPEAR_BTP_EINVAL, "%s: unknown flag bits 0x%x", who, flags & ~allowed_flags);
  const bool qkv = (flags & SPEAR_MIX_QKV_GATE) != 0, f32 = (flags & SPEAR_MIX_F32_RESULTS) != 0;
  if ((long long)B * L * H * 16ll >= (1ll << 40)) return fail(SPEAR_BTP_EINVAL, "%s: tensor too large", who);
  if ((long long)L * H * (f32 ? 64ll : 32ll) >= (1ll << 31))  // a batch row is addressed through one 32-bit buffer resource
    return fail(SPEAR_BTP_EINVAL, "%s: one batch row (L * H * 16 elements) must stay below 2 GiB", who);
  if ((long long)B * H == 0 || L == 0) return 1;
  if (spear_btp::fused_mix_workgroups(B, H, H / kv_heads, L, true) >= (1ll << 31))
    return fail(SPEAR_BTP_EINVAL, "%s: too many tiles for one launch (B * L / 64 * H / 8 must stay below 2^31)", who);
  for (const void* q : ptrs) {
    if (!q) return fail(SPEAR_BTP_ENULL, "%s: NULL tensor pointer", who);
    if (!aligned16(q)) return fail(SPEAR_BTP_EINVAL, "%s: tensor pointers must be 16-byte aligned", who);
  }
  const int widths[4] = {H, kv_heads * 16, kv_heads * 16, H * 16};
  for (int i = 0; i < 4; ++i) {
    if (lds[i] == 0) continue;
    // db, dc, dv are stored as pairs of elements (32-bit, or 64-bit in the check mode): their rows start on even
    // elements; da_logit is stored element by element
    if (lds[i] < widths[i] || (i != 0 && lds[i] % 2 != 0))
      return fail(SPEAR_BTP_EINVAL, "%s: a gradient's row stride must be 0 (dense) or a number of elements not below its width, even for db_logit, dc and dv (got %d for width %d)", who, lds[i], widths[i]);
    if ((long long)L * lds[i] * ((i == 0 && qkv) || f32 ? 4ll : 2ll) >= (1ll << 31))
      return fail(SPEAR_BTP_EINVAL, "%s: one batch row (L * row stride) must stay below 2 GiB", who);
  }
  return 0;
}

int spear_phalanx_mix_backward_ex(const void* a_logit, const void* b_logit, const void* c, const void* v,
                                  const void* dout, void* da_logit, void* db_logit, void* dc, void* dv, int ld_da,
                                  int ld_db, int ld_dc, int ld_dv, float* sum_da, float* sum_db, float* sum_dc,
                                  long long sum_rows, int B, int L, int H, int kv_heads, int dtype, unsigned flags,
                                  void* stream) {
  g_error[0] = '\0';
  const char* who = "spear_phalanx_mix_backward";
  const void* const ptrs[9] = {a_logit, b_logit, c, v, dout, da_logit, db_logit, dc, dv};
  const int lds[4] = {ld_da, ld_db, ld_dc, ld_dv};
  if (int rc = check_mix_backward(who, ptrs, lds, B, L, H, kv_heads, dtype, flags, SPEAR_MIX_QKV_GATE | SPEAR_MIX_F32_RESULTS))
    return rc < 0 ? rc : 0;
  const bool qkv = (flags & SPEAR_MIX_QKV_GATE) != 0, f32 = (flags & SPEAR_MIX_F32_RESULTS) != 0;
  const bool sums = sum_da || sum_db || sum_dc;
  if (sums && qkv) return fail(SPEAR_BTP_EINVAL, "%s: column sums are for the layer form, not SPEAR_MIX_QKV_GATE", who);
  if (sums && f32) return fail(SPEAR_BTP_EINVAL, "%s: column sums are not available with SPEAR_MIX_F32_RESULTS", who);
  if (sums) {
    if (!sum_da || !sum_db || !sum_dc) return fail(SPEAR_BTP_ENULL, "%s: the three sum arrays must be given together", who);
    if (!aligned16(sum_da) || !aligned16(sum_db) || !aligned16(sum_dc))
      return fail(SPEAR_BTP_EINVAL, "%s: sum arrays must be 16-byte aligned", who);
    const long long want = spear_btp::fused_mix_backward_sum_rows(B, H, L);
    if (sum_rows != want)
      return fail(SPEAR_BTP_EINVAL, "%s: sum arrays must have %lld rows for this shape (got %lld)", who, want, sum_rows);
  }
  spear_btp::MixBwdArgs a{a_logit, b_logit, c, v, dout, da_logit, db_logit, dc, dv, B, L, H, H / kv_heads, dtype,
                          sum_da, sum_db, sum_dc, ld_da, ld_db, ld_dc, ld_dv, qkv, f32};
  const hipError_t err = spear_btp::fused_mix_backward(a, static_cast<hipStream_t>(stream));
  if (err != hipSuccess) return fail(SPEAR_BTP_ELAUNCH, "%s: launch failed: %s", who, hipGetErrorString(err));
  return 0;
}

int spear_phalanx_mix_backward_bias(const void* a_logit, const void* b_logit, const void* c, const void* v,
                                    const void* dout, void* da_logit, void* db_logit, void* dc, void* dv, int ld_da,
                                    int ld_db, int ld_dc, int ld_dv, float* bias_da, float* bias_db, float* bias_dc,
                                    int B, int L, int H, int kv_heads, int dtype, unsigned flags, void* stream) {
  g_error[0] = '\0';
  const char* who = "spear_phalanx_mix_backward_bias";
  const void* const ptrs[9] = {a_logit, b_logit, c, v, dout, da_logit, db_logit, dc, dv};
  const int lds[4] = {ld_da, ld_db, ld_dc, ld_dv};
  const int rc = check_mix_backward(who, ptrs, lds, B, L, H, kv_heads, dtype, flags, 0u);
  if (rc < 0) return rc;
  if (!bias_da || !bias_db || !bias_dc) return fail(SPEAR_BTP_ENULL, "%s: the three bias gradient arrays are required", who);
  if (!aligned16(bias_da) || !aligned16(bias_db) || !aligned16(bias_dc))
    return fail(SPEAR_BTP_EINVAL, "%s: bias gradient arrays must be 16-byte aligned", who);
  if (rc == 1) return 0;  // empty tensors: nothing is read or written, as in the other entry points
  const long long need = spear_btp::fused_mix_backward_bias_scratch_floats(B, H, H / kv_heads, L);
  if (need > (long long)SPEAR_MIX_BIAS_SCRATCH_FLOATS)
    return fail(SPEAR_BTP_EINVAL,
                "%s: this shape needs %lld floats of partial sums, the library's static array holds %lld; use "
                "spear_phalanx_mix_backward_ex with caller-allocated sum arrays",
                who, need, (long long)SPEAR_MIX_BIAS_SCRATCH_FLOATS);
  spear_btp::MixBwdArgs a{a_logit, b_logit, c, v, dout, da_logit, db_logit, dc, dv, B, L, H, H / kv_heads, dtype,
                          nullptr, nullptr, nullptr, ld_da, ld_db, ld_dc, ld_dv, false};
  const hipError_t err =
      spear_btp::fused_mix_backward_bias(a, bias_da, bias_db, bias_dc, static_cast<hipStream_t>(stream));
  if (err != hipSuccess) return fail(SPEAR_BTP_ELAUNCH, "%s: launch failed: %s", who, hipGetErrorString(err));
  return 0;
}

int spear_phalanx_mix_step(const void* a_logit, const void* b_logit, const void* c, const void* v, void* out, float* h,
                           float* r, float* c_prev, int* pos, int boundary, int block_len, int B, int H, int kv_heads,
                           int dtype, unsigned flags, void* stream) {
  g_error[0] = '\0';
  const char* who = "spear_phalanx_mix_step";
  if (B < 0 || H < 0) return fail(SPEAR_BTP_EINVAL, "%s: negative dimension (B=%d H=%d)", who, B, H);
  if (block_len <= 0) return fail(SPEAR_BTP_EINVAL, "%s: block_len must be positive (got %d)", who, block_len);
  if (kv_heads <= 0 || H % kv_heads != 0)
    return fail(SPEAR_BTP_EINVAL, "%s: heads (%d) must be divisible by kv_heads (%d)", who, H, kv_heads);
  if (dtype != SPEAR_BTP_BF16 && dtype != SPEAR_BTP_F16)
    return fail(SPEAR_BTP_EINVAL, "%s: tensors must be float16 or bfloat16.", who);
  if (flags != 0u) return fail(SPEAR_BTP_EINVAL, "%s: unknown flag bits 0x%x", who, flags);
  if ((long long)B * H * 16ll >= (1ll << 40)) return fail(SPEAR_BTP_EINVAL, "%s: tensor too large", who);
  if ((long long)B * H == 0) return 0;
  // b_logit, c, v, out, h and c_prev move as 16-byte pieces; a_logit is read one 16-bit element and r one
  // fp32 element at a time, so a row of a [tokens, B, H] tensor (any B * H) can be passed as it lies
  const void* wide[] = {b_logit, c, v, out, h, c_prev};
  if (!a_logit || !r) return fail(SPEAR_BTP_ENULL, "%s: NULL tensor pointer", who);
  for (const void* q : wide) {
    if (!q) return fail(SPEAR_BTP_ENULL, "%s: NULL tensor pointer", who);
    if (!aligned16(q))
      return fail(SPEAR_BTP_EINVAL, "%s: b_logit, c, v, out, h and c_prev must be 16-byte aligned", who);
  }
  if (reinterpret_cast<uintptr_t>(a_logit) & 1u) return fail(SPEAR_BTP_EINVAL, "%s: a_logit must be 2-byte aligned", who);
  if (reinterpret_cast<uintptr_t>(r) & 3u) return fail(SPEAR_BTP_EINVAL, "%s: r must be 4-byte aligned", who);
  if (pos && (reinterpret_cast<uintptr_t>(pos) & 3u)) return fail(SPEAR_BTP_EINVAL, "%s: pos must be 4-byte aligned", who);
  spear_btp::MixStepArgs a{a_logit, b_logit, c, v, out, h, r, c_prev, pos, boundary ? 1 : 0, block_len, B, H, H / kv_heads, dtype};
  const hipError_t err = spear_btp::fused_mix_step(a, static_cast<hipStream_t>(stream));
  if (err != hipSuccess) return fail(SPEAR_BTP_ELAUNCH, "%s: launch failed: %s", who, hipGetErrorString(err));
  return 0;
}

int spear_jagged_prefill(const void* a, const void* x, const void* c, const void* v, const void* carry_init, void* y,
                         void* h_tail, void* r_tail, void* c_prev_tail, int B, int H, int D, int L, int block_len,
                         int a_dtype, int x_dtype, int state_dtype, int r_dtype, unsigned flags, void* stream) {
  g_error[0] = '\0';
  const char* who = "spear_jagged_prefill";
  if (B < 0 || H < 0 || L < 0) return fail(SPEAR_BTP_EINVAL, "%s: negative dimension (B=%d H=%d L=%d)", who, B, H, L);
  if (D <= 0 || block_len <= 0)
    return fail(SPEAR_BTP_EINVAL, "%s: D and block_len must be positive (D=%d block_len=%d)", who, D, block_len);
  if (!dtype_ok(a_dtype) || !dtype_ok(x_dtype) || !dtype_ok(state_dtype) || !dtype_ok(r_dtype))
    return fail(SPEAR_BTP_EINVAL, "%s: unknown dtype tag", who);
  if (a_dtype != x_dtype && a_dtype != SPEAR_BTP_F32)
    return fail(SPEAR_BTP_EINVAL, "%s: a must be float32 or match x dtype.", who);
  if (state_dtype != x_dtype && state_dtype != SPEAR_BTP_F32)
    return fail(SPEAR_BTP_EINVAL, "%s: the state must be float32 or match x dtype.", who);
  if (flags & ~SPEAR_JAGGED_LOG_A) return fail(SPEAR_BTP_EINVAL, "%s: unknown flag bits 0x%x", who, flags & ~SPEAR_JAGGED_LOG_A);
  if ((long long)B * H * (long long)D * L >= (1ll << 40)) return fail(SPEAR_BTP_EINVAL, "%s: tensor too large", who);
  if ((c == nullptr) != (v == nullptr)) return fail(SPEAR_BTP_EINVAL, "%s: c and v must be given together", who);
  const int n_state = (h_tail != nullptr) + (r_tail != nullptr) + (c_prev_tail != nullptr);
  if (n_state != 0 && n_state != 3)
    return fail(SPEAR_BTP_EINVAL, "%s: h_tail, r_tail and c_prev_tail must be given together", who);
  if ((long long)B * H == 0 || L == 0) return 0;
  if (!a || !x || !y) return fail(SPEAR_BTP_ENULL, "%s: NULL tensor pointer", who);
  const bool al = aligned16(a) && aligned16(x) && aligned16(y) && aligned16(c) && aligned16(v);
  spear_btp::JagPrefillArgs p{a, x, c, v, carry_init, y, h_tail, r_tail, c_prev_tail, B, H, D, L, block_len,
                              a_dtype, x_dtype, state_dtype, r_dtype, (flags & SPEAR_JAGGED_LOG_A) != 0, al};
  const hipError_t err = spear_btp::jagged_prefill(p, static_cast<hipStream_t>(stream));
  if (err != hipSuccess) return fail(SPEAR_BTP_ELAUNCH, "%s: launch failed: %s", who, hipGetErrorString(err));
  return 0;
}

int spear_jagged_step(const void* a_t, const void* x_t, const void* c_t, const void* v_t, void* y_t, const void* h_in,
                      const void* r_in, const void* c_prev_in, void* h_out, void* r_out, void* c_prev_out, int B, int H,
                      int D, int boundary, int a_dtype, int x_dtype, int state_dtype, int r_dtype, unsigned flags,
                      float tiny, void* stream) {
  g_error[0] = '\0';
  const char* who = "spear_jagged_step";
  if (B < 0 || H < 0) return fail(SPEAR_BTP_EINVAL, "%s: negative dimension (B=%d H=%d)", who, B, H);
  if (D <= 0) return fail(SPEAR_BTP_EINVAL, "%s: D must be positive (got %d)", who, D);
  if (!dtype_ok(a_dtype) || !dtype_ok(x_dtype) || !dtype_ok(state_dtype) || !dtype_ok(r_dtype))
    return fail(SPEAR_BTP_EINVAL, "%s: unknown dtype tag", who);
  if (state_dtype != x_dtype && state_dtype != SPEAR_BTP_F32)
    return fail(SPEAR_BTP_EINVAL, "%s: the state must be float32 or match x dtype.", who);
  const unsigned known = SPEAR_JAGGED_LOG_A | SPEAR_JAGGED_LOG_R;
  if (flags & ~known) return fail(SPEAR_BTP_EINVAL, "%s: unknown flag bits 0x%x", who, flags & ~known);
  if ((long long)B * H * (long long)D >= (1ll << 40)) return fail(SPEAR_BTP_EINVAL, "%s: tensor too large", who);
  if ((c_t == nullptr) != (v_t == nullptr)) return fail(SPEAR_BTP_EINVAL, "%s: c_t and v_t must be given together", who);
  if ((long long)B * H == 0) return 0;
  if (!a_t || !x_t || !y_t || !h_in || !r_in || !c_prev_in || !h_out || !r_out || (boundary && !c_prev_out))
    return fail(SPEAR_BTP_ENULL, "%s: NULL tensor pointer", who);
  const bool al = aligned16(x_t) && aligned16(c_t) && aligned16(v_t) && aligned16(y_t) && aligned16(h_in) &&
                  aligned16(c_prev_in) && aligned16(h_out) && aligned16(c_prev_out);
  spear_btp::JagStepArgs p{a_t, x_t, c_t, v_t, y_t, h_in, r_in, c_prev_in, h_out, r_out, c_prev_out, B, H, D,
                           boundary ? 1 : 0, a_dtype, x_dtype, state_dtype, r_dtype,
                           (flags & SPEAR_JAGGED_LOG_A) ? 1 : 0, (flags & SPEAR_JAGGED_LOG_R) ? 1 : 0, tiny, al};
  const hipError_t err = spear_btp::jagged_step(p, static_cast<hipStream_t>(stream));
  if (err != hipSuccess) return fail(SPEAR_BTP_ELAUNCH, "%s: launch failed: %s", who, hipGetErrorString(err));
  return 0;
}

}  // extern "C"
