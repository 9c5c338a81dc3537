// Compiled torch binding over the C ABI of libspear_btp.so: the module that stands where the
// reference has its extension module `spear._btp` (csrc/btp/_bindings.cu:240-243, built by
// CMakeLists.txt:86-101 there). It exports
//     forward (coeff, x, y, checkpoint, k, wpb)
//     backward(coeff, x, dy, checkpoint, dx, dA, k, wpb)
// with the reference's positional arguments, in-place semantics (the caller allocates every output)
// and argument checks and messages (csrc/btp/_bindings.cu:19-60, raised as RuntimeError by
// TORCH_CHECK), plus the shape / stride / device checks the reference leaves out, and the bindings
// of the entry points the reference has no counterpart for (log-space gates, fused layer layout).
// No kernel code lives here: every function unpacks tensors into raw pointers and sizes and calls
// the C ABI on torch's current stream of the tensors' device, without synchronising.
#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>
#include <torch/extension.h>

#include <string>
#include <vector>

#include "../../include/spear_btp.h"

namespace {

int tag_of(at::ScalarType t) {
  switch (t) {
    case at::kBFloat16: return SPEAR_BTP_BF16;
    case at::kHalf: return SPEAR_BTP_F16;
    case at::kFloat: return SPEAR_BTP_F32;
    default: return -1;
  }
}

bool is_16bit(const at::Tensor& t) { return t.scalar_type() == at::kHalf || t.scalar_type() == at::kBFloat16; }

void check_layout(const char* name, const at::Tensor& t, at::IntArrayRef shape) {
  // The reference reads B*H*L (resp. B*H*16*L) elements without looking at shapes or strides
  // (csrc/btp/_bindings.cu:80-87); a wrong shape there is an out-of-bounds read. Here it raises.
  TORCH_CHECK(t.sizes() == shape, name, " must have shape ", shape, ", got ", t.sizes(), ".");
  TORCH_CHECK(t.is_contiguous(), name, " must be contiguous.");
}

void check_same_device(std::initializer_list<const at::Tensor*> ts) {
  const at::Tensor* first = nullptr;
  for (const at::Tensor* t : ts) {
    if (t == nullptr || !t->defined()) continue;
    if (first == nullptr) first = t;
    TORCH_CHECK(t->device() == first->device(), "All tensors must be on the same device.");
  }
}

void* stream_of(const at::Tensor& t) { return c10::hip::getCurrentHIPStream(t.device().index()).stream(); }

void raise_native(int rc) {
  const char* msg = spear_btp_last_error();
  TORCH_CHECK(false, (msg && msg[0]) ? std::string(msg) : "spear_btp call failed with code " + std::to_string(rc));
}

void check_common(const at::Tensor& x, const at::Tensor& coeff, int64_t k, int64_t wpb, const char* wpb_msg) {
  TORCH_CHECK(x.dim() == 4, "x must be [B, H, 16, L].");
  TORCH_CHECK(x.size(2) == 16, "Channel dim (DH) must be 16.");
  TORCH_CHECK(k == 1 || k == 2, "k must be 1 or 2.");
  TORCH_CHECK(wpb == 4 || wpb == 8 || wpb == 16 || wpb == 32, wpb_msg, wpb);
  TORCH_CHECK(is_16bit(coeff), "coeff must be float16 or bfloat16.");
  TORCH_CHECK(x.scalar_type() == coeff.scalar_type(), "x dtype must match coeff.");
}

// csrc/btp/_bindings.cu:76-150. `flags` is an extension (default: store the carry checkpoint, as the
// reference does); without SPEAR_BTP_WRITE_CHECKPOINT the checkpoint may be a zero-element placeholder.
void forward(const at::Tensor& coeff, const at::Tensor& x, at::Tensor y, at::Tensor checkpoint, int64_t k,
             int64_t wpb, int64_t flags) {
  TORCH_CHECK(coeff.is_cuda() && x.is_cuda() && y.is_cuda() && checkpoint.is_cuda(), "All tensors must be CUDA.");
  check_common(x, coeff, k, wpb, "Unsupported WPB value: ");
  TORCH_CHECK(y.scalar_type() == at::kFloat || y.scalar_type() == x.scalar_type(), "y must be float32 or match x dtype.");
  TORCH_CHECK(checkpoint.scalar_type() == at::kFloat, "checkpoint must be float32.");
  const int64_t B = x.size(0), H = x.size(1), L = x.size(3);
  TORCH_CHECK(L % 16 == 0, "Length L must be multiple of 16");
  check_layout("coeff", coeff, {B, H, L});
  check_layout("x", x, {B, H, 16, L});
  check_layout("y", y, {B, H, 16, L});
  if ((flags & SPEAR_BTP_WRITE_CHECKPOINT) || checkpoint.numel() != 0) check_layout("checkpoint", checkpoint, {B, H, L / 16, 16});
  check_same_device({&coeff, &x, &y, &checkpoint});
  const c10::DeviceGuard guard(x.device());
  const int rc = spear_btp_forward(coeff.data_ptr(), x.data_ptr(), y.data_ptr(), static_cast<float*>(checkpoint.data_ptr()),
                                   (int)B, (int)H, (int)L, (int)k, tag_of(x.scalar_type()), tag_of(y.scalar_type()),
                                   (unsigned)flags, stream_of(x));
  if (rc != 0) raise_native(rc);
}

// csrc/btp/_bindings.cu:152-229. Every element of dA is written (it need not arrive zero-filled); the
// checkpoint is accepted for signature compatibility and not read. With SPEAR_BTP_DX_F32 in `flags`
// (an extension) dx is float32 and receives the kernel's fp32 values unrounded.
void backward(const at::Tensor& coeff, const at::Tensor& x, const at::Tensor& dy, const at::Tensor& checkpoint,
              at::Tensor dx, at::Tensor dA, int64_t k, int64_t wpb, int64_t flags) {
  TORCH_CHECK(coeff.is_cuda() && x.is_cuda() && dy.is_cuda() && checkpoint.is_cuda(), "coeff, x, dy, checkpoint must be CUDA.");
  TORCH_CHECK(dx.is_cuda() && dA.is_cuda(), "dx and dA must be CUDA.");
  check_common(x, coeff, k, wpb, "Unsupported WPB value for backward: ");
  if (flags & SPEAR_BTP_DX_F32) {
    TORCH_CHECK(dx.scalar_type() == at::kFloat, "dx must be float32 in the fp32 check mode.");
  } else {
    TORCH_CHECK(dx.scalar_type() == x.scalar_type(), "dx dtype must match x.");
  }
  TORCH_CHECK(dA.scalar_type() == at::kFloat, "dA must be float32.");
  TORCH_CHECK(dy.scalar_type() == at::kFloat || dy.scalar_type() == x.scalar_type(), "dy must be float32 or match x dtype.");
  const int64_t B = x.size(0), H = x.size(1), L = x.size(3);
  TORCH_CHECK(L % 16 == 0, "Length L must be multiple of 16");
  check_layout("coeff", coeff, {B, H, L});
  check_layout("x", x, {B, H, 16, L});
  check_layout("dy", dy, {B, H, 16, L});
  check_layout("dx", dx, {B, H, 16, L});
  check_layout("dA", dA, {B, H, L});
  check_same_device({&coeff, &x, &dy, &dx, &dA});
  const c10::DeviceGuard guard(x.device());
  const int rc = spear_btp_backward(coeff.data_ptr(), x.data_ptr(), dy.data_ptr(),
                                    checkpoint.numel() ? static_cast<const float*>(checkpoint.data_ptr()) : nullptr,
                                    dx.data_ptr(), static_cast<float*>(dA.data_ptr()), (int)B, (int)H, (int)L, (int)k,
                                    tag_of(x.scalar_type()), tag_of(dy.scalar_type()), (unsigned)flags, stream_of(x));
  if (rc != 0) raise_native(rc);
}

void check_log_common(const at::Tensor& gate, const at::Tensor& x, int64_t k) {
  TORCH_CHECK(gate.is_cuda() && x.is_cuda(), "All tensors must be CUDA.");
  TORCH_CHECK(x.dim() == 4, "x must be [B, H, 16, L].");
  TORCH_CHECK(x.size(2) == 16, "Channel dim (DH) must be 16.");
  TORCH_CHECK(k == 1 || k == 2, "k must be 1 or 2.");
  TORCH_CHECK(gate.scalar_type() == at::kFloat, "gate must be float32.");
  TORCH_CHECK(is_16bit(x), "x must be float16 or bfloat16.");
  const int64_t B = x.size(0), H = x.size(1), L = x.size(3);
  TORCH_CHECK(L % 16 == 0, "Length L must be multiple of 16");
  check_layout("gate", gate, {B, H, L});
  check_layout("x", x, {B, H, 16, L});
}

// y <- btp(exp(gate), x), the exponential taken in fp32 inside the kernel (no reference counterpart).
void forward_log(const at::Tensor& gate, const at::Tensor& x, at::Tensor y, int64_t k) {
  check_log_common(gate, x, k);
  const int64_t B = x.size(0), H = x.size(1), L = x.size(3);
  TORCH_CHECK(y.is_cuda(), "All tensors must be CUDA.");
  TORCH_CHECK(y.scalar_type() == at::kFloat || y.scalar_type() == x.scalar_type(), "y must be float32 or match x dtype.");
  check_layout("y", y, {B, H, 16, L});
  check_same_device({&gate, &x, &y});
  const c10::DeviceGuard guard(x.device());
  const int rc = spear_btp_forward_loggate(static_cast<const float*>(gate.data_ptr()), x.data_ptr(), y.data_ptr(), nullptr,
                                           (int)B, (int)H, (int)L, (int)k, tag_of(x.scalar_type()),
                                           tag_of(y.scalar_type()), 0u, stream_of(x));
  if (rc != 0) raise_native(rc);
}

// dx, dgate <- vjp of btp(exp(gate), x); a float32 dx selects the fp32 check mode.
void backward_log(const at::Tensor& gate, const at::Tensor& x, const at::Tensor& dy, at::Tensor dx, at::Tensor dgate,
                  int64_t k) {
  check_log_common(gate, x, k);
  const int64_t B = x.size(0), H = x.size(1), L = x.size(3);
  TORCH_CHECK(dy.is_cuda() && dx.is_cuda() && dgate.is_cuda(), "All tensors must be CUDA.");
  TORCH_CHECK(dx.scalar_type() == x.scalar_type() || dx.scalar_type() == at::kFloat, "dx must be float32 or match x dtype.");
  TORCH_CHECK(dgate.scalar_type() == at::kFloat, "dgate must be float32.");
  TORCH_CHECK(dy.scalar_type() == at::kFloat || dy.scalar_type() == x.scalar_type(), "dy must be float32 or match x dtype.");
  check_layout("dy", dy, {B, H, 16, L});
  check_layout("dx", dx, {B, H, 16, L});
  check_layout("dgate", dgate, {B, H, L});
  check_same_device({&gate, &x, &dy, &dx, &dgate});
  const c10::DeviceGuard guard(x.device());
  const unsigned flags = dx.scalar_type() == at::kFloat ? SPEAR_BTP_DX_F32 : 0u;
  const int rc = spear_btp_backward_loggate(static_cast<const float*>(gate.data_ptr()), x.data_ptr(), dy.data_ptr(),
                                            dx.data_ptr(), static_cast<float*>(dgate.data_ptr()), (int)B, (int)H, (int)L,
                                            (int)k, tag_of(x.scalar_type()), tag_of(dy.scalar_type()), flags, stream_of(x));
  if (rc != 0) raise_native(rc);
}

// The autograd node of btp(), compiled: forward allocates y (and the checkpoint, a zero-element placeholder
// unless the store is on), backward allocates dx and dA, both call the functions above. It does what
// _BTPFunction of the reference does (spear/ops/btp/interface.py:126-161) without the Python frames of
// torch.autograd.Function and of the custom-op dispatch, which at small batches cost several times the
// kernels' time. The Python side uses it for plain eager tensors only; under torch.compile and dispatch modes
// the Python node over the traceable custom ops runs instead.
struct BtpNode : public torch::autograd::Function<BtpNode> {
  static at::Tensor forward(torch::autograd::AutogradContext* ctx, const at::Tensor& coeff, const at::Tensor& x, int64_t k,
                            int64_t wpb, bool y_f32, int64_t forward_flags, int64_t backward_flags) {
    TORCH_CHECK(x.dim() == 4, "x must be [B, H, 16, L].");
    at::Tensor y = at::empty(x.sizes(), x.options().dtype(y_f32 ? at::kFloat : x.scalar_type()));
    at::Tensor checkpoint =
        (forward_flags & SPEAR_BTP_WRITE_CHECKPOINT)
            ? at::empty({x.size(0), x.size(1), x.size(3) / 16, 16}, x.options().dtype(at::kFloat))
            : at::empty({0}, x.options().dtype(at::kFloat));
    ::forward(coeff, x, y, checkpoint, k, wpb, forward_flags);
    ctx->save_for_backward({coeff, x, checkpoint});
    ctx->saved_data["k"] = k;
    ctx->saved_data["wpb"] = wpb;
    ctx->saved_data["flags"] = backward_flags;
    return y;
  }

  static torch::autograd::variable_list backward(torch::autograd::AutogradContext* ctx,
                                                 torch::autograd::variable_list grad_outputs) {
    const auto saved = ctx->get_saved_variables();
    const at::Tensor &coeff = saved[0], &x = saved[1], &checkpoint = saved[2];
    const at::Tensor dy = grad_outputs[0].contiguous();
    at::Tensor dx = at::empty(x.sizes(), x.options());
    at::Tensor dA = at::empty(coeff.sizes(), coeff.options().dtype(at::kFloat));
    ::backward(coeff, x, dy, checkpoint, dx, dA, ctx->saved_data["k"].toInt(), ctx->saved_data["wpb"].toInt(),
               ctx->saved_data["flags"].toInt());
    return {dA, dx, at::Tensor(), at::Tensor(), at::Tensor(), at::Tensor(), at::Tensor()};
  }
};

at::Tensor btp_autograd(const at::Tensor& coeff, const at::Tensor& x, int64_t k, int64_t wpb, bool y_f32,
                        int64_t forward_flags, int64_t backward_flags) {
  return BtpNode::apply(coeff, x, k, wpb, y_f32, forward_flags, backward_flags);
}

struct MixShape {
  int64_t B, L, F, Fkv;
};

MixShape check_mix_inputs(const at::Tensor& a_logit, const at::Tensor& b_logit, const at::Tensor& c, const at::Tensor& v,
                          int64_t heads, int64_t kv_heads, bool qkv_gate) {
  TORCH_CHECK(a_logit.is_cuda() && b_logit.is_cuda() && c.is_cuda() && v.is_cuda(), "All tensors must be CUDA.");
  TORCH_CHECK(v.dim() == 3 && v.size(2) == heads * 16, "v must be [B, L, heads * 16].");
  TORCH_CHECK(heads > 0 && kv_heads > 0 && heads % kv_heads == 0, "heads must be divisible by kv_heads.");
  TORCH_CHECK(is_16bit(v), "tensors must be float16 or bfloat16.");
  TORCH_CHECK(b_logit.scalar_type() == v.scalar_type() && c.scalar_type() == v.scalar_type(), "all tensors must share one dtype.");
  if (qkv_gate) {
    TORCH_CHECK(a_logit.scalar_type() == at::kFloat, "the log-decay gate must be float32.");
  } else {
    TORCH_CHECK(a_logit.scalar_type() == v.scalar_type(), "all tensors must share one dtype.");
  }
  const MixShape s{v.size(0), v.size(1), v.size(2), kv_heads * 16};
  TORCH_CHECK(s.L % 16 == 0, "Length L must be multiple of 16");
  check_layout("a_logit", a_logit, {s.B, s.L, heads});
  check_layout("b_logit", b_logit, {s.B, s.L, s.Fkv});
  check_layout("c", c, {s.B, s.L, s.Fkv});
  check_layout("v", v, {s.B, s.L, s.F});
  return s;
}

// out <- btp(sigmoid(a_logit), sigmoid(b_logit) * v) * c + v on [B, L, features] tensors, or with
// qkv_gate out <- c * btp(exp(a_logit), b_logit * v) + v. A float32 `out` selects the fp32 check mode.
void mix_forward(const at::Tensor& a_logit, const at::Tensor& b_logit, const at::Tensor& c, const at::Tensor& v,
                 at::Tensor out, int64_t heads, int64_t kv_heads, bool qkv_gate) {
  const MixShape s = check_mix_inputs(a_logit, b_logit, c, v, heads, kv_heads, qkv_gate);
  TORCH_CHECK(out.is_cuda(), "All tensors must be CUDA.");
  TORCH_CHECK(out.scalar_type() == v.scalar_type() || out.scalar_type() == at::kFloat,
              "out must be float32 (fp32 check mode) or match v dtype.");
  check_layout("out", out, {s.B, s.L, s.F});
  check_same_device({&a_logit, &b_logit, &c, &v, &out});
  const c10::DeviceGuard guard(v.device());
  const unsigned flags = (qkv_gate ? SPEAR_MIX_QKV_GATE : 0u) | (out.scalar_type() == at::kFloat ? SPEAR_MIX_F32_RESULTS : 0u);
  const int rc = spear_phalanx_mix_forward(a_logit.data_ptr(), b_logit.data_ptr(), c.data_ptr(), v.data_ptr(), out.data_ptr(),
                                           (int)s.B, (int)s.L, (int)heads, (int)kv_heads, tag_of(v.scalar_type()), flags,
                                           stream_of(v));
  if (rc != 0) raise_native(rc);
}

// Elements per time step of a [B, L, width] tensor that is dense or a column block of a wider buffer.
int64_t row_stride(const char* name, const at::Tensor& t, int64_t B, int64_t L, int64_t width) {
  TORCH_CHECK(t.dim() == 3 && t.size(0) == B && t.size(1) == L && t.size(2) == width, name, " must have shape [", B, ", ",
              L, ", ", width, "], got ", t.sizes(), ".");
  const int64_t ld = L > 1 ? t.stride(1) : (B > 1 ? t.stride(0) : width);
  TORCH_CHECK(t.stride(2) == 1 && (L <= 1 || t.stride(1) == ld) && (B <= 1 || t.stride(0) == L * ld), name,
              " must be dense or a column block of a dense [B, L, ld] buffer.");
  return ld;
}

// Gradients of mix_forward, written in place. Float32 db_logit / dc / dv (and da_logit) select the fp32
// check mode. `sums`: none, or three fp32 [rows, width] tensors receiving the column sums of every (batch row,
// tile of 64 time steps).
void mix_backward(const at::Tensor& a_logit, const at::Tensor& b_logit, const at::Tensor& c, const at::Tensor& v,
                  const at::Tensor& dout, at::Tensor da_logit, at::Tensor db_logit, at::Tensor dc, at::Tensor dv,
                  int64_t heads, int64_t kv_heads, const std::vector<at::Tensor>& sums, bool qkv_gate) {
  const MixShape s = check_mix_inputs(a_logit, b_logit, c, v, heads, kv_heads, qkv_gate);
  TORCH_CHECK(dout.is_cuda() && da_logit.is_cuda() && db_logit.is_cuda() && dc.is_cuda() && dv.is_cuda(), "All tensors must be CUDA.");
  TORCH_CHECK(dout.scalar_type() == v.scalar_type(), "all tensors must share one dtype.");
  check_layout("dout", dout, {s.B, s.L, s.F});
  const bool f32 = dv.scalar_type() == at::kFloat;
  TORCH_CHECK(db_logit.scalar_type() == dv.scalar_type() && dc.scalar_type() == dv.scalar_type() &&
                  (f32 || dv.scalar_type() == v.scalar_type()),
              "db_logit, dc and dv must all be float32 (fp32 check mode) or all match v dtype.");
  if (qkv_gate || f32) {
    TORCH_CHECK(da_logit.scalar_type() == at::kFloat, "the gradient of the gate must be float32.");
  } else {
    TORCH_CHECK(da_logit.scalar_type() == v.scalar_type(), "all tensors must share one dtype.");
  }
  TORCH_CHECK(sums.empty() || sums.size() == 3, "sums must be three tensors or none.");
  TORCH_CHECK(sums.empty() || !qkv_gate, "column sums belong to the layer form, not to qkv_gate.");
  TORCH_CHECK(sums.empty() || !f32, "column sums are not available in the fp32 check mode.");
  const int64_t ld_da = row_stride("da_logit", da_logit, s.B, s.L, heads), ld_db = row_stride("db_logit", db_logit, s.B, s.L, s.Fkv),
                ld_dc = row_stride("dc", dc, s.B, s.L, s.Fkv), ld_dv = row_stride("dv", dv, s.B, s.L, s.F);
  check_same_device({&a_logit, &b_logit, &c, &v, &dout, &da_logit, &db_logit, &dc, &dv});
  int64_t rows = 0;
  float* sp[3] = {nullptr, nullptr, nullptr};
  if (!sums.empty()) {
    rows = spear_phalanx_mix_backward_sum_rows((int)s.B, (int)s.L, (int)heads);
    const int64_t widths[3] = {heads, s.Fkv, s.Fkv};
    const char* names[3] = {"sum_da", "sum_db", "sum_dc"};
    for (int i = 0; i < 3; ++i) {
      TORCH_CHECK(sums[i].is_cuda() && sums[i].device() == v.device() && sums[i].scalar_type() == at::kFloat, names[i],
                  " must be float32 on v's device.");
      check_layout(names[i], sums[i], {rows, widths[i]});
      sp[i] = rows > 0 ? static_cast<float*>(sums[i].data_ptr()) : nullptr;
    }
  }
  const c10::DeviceGuard guard(v.device());
  const unsigned flags = (qkv_gate ? SPEAR_MIX_QKV_GATE : 0u) | (f32 ? SPEAR_MIX_F32_RESULTS : 0u);
  const int rc = spear_phalanx_mix_backward_ex(
      a_logit.data_ptr(), b_logit.data_ptr(), c.data_ptr(), v.data_ptr(), dout.data_ptr(), da_logit.data_ptr(),
      db_logit.data_ptr(), dc.data_ptr(), dv.data_ptr(), (int)ld_da, (int)ld_db, (int)ld_dc, (int)ld_dv, sp[0], sp[1], sp[2],
      rows, (int)s.B, (int)s.L, (int)heads, (int)kv_heads, tag_of(v.scalar_type()), flags, stream_of(v));
  if (rc != 0) raise_native(rc);
}

// The autograd node of btp_log(), compiled like BtpNode: forward allocates y, backward dx and dgate.
struct BtpLogNode : public torch::autograd::Function<BtpLogNode> {
  static at::Tensor forward(torch::autograd::AutogradContext* ctx, const at::Tensor& gate, const at::Tensor& x, int64_t k,
                            bool y_f32) {
    TORCH_CHECK(x.dim() == 4, "x must be [B, H, 16, L].");
    at::Tensor y = at::empty(x.sizes(), x.options().dtype(y_f32 ? at::kFloat : x.scalar_type()));
    forward_log(gate, x, y, k);
    ctx->save_for_backward({gate, x});
    ctx->saved_data["k"] = k;
    return y;
  }

  static torch::autograd::variable_list backward(torch::autograd::AutogradContext* ctx,
                                                 torch::autograd::variable_list grad_outputs) {
    const auto saved = ctx->get_saved_variables();
    const at::Tensor &gate = saved[0], &x = saved[1];
    at::Tensor dx = at::empty(x.sizes(), x.options());
    at::Tensor dgate = at::empty(gate.sizes(), gate.options());
    backward_log(gate, x, grad_outputs[0].contiguous(), dx, dgate, ctx->saved_data["k"].toInt());
    return {dgate, dx, at::Tensor(), at::Tensor()};
  }
};

at::Tensor btp_log_autograd(const at::Tensor& gate, const at::Tensor& x, int64_t k, bool y_f32) {
  return BtpLogNode::apply(gate, x, k, y_f32);
}

// The autograd node of phalanx_mix() and, with qkv_gate, of btp_qkv() (operands then in the kernel's order: gate,
// k, q, v), compiled: forward allocates out, backward the four gradients (the first one in a_logit's dtype, which
// for the q/k/v/gate form is the fp32 of the gate). What spear_amd/ops/btp/fused.py does in torch.autograd.Function
// classes over the traceable custom ops, without their Python frames; used for plain eager tensors only.
struct MixNode : public torch::autograd::Function<MixNode> {
  static at::Tensor forward(torch::autograd::AutogradContext* ctx, const at::Tensor& a_logit, const at::Tensor& b_logit,
                            const at::Tensor& c, const at::Tensor& v, int64_t heads, int64_t kv_heads, bool qkv_gate) {
    at::Tensor out = at::empty(v.sizes(), v.options());
    mix_forward(a_logit, b_logit, c, v, out, heads, kv_heads, qkv_gate);
    ctx->save_for_backward({a_logit, b_logit, c, v});
    ctx->saved_data["heads"] = heads;
    ctx->saved_data["kv_heads"] = kv_heads;
    ctx->saved_data["qkv_gate"] = qkv_gate;
    return out;
  }

  static torch::autograd::variable_list backward(torch::autograd::AutogradContext* ctx,
                                                 torch::autograd::variable_list grad_outputs) {
    const auto saved = ctx->get_saved_variables();
    const at::Tensor &a_logit = saved[0], &b_logit = saved[1], &c = saved[2], &v = saved[3];
    at::Tensor da = at::empty(a_logit.sizes(), a_logit.options()), db = at::empty(b_logit.sizes(), b_logit.options()),
               dc = at::empty(c.sizes(), c.options()), dv = at::empty(v.sizes(), v.options());
    mix_backward(a_logit, b_logit, c, v, grad_outputs[0].contiguous(), da, db, dc, dv, ctx->saved_data["heads"].toInt(),
                 ctx->saved_data["kv_heads"].toInt(), {}, ctx->saved_data["qkv_gate"].toBool());
    return {da, db, dc, dv, at::Tensor(), at::Tensor(), at::Tensor()};
  }
};

at::Tensor mix_autograd(const at::Tensor& a_logit, const at::Tensor& b_logit, const at::Tensor& c, const at::Tensor& v,
                        int64_t heads, int64_t kv_heads, bool qkv_gate) {
  return MixNode::apply(a_logit, b_logit, c, v, heads, kv_heads, qkv_gate);
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  namespace py = pybind11;
  m.doc() = "Compiled binding of the MI355X Block Two-Pass library (C ABI of libspear_btp.so)";
  m.def("forward", &forward, py::arg("coeff"), py::arg("x"), py::arg("y"), py::arg("checkpoint"), py::arg("k"), py::arg("wpb"),
        py::arg("flags") = (int64_t)SPEAR_BTP_WRITE_CHECKPOINT, "BTP Forward (HIP, gfx950)");
  m.def("backward", &backward, py::arg("coeff"), py::arg("x"), py::arg("dy"), py::arg("checkpoint"), py::arg("dx"),
        py::arg("dA"), py::arg("k"), py::arg("wpb"), py::arg("flags") = (int64_t)0, "BTP Backward (HIP, gfx950)");
  m.def("btp_autograd", &btp_autograd, py::arg("coeff"), py::arg("x"), py::arg("k"), py::arg("wpb"), py::arg("y_f32"),
        py::arg("forward_flags"), py::arg("backward_flags"),
        "y = btp(coeff, x) with its autograd node (contiguous plain tensors; gradients: dA float32, dx in x's dtype)");
  m.def("forward_log", &forward_log, py::arg("gate"), py::arg("x"), py::arg("y"), py::arg("k"));
  m.def("backward_log", &backward_log, py::arg("gate"), py::arg("x"), py::arg("dy"), py::arg("dx"), py::arg("dgate"), py::arg("k"));
  m.def("mix_forward", &mix_forward, py::arg("a_logit"), py::arg("b_logit"), py::arg("c"), py::arg("v"), py::arg("out"),
        py::arg("heads"), py::arg("kv_heads"), py::arg("qkv_gate") = false);
  m.def("mix_backward", &mix_backward, py::arg("a_logit"), py::arg("b_logit"), py::arg("c"), py::arg("v"), py::arg("dout"),
        py::arg("da_logit"), py::arg("db_logit"), py::arg("dc"), py::arg("dv"), py::arg("heads"), py::arg("kv_heads"),
        py::arg("sums") = std::vector<at::Tensor>(), py::arg("qkv_gate") = false);
  m.def("btp_log_autograd", &btp_log_autograd, py::arg("gate"), py::arg("x"), py::arg("k"), py::arg("y_f32"),
        "y = btp(exp(gate), x) with its autograd node (contiguous plain tensors; gradients: dgate float32, dx in x's dtype)");
  m.def("mix_autograd", &mix_autograd, py::arg("a_logit"), py::arg("b_logit"), py::arg("c"), py::arg("v"), py::arg("heads"),
        py::arg("kv_heads"), py::arg("qkv_gate") = false,
        "out = phalanx_mix(...) (or the q/k/v/gate form) with its autograd node (contiguous plain tensors)");
  m.def("abi_version", []() { return spear_btp_abi_version(); });
  m.def("mix_backward_sum_rows", [](int64_t B, int64_t L, int64_t heads) {
    return (int64_t)spear_phalanx_mix_backward_sum_rows((int)B, (int)L, (int)heads);
  }, py::arg("B"), py::arg("L"), py::arg("heads"));
}
