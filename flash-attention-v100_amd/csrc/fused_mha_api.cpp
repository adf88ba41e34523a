// PyTorch-ROCm extension `flash_attn_v100_cuda`: validation, allocation, device
// guard and stream lookup around the C launchers declared in fused_mha.h.
//
// Mirrors the reference extension kernel/fused_mha_api.cpp (mha_fwd :13-72,
// mha_bwd :74-162, pybind :164-168): same module name, same function names
// (`fwd`, `bwd`), same argument meaning and the same error convention
// (TORCH_CHECK -> RuntimeError).  Differences:
//   * fwd returns [out, lse] (one logsumexp) instead of [out, max, sum];
//   * bwd takes lse instead of (D, sum, max); delta is computed on the device
//     in fp32 inside the launcher;
//   * head size 64 is accepted as well as 128; any seqlen > 0 is accepted (the
//     reference assumes a multiple of 32, README.md:3, without checking);
//   * inputs that are not dense (B, N, H, D) are read through their strides
//     (or copied dense when the strides do not qualify) instead of being read
//     with wrong strides;
//   * the arch gate asks for gfx950 instead of sm_70 (:21-23).
#include <torch/extension.h>
#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime_api.h>

#include <cstring>
#include <vector>

#include "fused_mha.h"

#define CHECK_DEVICE(x) TORCH_CHECK(x.is_cuda(), #x " must be on the GPU")
#define CHECK_SHAPE(x, ...) \
  TORCH_CHECK(x.sizes() == torch::IntArrayRef({__VA_ARGS__}), #x " must have shape (" #__VA_ARGS__ ")")

namespace {

void check_arch(int device) {
  hipDeviceProp_t prop;
  TORCH_CHECK(hipGetDeviceProperties(&prop, device) == hipSuccess, "hipGetDeviceProperties failed");
  TORCH_CHECK(std::strncmp(prop.gcnArchName, "gfx950", 6) == 0, "This repo only supports gfx950 (MI355X) GPUs, got ",
              prop.gcnArchName);
}

void check_rc(int rc, const char* what) {
  TORCH_CHECK(rc == FUSED_MHA_OK, what, " failed: ", fused_mha_error_string(rc));
}

at::Tensor dense(const at::Tensor& x) { return x.is_contiguous() ? x : x.contiguous(); }

// A (batch, seqlen, heads, head_size) input as the kernels take it: the tensor
// itself with its strides when they qualify (last dimension contiguous, rows on
// 16-byte boundaries; e.g. a slice of a packed QKV projection or a
// (batch, heads, seqlen, head_size)-backed view), otherwise a dense copy.  The
// reference copies (flash_attn_interface.py:14-15) or mis-reads such inputs.
struct Operand {
  at::Tensor t;
  fused_mha_strides st;
};
Operand operand(const at::Tensor& x) {
  const int64_t sb = x.stride(0), sn = x.stride(1), sh = x.stride(2);
  const bool ok = x.stride(3) == 1 && sb >= 0 && sn >= 0 && sh >= 0 && ((sb | sn | sh) & 7) == 0 &&
                  sn < (int64_t(1) << 24) && sh < (int64_t(1) << 31) &&
                  (reinterpret_cast<uintptr_t>(x.data_ptr()) & 15u) == 0;
  if (ok) return {x, {sb, sn, sh}};
  at::Tensor c = x.contiguous();
  return {c, {c.stride(0), c.stride(1), c.stride(2)}};
}

}  // namespace

std::vector<at::Tensor> mha_fwd(at::Tensor& q,        // batch x seqlen x heads x head_size
                                const at::Tensor& k,  // batch x seqlen x heads x head_size
                                const at::Tensor& v,  // batch x seqlen x heads x head_size
                                c10::optional<at::Tensor>& out_, const float softmax_scale, bool is_causal) {
  auto q_dtype = q.dtype();
  TORCH_CHECK(q_dtype == torch::kFloat16, "This repo only supports fp16 data type");
  TORCH_CHECK(k.dtype() == q_dtype, "query and key must have the same dtype");
  TORCH_CHECK(v.dtype() == q_dtype, "query and value must have the same dtype");

  TORCH_CHECK(q.dim() == 4, "query must have 4 dimensions (batch, seqlen, heads, head_size)");
  TORCH_CHECK(k.dim() == 4 && v.dim() == 4, "key and value must have 4 dimensions");
  TORCH_CHECK(q.stride(-1) == 1, "Input tensor must have contiguous last dimension");
  TORCH_CHECK(k.stride(-1) == 1, "Input tensor must have contiguous last dimension");
  TORCH_CHECK(v.stride(-1) == 1, "Input tensor must have contiguous last dimension");

  const auto sizes = q.sizes();
  const int batch_size = sizes[0];
  const int seqlen_q = sizes[1];
  const int num_heads = sizes[2];
  const int head_size = sizes[3];
  TORCH_CHECK(batch_size > 0, "batch size must be postive");
  TORCH_CHECK(head_size == 64 || head_size == 128, "current repo only supports head dimension 64 or 128");
  TORCH_CHECK(seqlen_q > 0, "seqlen must be positive");
  CHECK_SHAPE(q, batch_size, seqlen_q, num_heads, head_size);
  CHECK_SHAPE(k, batch_size, seqlen_q, num_heads, head_size);
  CHECK_SHAPE(v, batch_size, seqlen_q, num_heads, head_size);

  CHECK_DEVICE(q); CHECK_DEVICE(k); CHECK_DEVICE(v);
  check_arch(q.get_device());

  at::Tensor out;
  if (out_.has_value()) {
    out = out_.value();
    TORCH_CHECK(out.dtype() == q_dtype, "Output must have the same dtype as inputs");
    CHECK_DEVICE(out);
    TORCH_CHECK(out.is_contiguous(), "Output tensor must be contiguous");
    CHECK_SHAPE(out, batch_size, seqlen_q, num_heads, head_size);
  } else {
    out = torch::empty({batch_size, seqlen_q, num_heads, head_size}, q.options());
  }

  c10::DeviceGuard device_guard(q.device());
  const Operand qo = operand(q), ko = operand(k), vo = operand(v);
  auto lse = torch::empty({batch_size, num_heads, seqlen_q}, q.options().dtype(at::kFloat));
  hipStream_t stream = c10::hip::getCurrentHIPStream().stream();
  check_rc(fused_mha_forward_strided(qo.t.data_ptr(), &qo.st, ko.t.data_ptr(), &ko.st, vo.t.data_ptr(), &vo.st,
                                     out.data_ptr(), lse.data_ptr(), batch_size, num_heads, seqlen_q, head_size,
                                     softmax_scale, is_causal ? 1 : 0, stream),
           "fused_mha_forward");
  return {out, lse};
}

std::vector<at::Tensor> mha_bwd(const at::Tensor& dout,  // batch x seqlen x heads x head_size
                                const at::Tensor& q, const at::Tensor& k, const at::Tensor& v,
                                const at::Tensor& out,   // batch x seqlen x heads x head_size
                                const at::Tensor& lse,   // batch x heads x seqlen, fp32
                                c10::optional<at::Tensor>& dq_, c10::optional<at::Tensor>& dk_,
                                c10::optional<at::Tensor>& dv_, const float softmax_scale, const bool is_causal) {
  auto q_dtype = q.dtype();
  TORCH_CHECK(q_dtype == torch::kFloat16, "This repo only supports fp16 data type");
  TORCH_CHECK(k.dtype() == q_dtype, "query and key must have the same dtype");
  TORCH_CHECK(v.dtype() == q_dtype, "query and value must have the same dtype");
  TORCH_CHECK(out.dtype() == q_dtype, "query and out must have the same dtype");
  TORCH_CHECK(dout.dtype() == q_dtype, "query and dout must have the same dtype");
  TORCH_CHECK(lse.dtype() == torch::kFloat32, "lse must be fp32");

  TORCH_CHECK(q.dim() == 4, "query must have 4 dimensions (batch, seqlen, heads, head_size)");
  TORCH_CHECK(k.dim() == 4 && v.dim() == 4, "key and value must have 4 dimensions");
  TORCH_CHECK(out.dim() == 4 && dout.dim() == 4, "out and dout must have 4 dimensions");
  TORCH_CHECK(q.stride(-1) == 1, "Input tensor must have contiguous last dimension");
  TORCH_CHECK(k.stride(-1) == 1, "Input tensor must have contiguous last dimension");
  TORCH_CHECK(v.stride(-1) == 1, "Input tensor must have contiguous last dimension");
  TORCH_CHECK(dout.stride(-1) == 1, "Input tensor must have contiguous last dimension");

  const auto sizes = q.sizes();
  const int batch_size = sizes[0];
  const int seqlen_q = sizes[1];
  const int num_heads = sizes[2];
  const int head_size = sizes[3];
  TORCH_CHECK(batch_size > 0, "batch size must be postive");
  TORCH_CHECK(head_size == 64 || head_size == 128, "current repo only supports head dimension 64 or 128");
  TORCH_CHECK(seqlen_q > 0, "seqlen must be positive");
  CHECK_SHAPE(q, batch_size, seqlen_q, num_heads, head_size);
  CHECK_SHAPE(k, batch_size, seqlen_q, num_heads, head_size);
  CHECK_SHAPE(v, batch_size, seqlen_q, num_heads, head_size);
  CHECK_SHAPE(out, batch_size, seqlen_q, num_heads, head_size);
  CHECK_SHAPE(dout, batch_size, seqlen_q, num_heads, head_size);
  CHECK_SHAPE(lse, batch_size, num_heads, seqlen_q);

  CHECK_DEVICE(q); CHECK_DEVICE(k); CHECK_DEVICE(v);
  CHECK_DEVICE(out); CHECK_DEVICE(dout); CHECK_DEVICE(lse);
  check_arch(q.get_device());

  c10::DeviceGuard device_guard(q.device());
  auto grad_like = [&](c10::optional<at::Tensor>& g, const char* name) {
    if (g.has_value()) {
      at::Tensor t = g.value();
      TORCH_CHECK(t.dtype() == q_dtype, name, " must have the same dtype as q");
      TORCH_CHECK(t.is_cuda(), name, " must be on the GPU");
      TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
      TORCH_CHECK(t.sizes() == q.sizes(), name, " must have the shape of q");
      return t;
    }
    return torch::empty({batch_size, seqlen_q, num_heads, head_size}, q.options());
  };
  at::Tensor dq = grad_like(dq_, "dq"), dk = grad_like(dk_, "dk"), dv = grad_like(dv_, "dv");

  const Operand qo = operand(q), ko = operand(k), vo = operand(v), go = operand(dout);
  at::Tensor od = dense(out), ld = dense(lse);
  const size_t ws_bytes = fused_mha_backward_workspace_bytes(batch_size, num_heads, seqlen_q, head_size);
  auto workspace = torch::empty({(int64_t)ws_bytes}, q.options().dtype(at::kByte));
  hipStream_t stream = c10::hip::getCurrentHIPStream().stream();
  check_rc(fused_mha_backward_strided(qo.t.data_ptr(), &qo.st, ko.t.data_ptr(), &ko.st, vo.t.data_ptr(), &vo.st,
                                      od.data_ptr(), go.t.data_ptr(), &go.st, ld.data_ptr(), workspace.data_ptr(),
                                      ws_bytes, dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), batch_size, num_heads,
                                      seqlen_q, head_size, softmax_scale, is_causal ? 1 : 0, stream),
           "fused_mha_backward");
  return {dq, dk, dv};
}

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.doc() = "FlashAttention forward/backward for gfx950";
  m.def("fwd", &mha_fwd, "Forward pass");
  m.def("bwd", &mha_bwd, "Backward pass");
}
