// Autograd boundary in C++: FlashAttentionV2Function of the reference
// (src/flash_attention_triton/flash_attention_2.py:280-384) as a torch::autograd::Function whose
// forward and backward call the C ABI of libfa2_gfx950.so directly.
//
// Why it exists: with the autograd function written in Python, PyTorch's backward engine has to
// hand the backward to its device thread and that thread has to take the interpreter lock; at
// the smallest workloads that hand-over and the interpreter's own overhead cost three times what
// the kernels take (B=2 H=4 N=512 D=64: 110 us per forward + backward step, 38 us of kernels).  A
// C++ node needs neither.  The Python module keeps the reference-shaped class as well and uses
// this one when it is built.
//
// Host code only: tensors come in validated (CUDA device, fp16 or bf16, contiguous, equal dtypes)
// from the Python wrapper, which also owns the reference's assertions and exception types.
#include <torch/extension.h>

#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>

#include <cmath>
#include <stdexcept>
#include <string>

#include "fa2_gfx950.h"

namespace {

fa2_tensor as_arg(const at::Tensor &t) {
  return fa2_tensor{t.data_ptr(), t.stride(0), t.stride(1), t.stride(2)};
}

void check(int status, const char *what) {
  if (status == FA2_OK) return;
  throw std::runtime_error(std::string(what) + " failed: " + fa2_status_string(status) + ": " +
                           fa2_last_error_string());
}

void *current_stream(const at::Tensor &t) {
  return static_cast<void *>(c10::hip::getCurrentHIPStream(t.device().index()).stream());
}

int dtype_code(const at::Tensor &t) { return t.scalar_type() == at::kBFloat16 ? FA2_DTYPE_BF16 : FA2_DTYPE_F16; }

int64_t rounded(int64_t seqlen_q, int64_t max_headdim) {
  return (seqlen_q + max_headdim - 1) / max_headdim * max_headdim;
}

struct FlashAttentionV2 : public torch::autograd::Function<FlashAttentionV2> {
  // softmax_scale > 0 (the wrapper folds a negative scale into the sign of q).
  static at::Tensor forward(torch::autograd::AutogradContext *ctx, const at::Tensor &q, const at::Tensor &k,
                            const at::Tensor &v, double softmax_scale, bool deterministic,
                            int64_t max_headdim, bool forward_only) {
    const c10::DeviceGuard guard(q.device());
    const int64_t batch = q.size(0), nheads = q.size(1), seqlen_q = q.size(2), headdim = q.size(3);
    const int64_t seqlen_k = k.size(2);
    const int64_t seqlen_q_rounded = rounded(seqlen_q, max_headdim);
    at::Tensor o = at::empty_like(q);
    at::Tensor lse = at::empty({batch, nheads, seqlen_q_rounded}, q.options().dtype(at::kFloat));

    fa2_fwd_args a;
    a.q = as_arg(q);
    a.k = as_arg(k);
    a.v = as_arg(v);
    a.o = as_arg(o);
    a.lse = lse.data_ptr<float>();
    a.batch = (int)batch;
    a.nheads = (int)nheads;
    a.seqlen_q = (int)seqlen_q;
    a.seqlen_k = (int)seqlen_k;
    a.headdim = (int)headdim;
    a.seqlen_q_rounded = (int)seqlen_q_rounded;
    a.softmax_scale = (float)softmax_scale;
    a.dtype = dtype_code(q);
    // forward_only: the caller knows that nothing will be differentiated, so no backward reads lse.
    a.config_id = forward_only ? fa2_pick_config_forward_only(a.dtype, a.headdim, a.seqlen_q, a.seqlen_k)
                               : FA2_CONFIG_AUTO;
    if (forward_only && a.config_id < 0) check(-a.config_id, "fa2_pick_config_forward_only");
    check(fa2_fwd_packed(&a, current_stream(q)), "fa2_fwd");

    ctx->save_for_backward({q, k, v, o, lse});
    ctx->saved_data["softmax_scale"] = softmax_scale;
    ctx->saved_data["deterministic"] = deterministic;
    return o;
  }

  static torch::autograd::variable_list backward(torch::autograd::AutogradContext *ctx,
                                                 torch::autograd::variable_list grads) {
    const auto saved = ctx->get_saved_variables();
    const at::Tensor &q = saved[0], &k = saved[1], &v = saved[2], &o = saved[3], &lse = saved[4];
    const c10::DeviceGuard guard(q.device());
    // Like the reference (flash_attention_2.py:364) the backward is not differentiable.
    const at::NoGradGuard no_grad;
    at::Tensor d_o = grads[0];
    if (d_o.scalar_type() != q.scalar_type()) d_o = d_o.to(q.scalar_type());
    d_o = d_o.contiguous();
    at::Tensor dq = at::empty_like(q), dk = at::empty_like(k), dv = at::empty_like(v);
    at::Tensor delta = at::empty_like(lse);

    // Both launches of the reference launcher (preprocess, then the main kernel) in one call:
    // with `o` in the record the library forms delta on the way.
    fa2_bwd_args a;
    a.q = as_arg(q);
    a.k = as_arg(k);
    a.v = as_arg(v);
    a.o = as_arg(o);
    a.d_o = as_arg(d_o);
    a.dq = as_arg(dq);
    a.dk = as_arg(dk);
    a.dv = as_arg(dv);
    a.lse = lse.data_ptr<float>();
    a.delta = delta.data_ptr<float>();
    a.workspace = nullptr;  // fa2_bwd_workspace_bytes is 0: dQ is written directly
    a.batch = (int)q.size(0);
    a.nheads = (int)q.size(1);
    a.seqlen_q = (int)q.size(2);
    a.seqlen_k = (int)k.size(2);
    a.headdim = (int)q.size(3);
    a.seqlen_q_rounded = (int)lse.size(2);
    a.softmax_scale = (float)ctx->saved_data["softmax_scale"].toDouble();
    a.dtype = dtype_code(q);
    a.deterministic = ctx->saved_data["deterministic"].toBool() ? 1 : 0;
    a.config_id = FA2_CONFIG_AUTO;
    check(fa2_bwd_packed(&a, current_stream(q)), "fa2_bwd");
    return {dq, dk, dv, at::Tensor(), at::Tensor(), at::Tensor(), at::Tensor()};
  }
};

at::Tensor flash_attention_v2(const at::Tensor &q, const at::Tensor &k, const at::Tensor &v,
                              double softmax_scale, bool deterministic, int64_t max_headdim, bool forward_only) {
  return FlashAttentionV2::apply(q, k, v, softmax_scale, deterministic, max_headdim, forward_only);
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.doc() = "C++ autograd node over the C ABI of libfa2_gfx950.so";
  m.def("flash_attention_v2", &flash_attention_v2,
        "q, k, v: contiguous CUDA fp16/bf16 (B, H, N, D); softmax_scale > 0; returns o",
        py::arg("q"), py::arg("k"), py::arg("v"), py::arg("softmax_scale"), py::arg("deterministic"),
        py::arg("max_headdim"), py::arg("forward_only") = false);
  m.def("abi_version", []() { return fa2_abi_version(); });
}
