// Compiled PyTorch binding of the librlk_hip C ABI under the symbol names of the reference's
// extension module (csrc/ops.cpp:75-99, rl_engine/_C.pyi:5-43 of the reference): a wrapper that
// probes `hasattr(_C, "fused_linear_logp_sm90")` or `hasattr(_C, "fused_logp_forward_out")` finds
// them here.  Host code only: tensors in, raw device pointers and the current HIP stream down to
// the C ABI, error codes back up as exceptions (TORCH_CHECK -> RuntimeError, as the reference's
// native side raises).
#include <torch/extension.h>

#include <ATen/hip/HIPContext.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>

#include <vector>

#include "rlk_hip.h"

namespace {

int dtype_id(at::ScalarType t)
{
    switch (t) {
        case at::kBFloat16: return RLK_DTYPE_BF16;
        case at::kHalf: return RLK_DTYPE_F16;
        case at::kFloat: return RLK_DTYPE_F32;
        case at::kDouble: return RLK_DTYPE_F64;
        default: return -1;
    }
}

rlk_stream_t current_stream(const at::Tensor& t)
{
    return reinterpret_cast<rlk_stream_t>(at::hip::getCurrentHIPStream(t.get_device()).stream());
}

// [logp, lse] fp32 of a (possibly vocab-sharded) head; a target outside the shard gives
// logp = -lse (z_t = 0), as csrc/cuda/fused_linear_logp_sm90.cu:256-280 of the reference does.
std::vector<at::Tensor> fused_linear_logp(at::Tensor hidden, at::Tensor weight, at::Tensor target,
                                          c10::optional<at::Tensor> bias)
{
    TORCH_CHECK(hidden.dim() == 2 && weight.dim() == 2, "hidden and weight must be 2D tensors");
    TORCH_CHECK(hidden.is_cuda() && weight.is_cuda(), "hidden and weight must be CUDA tensors");
    // allocations and launches below go to the tensors' GPU, whichever device is current
    const c10::hip::HIPGuardMasqueradingAsCUDA device_guard(hidden.device());
    TORCH_CHECK(weight.size(1) == hidden.size(1), "hidden/weight hidden-dim mismatch");
    TORCH_CHECK(target.numel() == hidden.size(0), "target must have one id per token: expected ",
                hidden.size(0), " (hidden rows), got ", target.numel());
    TORCH_CHECK(weight.scalar_type() == hidden.scalar_type(), "hidden and weight must share a dtype");
    const int dt = dtype_id(hidden.scalar_type());
    TORCH_CHECK(dt == RLK_DTYPE_BF16 || dt == RLK_DTYPE_F16 || dt == RLK_DTYPE_F32,
                "hidden dtype must be bfloat16, float16 or float32");
    auto h = hidden.contiguous(), w = weight.contiguous();
    auto t = target.reshape({-1}).to(hidden.device(), at::kLong).contiguous();
    const int64_t n = h.size(0), v = w.size(0);
    const int32_t hd = static_cast<int32_t>(h.size(1));
    auto f32 = h.options().dtype(at::kFloat);
    auto logp = at::empty({n}, f32), lse = at::empty({n}, f32);
    if (n == 0) return {logp, lse};
    size_t ws_bytes = 0;
    TORCH_CHECK(rlk_linear_logp_fwd_workspace_bytes(n, hd, v, dt, &ws_bytes) == 0, rlk_last_error());
    auto ws = at::empty({static_cast<int64_t>(ws_bytes < 16 ? 16 : ws_bytes)}, h.options().dtype(at::kByte));
    at::Tensor bias_f;
    const float* bias_p = nullptr;
    if (bias.has_value() && bias->defined()) {
        TORCH_CHECK(bias->numel() == v, "bias must have one value per vocab row");
        bias_f = bias->to(hidden.device(), at::kFloat).contiguous();
        bias_p = bias_f.data_ptr<float>();
    }
    const int rc = rlk_linear_logp_fwd(h.data_ptr(), w.data_ptr(), bias_p, t.data_ptr<int64_t>(),
                                       logp.data_ptr<float>(), lse.data_ptr<float>(), ws.data_ptr(),
                                       static_cast<size_t>(ws.numel()), n, hd, v, /*vocab_start=*/0, dt,
                                       /*temperature=*/1.f, /*ignore_index=*/0, /*use_ignore=*/0,
                                       /*strict_targets=*/0, /*err_flag=*/nullptr, current_stream(h));
    TORCH_CHECK(rc == 0, "rlk_linear_logp_fwd: ", rlk_last_error());
    return {logp, lse};
}

// Forward with the keyword extensions of the op classes (temperature, ignore-index, strictness):
// [logp, lse, err_flag]; err_flag (int32[1], device) is non-zero when strict_targets and a
// non-ignored target lies outside the shard.  Does not synchronise.
std::vector<at::Tensor> fused_linear_logp_forward_ex(at::Tensor hidden, at::Tensor weight, at::Tensor target,
                                                     c10::optional<at::Tensor> bias, double temperature,
                                                     c10::optional<int64_t> ignore_index, int64_t vocab_start,
                                                     bool strict_targets)
{
    TORCH_CHECK(hidden.dim() == 2 && weight.dim() == 2, "hidden and weight must be 2D tensors");
    TORCH_CHECK(hidden.is_cuda() && weight.is_cuda(), "hidden and weight must be CUDA tensors");
    const c10::hip::HIPGuardMasqueradingAsCUDA device_guard(hidden.device());
    TORCH_CHECK(weight.size(1) == hidden.size(1), "hidden/weight hidden-dim mismatch");
    TORCH_CHECK(target.numel() == hidden.size(0), "target must have one id per token");
    TORCH_CHECK(weight.scalar_type() == hidden.scalar_type(), "hidden and weight must share a dtype");
    TORCH_CHECK(hidden.is_contiguous() && weight.is_contiguous(), "hidden and weight must be contiguous");
    TORCH_CHECK(target.scalar_type() == at::kLong && target.is_contiguous() && target.is_cuda(),
                "target must be a contiguous int64 CUDA tensor");
    const int dt = dtype_id(hidden.scalar_type());
    TORCH_CHECK(dt == RLK_DTYPE_BF16 || dt == RLK_DTYPE_F16 || dt == RLK_DTYPE_F32,
                "hidden dtype must be bfloat16, float16 or float32");
    const int64_t n = hidden.size(0), v = weight.size(0);
    const int32_t hd = static_cast<int32_t>(hidden.size(1));
    auto f32 = hidden.options().dtype(at::kFloat);
    auto logp = at::empty({n}, f32), lse = at::empty({n}, f32);
    auto err = at::zeros({1}, hidden.options().dtype(at::kInt));
    if (n == 0) return {logp, lse, err};
    size_t ws_bytes = 0;
    TORCH_CHECK(rlk_linear_logp_fwd_workspace_bytes(n, hd, v, dt, &ws_bytes) == 0, rlk_last_error());
    auto ws = at::empty({static_cast<int64_t>(ws_bytes < 16 ? 16 : ws_bytes)}, hidden.options().dtype(at::kByte));
    at::Tensor bias_f;
    const float* bias_p = nullptr;
    if (bias.has_value() && bias->defined()) {
        TORCH_CHECK(bias->numel() == v, "bias must have one value per vocab row");
        bias_f = bias->detach().to(hidden.device(), at::kFloat).contiguous();
        bias_p = bias_f.data_ptr<float>();
    }
    const int rc = rlk_linear_logp_fwd(hidden.data_ptr(), weight.data_ptr(), bias_p, target.data_ptr<int64_t>(),
                                       logp.data_ptr<float>(), lse.data_ptr<float>(), ws.data_ptr(),
                                       static_cast<size_t>(ws.numel()), n, hd, v, vocab_start, dt,
                                       static_cast<float>(temperature), ignore_index.value_or(0),
                                       ignore_index.has_value() ? 1 : 0, strict_targets ? 1 : 0,
                                       err.data_ptr<int32_t>(), current_stream(hidden));
    TORCH_CHECK(rc != RLK_ERR_ARG, "rlk_linear_logp_fwd: ", rlk_last_error());
    TORCH_CHECK(rc == 0, "rlk_linear_logp_fwd: ", rlk_last_error());
    return {logp, lse, err};
}

// Backward: [d_hidden (input dtype), d_weight (f32), d_bias (f32)], an undefined tensor for every
// gradient that is not wanted.  weight_grad_out / bias_grad_out: caller-owned fp32 buffers that
// receive (accumulate: are added) the gradients and are what the call returns in their place.
std::vector<at::Tensor> fused_linear_logp_backward(at::Tensor grad_logp, at::Tensor hidden, at::Tensor weight,
                                                   at::Tensor target, at::Tensor lse,
                                                   c10::optional<at::Tensor> bias, double temperature,
                                                   c10::optional<int64_t> ignore_index, int64_t vocab_start,
                                                   bool need_hidden, bool need_weight, bool need_bias,
                                                   int64_t dz_budget_bytes,
                                                   c10::optional<at::Tensor> weight_grad_out,
                                                   c10::optional<at::Tensor> bias_grad_out, bool accumulate)
{
    TORCH_CHECK(hidden.dim() == 2 && weight.dim() == 2, "hidden and weight must be 2D tensors");
    TORCH_CHECK(hidden.is_cuda() && weight.is_cuda(), "hidden and weight must be CUDA tensors");
    const c10::hip::HIPGuardMasqueradingAsCUDA device_guard(hidden.device());
    TORCH_CHECK(hidden.is_contiguous() && weight.is_contiguous(), "hidden and weight must be contiguous");
    TORCH_CHECK(target.scalar_type() == at::kLong && target.is_contiguous() && target.is_cuda(),
                "target must be a contiguous int64 CUDA tensor");
    TORCH_CHECK(lse.scalar_type() == at::kFloat && lse.is_contiguous(), "lse must be contiguous float32");
    const int dt = dtype_id(hidden.scalar_type());
    TORCH_CHECK(dt == RLK_DTYPE_BF16 || dt == RLK_DTYPE_F16 || dt == RLK_DTYPE_F32,
                "hidden dtype must be bfloat16, float16 or float32");
    const int64_t n = hidden.size(0), v = weight.size(0);
    const int32_t hd = static_cast<int32_t>(hidden.size(1));
    auto g = grad_logp.reshape({-1}).to(at::kFloat).contiguous();
    TORCH_CHECK(g.numel() == n, "grad_logp must have one value per token");
    auto f32 = hidden.options().dtype(at::kFloat);
    const bool has_bias = bias.has_value() && bias->defined();
    const bool want_bias = has_bias && need_bias;
    at::Tensor d_hidden, d_weight, d_bias, bias_f;
    if (need_hidden) d_hidden = at::empty_like(hidden);
    if (need_weight) d_weight = weight_grad_out.has_value() && weight_grad_out->defined() ? *weight_grad_out
                                                                                          : at::empty({v, hd}, f32);
    if (want_bias) d_bias = bias_grad_out.has_value() && bias_grad_out->defined() ? *bias_grad_out : at::empty({v}, f32);
    if (d_weight.defined())
        TORCH_CHECK(d_weight.scalar_type() == at::kFloat && d_weight.is_contiguous() && d_weight.numel() == v * hd,
                    "weight_grad_out must be contiguous float32 [V, H]");
    if (d_bias.defined())
        TORCH_CHECK(d_bias.scalar_type() == at::kFloat && d_bias.is_contiguous() && d_bias.numel() == v,
                    "bias_grad_out must be contiguous float32 [V]");
    const float* bias_p = nullptr;
    if (has_bias) {
        bias_f = bias->detach().to(hidden.device(), at::kFloat).contiguous();
        bias_p = bias_f.data_ptr<float>();
    }
    size_t ws_bytes = 0;
    TORCH_CHECK(rlk_linear_logp_bwd_workspace_bytes(n, hd, v, dt, static_cast<size_t>(dz_budget_bytes), &ws_bytes) == 0,
                rlk_last_error());
    auto ws = at::empty({static_cast<int64_t>(ws_bytes)}, hidden.options().dtype(at::kByte));
    const int rc = rlk_linear_logp_bwd_accum(
        g.data_ptr<float>(), hidden.data_ptr(), weight.data_ptr(), bias_p, target.data_ptr<int64_t>(),
        lse.data_ptr<float>(), d_hidden.defined() ? d_hidden.data_ptr() : nullptr,
        d_weight.defined() ? d_weight.data_ptr<float>() : nullptr,
        d_bias.defined() ? d_bias.data_ptr<float>() : nullptr, ws.data_ptr(), static_cast<size_t>(ws.numel()),
        static_cast<size_t>(dz_budget_bytes), n, hd, v, vocab_start, dt, static_cast<float>(temperature),
        ignore_index.value_or(0), ignore_index.has_value() ? 1 : 0, accumulate ? 1 : 0, current_stream(hidden));
    TORCH_CHECK(rc == 0, "rlk_linear_logp_bwd_accum: ", rlk_last_error());
    return {d_hidden, d_weight, d_bias};
}

// Selected-token log-prob of materialised logits into `output` (all rows, or only row_indices).
at::Tensor scan_into(const at::Tensor& logits, const at::Tensor& token_ids,
                     const c10::optional<at::Tensor>& row_indices, at::Tensor output)
{
    TORCH_CHECK(logits.dim() == 2, "logits must be a 2D tensor");
    TORCH_CHECK(token_ids.dim() == 1 && output.dim() == 1, "token_ids and output must be 1D tensors");
    TORCH_CHECK(logits.is_cuda() && token_ids.is_cuda() && output.is_cuda(),
                "logits, token_ids and output must be CUDA tensors");
    TORCH_CHECK(token_ids.scalar_type() == at::kLong, "token_ids must be int64");
    const int64_t n = logits.size(0), v = logits.size(1);
    TORCH_CHECK(token_ids.numel() == n, "token_ids length must match logits rows");
    TORCH_CHECK(output.numel() == n, "output length must match logits rows");
    TORCH_CHECK(output.is_contiguous(), "output must be contiguous");
    TORCH_CHECK(v > 0, "logits vocab dimension must be non-empty");
    const int in_dt = dtype_id(logits.scalar_type()), out_dt = dtype_id(output.scalar_type());
    TORCH_CHECK(in_dt == RLK_DTYPE_BF16 || in_dt == RLK_DTYPE_F16 || in_dt == RLK_DTYPE_F32,
                "logits dtype must be float32, float16 or bfloat16");
    TORCH_CHECK(out_dt >= 0, "output dtype must be float64, float32, float16, or bfloat16");
    const c10::hip::HIPGuardMasqueradingAsCUDA device_guard(logits.device());
    auto lg = logits.contiguous();
    auto ids = token_ids.contiguous();
    at::Tensor idx;
    const int64_t* idx_p = nullptr;
    int64_t n_launch = n;
    if (row_indices.has_value()) {
        TORCH_CHECK(row_indices->dim() == 1 && row_indices->scalar_type() == at::kLong && row_indices->is_cuda(),
                    "row_indices must be a 1D int64 CUDA tensor");
        idx = row_indices->contiguous();
        idx_p = idx.data_ptr<int64_t>();
        n_launch = idx.numel();
    }
    const int rc = rlk_logp_from_logits(lg.data_ptr(), in_dt, ids.data_ptr<int64_t>(), output.data_ptr(),
                                        out_dt, nullptr, idx_p, n_launch, n, v, current_stream(lg));
    TORCH_CHECK(rc == 0, "rlk_logp_from_logits: ", rlk_last_error());
    return output;
}

at::Tensor fused_logp(at::Tensor logits, at::Tensor token_ids)
{
    TORCH_CHECK(logits.dim() == 2, "logits must be a 2D tensor");
    return scan_into(logits, token_ids, c10::nullopt, at::empty({logits.size(0)}, logits.options()));
}

at::Tensor fused_logp_forward_out(at::Tensor logits, at::Tensor token_ids, at::Tensor output)
{
    return scan_into(logits, token_ids, c10::nullopt, output);
}

at::Tensor fused_logp_forward_fp32(at::Tensor logits, at::Tensor token_ids)
{
    TORCH_CHECK(logits.dim() == 2, "logits must be a 2D tensor");
    return scan_into(logits, token_ids, c10::nullopt,
                     at::empty({logits.size(0)}, logits.options().dtype(at::kFloat)));
}

at::Tensor fused_logp_forward_indexed_out(at::Tensor logits, at::Tensor token_ids, at::Tensor row_indices,
                                          at::Tensor output)
{
    return scan_into(logits, token_ids, row_indices, output);
}

at::Tensor fused_logp_forward_indexed_fp32(at::Tensor logits, at::Tensor token_ids, at::Tensor row_indices)
{
    TORCH_CHECK(logits.dim() == 2, "logits must be a 2D tensor");
    return scan_into(logits, token_ids, row_indices,
                     at::zeros({logits.size(0)}, logits.options().dtype(at::kFloat)));
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m)
{
    m.doc() = "librlk_hip (gfx950) under the symbol names of the RL-Kernel extension module";
    m.def("fused_logp", &fused_logp, "Selected-token logp of logits (logits dtype)");
    m.def("fused_logp_sm90", &fused_logp, "Alias of fused_logp (the reference's TMA variant)");
    m.def("fused_linear_logp", &fused_linear_logp, "Fused linear log-prob -> [logp, lse]",
          pybind11::arg("hidden"), pybind11::arg("weight"), pybind11::arg("target"),
          pybind11::arg("bias") = pybind11::none());
    m.def("fused_linear_logp_sm90", &fused_linear_logp, "Fused linear log-prob -> [logp, lse]",
          pybind11::arg("hidden"), pybind11::arg("weight"), pybind11::arg("target"),
          pybind11::arg("bias") = pybind11::none());
    m.def("fused_linear_logp_forward_ex", &fused_linear_logp_forward_ex,
          "Fused linear log-prob with temperature / ignore-index -> [logp, lse, err_flag]",
          pybind11::arg("hidden"), pybind11::arg("weight"), pybind11::arg("target"),
          pybind11::arg("bias") = pybind11::none(), pybind11::arg("temperature") = 1.0,
          pybind11::arg("ignore_index") = pybind11::none(), pybind11::arg("vocab_start") = 0,
          pybind11::arg("strict_targets") = true);
    m.def("fused_linear_logp_backward", &fused_linear_logp_backward,
          "Backward of the fused linear log-prob -> [d_hidden, d_weight (f32), d_bias (f32)]",
          pybind11::arg("grad_logp"), pybind11::arg("hidden"), pybind11::arg("weight"),
          pybind11::arg("target"), pybind11::arg("lse"), pybind11::arg("bias") = pybind11::none(),
          pybind11::arg("temperature") = 1.0, pybind11::arg("ignore_index") = pybind11::none(),
          pybind11::arg("vocab_start") = 0, pybind11::arg("need_hidden") = true,
          pybind11::arg("need_weight") = true, pybind11::arg("need_bias") = true,
          pybind11::arg("dz_budget_bytes") = 0, pybind11::arg("weight_grad_out") = pybind11::none(),
          pybind11::arg("bias_grad_out") = pybind11::none(), pybind11::arg("accumulate") = false);
    m.def("fused_logp_forward_out", &fused_logp_forward_out, "Fused logp out");
    m.def("fused_logp_forward_fp32", &fused_logp_forward_fp32, "Fused logp fp32");
    m.def("fused_logp_forward_indexed_out", &fused_logp_forward_indexed_out, "Fused logp indexed out");
    m.def("fused_logp_forward_indexed_fp32", &fused_logp_forward_indexed_fp32, "Fused logp indexed fp32");
    m.def("fused_logp_forward_online_out", &fused_logp_forward_out, "Fused logp online out");
    m.def("fused_logp_forward_online_fp32", &fused_logp_forward_fp32, "Fused logp online fp32");
    m.def("fused_logp_forward_online_indexed_out", &fused_logp_forward_indexed_out, "Fused logp online indexed out");
    m.def("fused_logp_forward_online_indexed_fp32", &fused_logp_forward_indexed_fp32, "Fused logp online indexed fp32");
    m.def("rlk_version", []() { return rlk_version(); }, "ABI version of the linked librlk_hip");
}
