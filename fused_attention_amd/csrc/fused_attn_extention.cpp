// PyTorch-ROCm binding of the gfx950 fused attention forward: Python module `fused_attn`.
//
// Host-only C++ (compiled by g++, no device code): it validates the tensors, allocates the
// output and hands raw device pointers plus torch's current HIP stream to the C ABI of
// libfused_attn_gfx950.so.  It keeps the entry point of the reference binding
// (reference src/fused_attn_extention.cu:15-22 and :119-129): same module name, same function
// name, same argument names, order and default.
//
// Contract kept from the reference (src/fused_attn_extention.cu:24-64):
//   queries, keys, values : fp16, on the GPU, contiguous, 3-D [batch, seq_len, num_features],
//                           equal shapes, num_features % head_dim == 0
//   mask (optional)       : fp16, on the GPU, contiguous, 3-D
//   head_dim, chunk_size  : powers of two, 16 <= head_dim <= 128, 16 <= chunk_size <= 128,
//                           chunk_size <= 2 * head_dim, not (chunk_size 16 with head_dim 128)
//   returns               : new fp16 [batch, seq_len, num_features] tensor
// Deliberate differences:
//   - seq_len need not be a multiple of chunk_size (the reference rejects it at :63); the key
//     tile is chosen by the kernel library and chunk_size is only validated;
//   - the mask must be [batch, seq_len, seq_len] and is applied to every key;
//   - the output lives on the device of `queries` and the launch goes to torch's current
//     stream (the reference uses the default device and the legacy default stream);
//   - every rejected argument raises with a message, and a launch failure raises instead of
//     terminating the process (reference include/fused_attn.cuh:17-42 calls std::exit).
#include <torch/extension.h>

// PyTorch-ROCm presents its HIP devices under the device type "cuda"; these are the guard and
// stream accessors that understand that.
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>

#include <cmath>
#include <string>
#include <utility>
#include <vector>

#include "fused_attn.h"

namespace {

void check_qkv(const torch::Tensor& t, const char* name) {
    TORCH_CHECK(t.dtype() == torch::kFloat16, name, " must be float16, got ", t.dtype());
    TORCH_CHECK(t.device().type() == torch::kCUDA, name, " must be a GPU tensor, got device ",
                t.device());
    TORCH_CHECK(t.dim() == 3, name, " must be 3-D [batch, seq_len, num_features], got ", t.dim(),
                " dimensions");
    TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
}

bool is_pow2(int64_t x) { return x > 0 && (x & (x - 1)) == 0; }

torch::Tensor attention_forward(int64_t head_dim, int64_t chunk_size, torch::Tensor queries,
                                torch::Tensor keys, torch::Tensor values,
                                std::optional<torch::Tensor> mask) {
    TORCH_CHECK(is_pow2(head_dim) && 16 <= head_dim && head_dim <= 128,
                "head_dim must be a power of two in [16, 128], got ", head_dim);
    TORCH_CHECK(is_pow2(chunk_size) && 16 <= chunk_size && chunk_size <= 128,
                "chunk_size must be a power of two in [16, 128], got ", chunk_size);
    TORCH_CHECK(chunk_size <= 2 * head_dim, "chunk_size must not exceed 2 * head_dim, got chunk_size ",
                chunk_size, " with head_dim ", head_dim);
    TORCH_CHECK(!(chunk_size == 16 && head_dim == 128),
                "chunk_size 16 with head_dim 128 is not a supported combination");
    TORCH_CHECK(fa_fwd_query(head_dim) == 1, "head_dim ", head_dim,
                " is not supported by the kernel library");

    check_qkv(queries, "queries");
    check_qkv(keys, "keys");
    check_qkv(values, "values");

    const int64_t batch_size = queries.size(0);
    const int64_t seq_len = queries.size(1);
    const int64_t num_features = queries.size(2);
    TORCH_CHECK(keys.sizes() == queries.sizes(), "keys must have the shape of queries ",
                queries.sizes(), ", got ", keys.sizes());
    TORCH_CHECK(values.sizes() == queries.sizes(), "values must have the shape of queries ",
                queries.sizes(), ", got ", values.sizes());
    TORCH_CHECK(keys.device() == queries.device() && values.device() == queries.device(),
                "queries, keys and values must be on the same device");
    TORCH_CHECK(batch_size >= 1 && seq_len >= 1 && num_features >= 1,
                "queries must not have an empty dimension, got ", queries.sizes());
    TORCH_CHECK(num_features % head_dim == 0, "num_features (", num_features,
                ") must be a multiple of head_dim (", head_dim, ")");

    const void* mask_ptr = nullptr;
    if (mask.has_value()) {
        const torch::Tensor& m = *mask;
        TORCH_CHECK(m.dtype() == torch::kFloat16, "mask must be float16, got ", m.dtype());
        TORCH_CHECK(m.device() == queries.device(), "mask must be on the device of queries");
        TORCH_CHECK(m.dim() == 3 && m.is_contiguous(), "mask must be a contiguous 3-D tensor");
        TORCH_CHECK(m.size(0) == batch_size && m.size(1) == seq_len && m.size(2) == seq_len,
                    "mask must have shape [batch, seq_len, seq_len] = [", batch_size, ", ", seq_len,
                    ", ", seq_len, "], got ", m.sizes());
        mask_ptr = m.data_ptr<at::Half>();
    }

    const c10::hip::HIPGuardMasqueradingAsCUDA device_guard(queries.device());
    torch::Tensor output = torch::empty_like(queries);
    const int64_t num_heads = num_features / head_dim;
    const float scale = 1.0f / std::sqrt(static_cast<float>(head_dim));
    hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(queries.device().index()).stream();

    const int status = fa_fwd(queries.data_ptr<at::Half>(), keys.data_ptr<at::Half>(),
                              values.data_ptr<at::Half>(), mask_ptr, output.data_ptr<at::Half>(),
                              batch_size, num_heads, seq_len, head_dim,
                              /*stride_b=*/seq_len * num_features, /*stride_h=*/head_dim,
                              /*stride_l=*/num_features, scale, static_cast<void*>(stream));
    TORCH_CHECK(status == FA_OK, "fused attention launch failed: ", fa_strerror(status));
    return output;
}

// The extensions of the C ABI through the compiled module (no counterpart in the reference, whose
// entry point takes contiguous fp16 tensors only, reference src/fused_attn_extention.cu:24-44, and
// is kept untouched above): fp16 or bf16; q, k, v may be views with a dense last dimension and
// equal strides (three slices of the packed tensor qkv_projection returns, say); layout "blf" takes
// [batch, seq_len, num_heads * head_dim] tensors, "bhld" [batch, num_heads, seq_len, head_dim];
// causal restricts query i to keys j <= i (not together with a mask); return_lse adds the float32
// [batch, num_heads, seq_len] log-sum-exp of every score row.  The output is a new dense tensor
// of the shape of queries.  Returns {output} or {output, lse} (a tensor or a pair in Python).
std::vector<torch::Tensor> attention_forward_ex(torch::Tensor queries, torch::Tensor keys, torch::Tensor values,
                                                int64_t head_dim, std::optional<torch::Tensor> mask, bool causal,
                                                bool return_lse, const std::string& layout,
                                                std::optional<double> scale) {
    TORCH_CHECK(fa_fwd_query(head_dim) == 1, "head_dim must be 16, 32, 64 or 128, got ", head_dim);
    TORCH_CHECK(layout == "blf" || layout == "bhld", "layout must be \"blf\" or \"bhld\", got \"", layout, "\"");
    const bool blf = layout == "blf";
    TORCH_CHECK(queries.dtype() == torch::kFloat16 || queries.dtype() == torch::kBFloat16,
                "queries must be float16 or bfloat16, got ", queries.dtype());
    const int64_t want_dim = blf ? 3 : 4;
    TORCH_CHECK(queries.dim() == want_dim, "layout \"", layout, "\" takes ", want_dim, "-D tensors, queries has ",
                queries.dim(), " dimensions");
    for (const auto& [t, name] : {std::pair<const torch::Tensor&, const char*>{keys, "keys"}, {values, "values"}}) {
        TORCH_CHECK(t.dtype() == queries.dtype(), name, " must have the dtype of queries (", queries.dtype(), "), got ",
                    t.dtype());
        TORCH_CHECK(t.device() == queries.device(), name, " must be on the device of queries");
        TORCH_CHECK(t.sizes() == queries.sizes(), name, " must have the shape of queries ", queries.sizes(), ", got ",
                    t.sizes());
        TORCH_CHECK(t.strides() == queries.strides(), name, " must have the strides of queries ", queries.strides(),
                    ", got ", t.strides());
    }
    TORCH_CHECK(queries.numel() > 0, "queries must not have an empty dimension, got ", queries.sizes());
    TORCH_CHECK(queries.stride(-1) == 1, "the last dimension of queries, keys and values must be contiguous");
    int64_t batch_size, num_heads, seq_len, stride_b, stride_h, stride_l;
    if (blf) {
        TORCH_CHECK(queries.size(2) % head_dim == 0, "num_features (", queries.size(2),
                    ") must be a multiple of head_dim (", head_dim, ")");
        batch_size = queries.size(0), seq_len = queries.size(1), num_heads = queries.size(2) / head_dim;
        stride_b = queries.stride(0), stride_h = head_dim, stride_l = queries.stride(1);
    } else {
        TORCH_CHECK(queries.size(3) == head_dim, "the last dimension (", queries.size(3), ") must equal head_dim (",
                    head_dim, ")");
        batch_size = queries.size(0), num_heads = queries.size(1), seq_len = queries.size(2);
        stride_b = queries.stride(0), stride_h = queries.stride(1), stride_l = queries.stride(2);
    }
    TORCH_CHECK(!(causal && mask.has_value()), "causal and mask cannot be combined");
    const void* mask_ptr = nullptr;
    if (mask.has_value()) {
        const torch::Tensor& m = *mask;
        TORCH_CHECK(m.dtype() == queries.dtype(), "mask must have the dtype of queries (", queries.dtype(), "), got ",
                    m.dtype());
        TORCH_CHECK(m.device() == queries.device(), "mask must be on the device of queries");
        TORCH_CHECK(m.dim() == 3 && m.is_contiguous(), "mask must be a contiguous 3-D tensor");
        TORCH_CHECK(m.size(0) == batch_size && m.size(1) == seq_len && m.size(2) == seq_len,
                    "mask must have shape [batch, seq_len, seq_len] = [", batch_size, ", ", seq_len, ", ", seq_len,
                    "], got ", m.sizes());
        mask_ptr = m.data_ptr();
    }
    // last, so that everything above can be exercised on host tensors
    TORCH_CHECK(queries.device().type() == torch::kCUDA, "queries must be a GPU tensor, got device ", queries.device());
    const float scale_f = scale.has_value() ? static_cast<float>(*scale) : 1.0f / std::sqrt(static_cast<float>(head_dim));

    const c10::hip::HIPGuardMasqueradingAsCUDA device_guard(queries.device());
    torch::Tensor output = torch::empty(queries.sizes(), queries.options());       // dense
    const int64_t out_b = output.stride(0), out_h = blf ? head_dim : output.stride(1),
                  out_l = blf ? output.stride(1) : output.stride(2);
    torch::Tensor lse;
    if (return_lse) lse = torch::empty({batch_size, num_heads, seq_len}, queries.options().dtype(torch::kFloat32));
    const int flags = (causal ? FA_FLAG_CAUSAL : 0) | (queries.dtype() == torch::kBFloat16 ? FA_FLAG_BF16 : 0);
    hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(queries.device().index()).stream();
    const int status = fa_fwd_strided(queries.data_ptr(), keys.data_ptr(), values.data_ptr(), mask_ptr, output.data_ptr(),
                                      return_lse ? lse.data_ptr() : nullptr, batch_size, num_heads, seq_len, head_dim,
                                      stride_b, stride_h, stride_l, out_b, out_h, out_l, scale_f, flags,
                                      static_cast<void*>(stream));
    TORCH_CHECK(status == FA_OK, "fused attention launch failed: ", fa_strerror(status));
    if (return_lse) return {output, lse};
    return {output};
}

// The projection in front of the attention kernel, which the reference lists as not done (reference
// README.md:137): hidden [batch, seq_len, in_features] times weight [in_features, 3 * num_heads *
// head_dim] (+ bias) -> packed [batch, seq_len, 3, num_heads * head_dim], optionally with a rotary
// position encoding (float32 [seq_len, head_dim / 2] cos and sin tables) on the q and k slices.
torch::Tensor qkv_projection(torch::Tensor hidden, torch::Tensor weight, std::optional<torch::Tensor> bias,
                             int64_t num_heads, int64_t head_dim, std::optional<torch::Tensor> rope_cos,
                             std::optional<torch::Tensor> rope_sin) {
    TORCH_CHECK(hidden.dtype() == torch::kFloat16 || hidden.dtype() == torch::kBFloat16,
                "hidden must be float16 or bfloat16, got ", hidden.dtype());
    TORCH_CHECK(hidden.device().type() == torch::kCUDA, "hidden must be a GPU tensor, got device ", hidden.device());
    TORCH_CHECK(hidden.dim() == 3 && hidden.is_contiguous(), "hidden must be a contiguous 3-D tensor");
    TORCH_CHECK(fa_fwd_query(head_dim) == 1 && num_heads >= 1, "head_dim must be 16, 32, 64 or 128 and num_heads >= 1");
    const int64_t batch_size = hidden.size(0), seq_len = hidden.size(1), in_features = hidden.size(2);
    const int64_t num_features = num_heads * head_dim;
    TORCH_CHECK(num_features % 64 == 0, "num_heads * head_dim (", num_features,
                ") must be a multiple of 64: the three slices of the packed output start on 64-feature boundaries");
    TORCH_CHECK(in_features % 64 == 0, "in_features (", in_features,
                ") must be a multiple of 64: the contraction is walked in steps of 64");
    auto same_kind = [&](const torch::Tensor& t, const char* name) {
        TORCH_CHECK(t.dtype() == hidden.dtype() && t.device() == hidden.device() && t.is_contiguous(), name,
                    " must be a contiguous tensor with the dtype and device of hidden");
    };
    same_kind(weight, "weight");
    TORCH_CHECK(weight.dim() == 2 && weight.size(0) == in_features && weight.size(1) == 3 * num_features,
                "weight must have shape [in_features, 3 * num_heads * head_dim] = [", in_features, ", ",
                3 * num_features, "], got ", weight.sizes());
    const void* bias_ptr = nullptr;
    if (bias.has_value()) {
        same_kind(*bias, "bias");
        TORCH_CHECK(bias->dim() == 1 && bias->size(0) == 3 * num_features, "bias must have shape [", 3 * num_features, "]");
        bias_ptr = bias->data_ptr();
    }
    TORCH_CHECK(rope_cos.has_value() == rope_sin.has_value(), "rope_cos and rope_sin go together");
    const float* cos_ptr = nullptr;
    const float* sin_ptr = nullptr;
    if (rope_cos.has_value()) {
        for (const torch::Tensor* t : {&*rope_cos, &*rope_sin})
            TORCH_CHECK(t->dtype() == torch::kFloat32 && t->device() == hidden.device() && t->is_contiguous() &&
                            t->dim() == 2 && t->size(0) == seq_len && t->size(1) == head_dim / 2,
                        "rope tables must be contiguous float32 [seq_len, head_dim / 2] tensors on the device of hidden");
        cos_ptr = rope_cos->data_ptr<float>();
        sin_ptr = rope_sin->data_ptr<float>();
    }
    const c10::hip::HIPGuardMasqueradingAsCUDA device_guard(hidden.device());
    torch::Tensor qkv = torch::empty({batch_size, seq_len, 3, num_features}, hidden.options());
    hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(hidden.device().index()).stream();
    const int status = fa_qkv_proj(hidden.data_ptr(), weight.data_ptr(), bias_ptr, qkv.data_ptr(), batch_size, seq_len,
                                   in_features, num_heads, head_dim, cos_ptr, sin_ptr,
                                   hidden.dtype() == torch::kBFloat16 ? FA_FLAG_BF16 : 0, static_cast<void*>(stream));
    TORCH_CHECK(status == FA_OK, "fused QKV projection failed: ", fa_strerror(status));
    return qkv;
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.def("attention_forward", &attention_forward, py::arg("head_dim"), py::arg("chunk_size"),
          py::arg("queries"), py::arg("keys"), py::arg("values"),
          py::arg("mask") = std::optional<torch::Tensor>(), "Fused multihead attention");
    m.def("attention_forward_ex",
          [](torch::Tensor queries, torch::Tensor keys, torch::Tensor values, int64_t head_dim,
             std::optional<torch::Tensor> mask, bool causal, bool return_lse, const std::string& layout,
             std::optional<double> scale) -> py::object {
              const std::vector<torch::Tensor> r =
                  attention_forward_ex(queries, keys, values, head_dim, mask, causal, return_lse, layout, scale);
              if (r.size() == 1) return py::cast(r[0]);
              return py::make_tuple(r[0], r[1]);
          },
          py::arg("queries"), py::arg("keys"), py::arg("values"),
          py::arg("head_dim"), py::arg("mask") = std::optional<torch::Tensor>(), py::arg("causal") = false,
          py::arg("return_lse") = false, py::arg("layout") = "blf", py::arg("scale") = std::optional<double>(),
          "Fused multihead attention on fp16 or bf16 tensors or views: causal flag, additive mask, log-sum-exp, "
          "[batch, seq_len, features] or [batch, heads, seq_len, head_dim] layout.  Returns output, or (output, lse).");
    m.def("qkv_projection", &qkv_projection, py::arg("hidden"), py::arg("weight"),
          py::arg("bias") = std::optional<torch::Tensor>(), py::arg("num_heads"), py::arg("head_dim"),
          py::arg("rope_cos") = std::optional<torch::Tensor>(), py::arg("rope_sin") = std::optional<torch::Tensor>(),
          "Fused QKV projection into the packed [batch, seq_len, 3, num_heads * head_dim] tensor");
}
