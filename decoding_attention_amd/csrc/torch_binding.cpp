// PyTorch-ROCm extension module `decoding_attn_hip`: tensor-level entry `fwd` over the C-ABI of
// libdecoding_attn_hip.so.
//
// Stands where the reference's pybind module does (csrc/torch/decoding_torch.cpp:19-85, module
// `decoding_attn_cuda`, function `fwd`): same argument list, same checks in the same order, an output tensor
// allocated when none is passed, launch on torch's current stream.  Added over the reference: a device guard on
// q's device, dense layouts required (the op derives strides from head counts), total_q == batch, supported
// (dim, dim_v) only, an error instead of a silent no-op, and the two optional constants (softmax scale, ALiBi
// slopes) of the extended C-ABI entry.  This file is host C++ only; it contains no device code.
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <torch/extension.h>

#include <optional>

#include "../../include/decoding_attn_hip.h"

namespace {

#define DA_CHECK_DEVICE(x) TORCH_CHECK(x.is_cuda(), #x " must be on the GPU")
#define DA_CHECK_SHAPE(x, ...) \
    TORCH_CHECK(x.sizes() == torch::IntArrayRef({__VA_ARGS__}), #x " must have shape (" #__VA_ARGS__ ")")
#define DA_CHECK_CONTIGUOUS(x) TORCH_CHECK(x.is_contiguous(), #x " must be contiguous")

at::Tensor dmha_fwd(const at::Tensor &q, const at::Tensor &k, const std::optional<at::Tensor> &v_,
                    const std::optional<at::Tensor> &o_, const at::Tensor &cu_seq_k, const int64_t max_seq_k,
                    const int64_t dim_v, const bool is_alibi, const std::optional<double> softmax_scale,
                    const std::optional<at::Tensor> &alibi_slopes) {
    auto q_dtype = q.dtype();
    TORCH_CHECK(q_dtype == torch::kFloat16 || q_dtype == torch::kBFloat16,
                "Decoding-Attention only support FP16 and BF16 data type");
    const bool is_bf16 = q_dtype == torch::kBFloat16;
    TORCH_CHECK(k.dtype() == q_dtype, "query and key must have the same dtype");
    TORCH_CHECK(cu_seq_k.dtype() == torch::kInt32, "cu_seq_k must have dtype int32");

    DA_CHECK_DEVICE(q);
    DA_CHECK_DEVICE(k);
    DA_CHECK_DEVICE(cu_seq_k);
    TORCH_CHECK(k.device() == q.device() && cu_seq_k.device() == q.device(), "q, k and cu_seq_k must share a device");

    TORCH_CHECK(q.dim() == 3 && k.dim() == 3, "q and k must have three dimensions (tokens, heads, dim)");
    TORCH_CHECK(q.stride(-1) == 1, "query must have contiguous last dimension");
    TORCH_CHECK(k.stride(-1) == 1, "key must have contiguous last dimension");
    DA_CHECK_CONTIGUOUS(cu_seq_k);

    const int64_t batch = cu_seq_k.numel() - 1;
    const int64_t total_q = q.size(0);
    const int64_t head_q = q.size(1);
    const int64_t dim = q.size(2);
    const int64_t total_k = k.size(0);
    const int64_t head_k = k.size(1);
    TORCH_CHECK(batch > 0, "batch size must be positive");
    TORCH_CHECK(dim <= 576, "dim should be at most 576");
    TORCH_CHECK(dim_v <= 512, "dim_v should be at most 512");
    TORCH_CHECK(head_q % head_k == 0, "number of heads in key/value must divide number of heads in query");

    DA_CHECK_SHAPE(q, total_q, head_q, dim);
    DA_CHECK_SHAPE(k, total_k, head_k, dim);
    DA_CHECK_SHAPE(cu_seq_k, batch + 1);
    DA_CHECK_CONTIGUOUS(q);
    DA_CHECK_CONTIGUOUS(k);
    TORCH_CHECK(total_q == batch, "one query token per sequence: q.size(0) must equal cu_seq_k.numel() - 1");
    TORCH_CHECK(da_supported_head_dims((size_t)dim, (size_t)dim_v) == 1, "unsupported head dims (dim ", dim,
                ", dim_v ", dim_v, "): supported are (64,64) (96,96) (128,128) (256,256) (576,512)");

    const void *v_ptr = nullptr;
    if (v_.has_value()) {
        const at::Tensor &v = v_.value();
        TORCH_CHECK(v.dtype() == q_dtype, "query and value must have the same dtype");
        DA_CHECK_DEVICE(v);
        TORCH_CHECK(v.device() == q.device(), "v must be on q's device");
        TORCH_CHECK(v.stride(-1) == 1, "value must have contiguous last dimension");
        DA_CHECK_SHAPE(v, total_k, head_k, dim_v);
        DA_CHECK_CONTIGUOUS(v);
        v_ptr = v.data_ptr();
    } else {
        TORCH_CHECK(dim_v <= dim, "without v the values are the first dim_v columns of k: dim_v must not exceed dim");
    }

    at::Tensor o;
    if (o_.has_value()) {
        o = o_.value();
        TORCH_CHECK(o.dtype() == q_dtype, "Output must have the same dtype as inputs");
        DA_CHECK_DEVICE(o);
        TORCH_CHECK(o.device() == q.device(), "o must be on q's device");
        TORCH_CHECK(o.stride(-1) == 1, "Output tensor must have contiguous last dimension");
        DA_CHECK_SHAPE(o, total_q, head_q, dim_v);
        DA_CHECK_CONTIGUOUS(o);
    } else {
        o = torch::empty({total_q, head_q, dim_v}, q.options());
    }

    const float *slopes_ptr = nullptr;
    if (alibi_slopes.has_value()) {
        const at::Tensor &s = alibi_slopes.value();
        TORCH_CHECK(s.dtype() == torch::kFloat32 && s.is_cuda() && s.device() == q.device() && s.is_contiguous() &&
                        s.numel() == head_q,
                    "alibi_slopes must be a contiguous float32 GPU tensor of head_q values");
        slopes_ptr = s.data_ptr<float>();
    }

    // launch on q's device and on torch's current stream for it
    c10::hip::HIPGuardMasqueradingAsCUDA guard(q.device());
    hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(q.device().index()).stream();

    // k.size(0) is the sum of the key lengths: a free host-side hint for sizing the sequence splits
    const size_t ws_bytes = da_workspace_bytes((size_t)max_seq_k, (size_t)batch, (size_t)head_q, (size_t)head_k,
                                               (size_t)dim, (size_t)dim_v, (size_t)total_k);
    at::Tensor ws;  // from torch's stream-aware caching allocator
    if (ws_bytes > 0) ws = torch::empty({(int64_t)ws_bytes}, q.options().dtype(torch::kUInt8));

    const int rc = da_decoding_attn_ex(
        q.data_ptr(), k.data_ptr(), v_ptr, o.data_ptr(), cu_seq_k.data_ptr<int32_t>(), (size_t)max_seq_k,
        (size_t)batch, (size_t)head_q, (size_t)head_k, (size_t)dim, (size_t)dim_v, is_alibi ? 1 : 0, is_bf16 ? 1 : 0,
        softmax_scale.has_value() ? (float)softmax_scale.value() : 0.0f, slopes_ptr, (size_t)total_k,
        ws_bytes > 0 ? ws.data_ptr() : nullptr, ws_bytes, (void *)stream);
    TORCH_CHECK(rc == DA_OK, "decoding_attn failed (", rc, "): ", da_last_error());
    return o;
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.doc() = "Decoding-Attention for MI355X (gfx950)";
    m.def("fwd", &dmha_fwd, "Forward pass", pybind11::arg("q"), pybind11::arg("k"), pybind11::arg("v_"),
          pybind11::arg("o_"), pybind11::arg("cu_seq_k"), pybind11::arg("max_seq_k"), pybind11::arg("dim_v"),
          pybind11::arg("is_alibi"), pybind11::arg("softmax_scale") = pybind11::none(),
          pybind11::arg("alibi_slopes") = pybind11::none());
}
