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

// K/V element format: the 16-bit type of q (0), or FP8 e4m3 (1), int8 (2) or int4 (3: a uint8 tensor whose last
// dimension holds two elements to a byte) with optional per-KV-head de-quantisation factors.
int kv8_format(const at::Tensor &q, const at::Tensor &k) {
    if (k.dtype() == torch::kFloat8_e4m3fn) return 1;
    if (k.dtype() == torch::kInt8) return 2;
    if (k.dtype() == torch::kUInt8) return 3;
    TORCH_CHECK(k.dtype() == q.dtype(),
                "query and key must have the same dtype (or the key cache is float8_e4m3fn, int8, or uint8 holding "
                "int4 pairs)");
    return 0;
}

const float *scale_ptr(const std::optional<at::Tensor> &t, const at::Tensor &q, int64_t head_k, const char *name,
                       int kv8) {
    if (!t.has_value()) return nullptr;
    TORCH_CHECK(kv8 != 0, name, " applies to a float8_e4m3fn, int8 or int4 K/V cache only");
    const at::Tensor &s = t.value();
    TORCH_CHECK(s.dtype() == torch::kFloat32 && s.is_cuda() && s.device() == q.device() && s.is_contiguous() &&
                    s.numel() == head_k,
                name, " must be a contiguous float32 GPU tensor of head_k values");
    return s.data_ptr<float>();
}

// int4 or int8 with a (scale, zero) pair per (token, KV head): k_scale and v_scale are then tensors shaped like the rows they
// belong to with a last dimension of 2 (`rows` = the leading dimensions of the K tensor) instead of head_k values.
// One dimension more, [..., head_k, dim / 64, 2], is a pair per run of 64 elements of every row.
// Returns 0 (per-head factors), 1 (a pair per row) or 2 (a pair per 64 elements).
int per_token_pairs(const std::optional<at::Tensor> &ks, const std::optional<at::Tensor> &vs, const at::Tensor &q,
                    const at::Tensor &k, int kv8) {
    const int64_t kd = k.dim();
    const auto form = [kd](const std::optional<at::Tensor> &t) {
        return !t.has_value() ? 0 : (t.value().dim() == kd ? 1 : (t.value().dim() == kd + 1 ? 2 : 0));
    };
    const int k_form = form(ks), v_form = form(vs);
    if (k_form == 0 && v_form == 0) return 0;
    TORCH_CHECK(kv8 == 3 || kv8 == 2, "per-token (scale, zero) pairs apply to an int4 or int8 K/V cache only");
    TORCH_CHECK(k_form == v_form, "per-token (scale, zero) pairs must be given for both K and V, in the same form");
    for (const at::Tensor *t : {&ks.value(), &vs.value()}) {
        TORCH_CHECK(t->dtype() == torch::kFloat32 && t->is_cuda() && t->device() == q.device() && t->is_contiguous(),
                    "per-token pairs must be contiguous float32 GPU tensors");
        for (int64_t d = 0; d + 1 < kd; ++d)
            TORCH_CHECK(t->size(d) == k.size(d), "per-token pairs must have the K tensor's leading dimensions");
        if (k_form == 2)
            TORCH_CHECK(t->size(kd - 1) * 64 == q.size(-1), "pairs per 64 elements: [..., head_k, dim / 64, 2]");
        TORCH_CHECK(t->size(-1) == 2, "per-token pairs must have a last dimension of 2 (scale, zero)");
    }
    return k_form;
}

at::Tensor dmha_fwd(const at::Tensor &q, const at::Tensor &k, const std::optional<at::Tensor> &v_,
                    const std::optional<at::Tensor> &o_, const at::Tensor &cu_seq_k, const int64_t max_seq_k,
                    const int64_t dim_v, const bool is_alibi, const std::optional<double> softmax_scale,
                    const std::optional<at::Tensor> &alibi_slopes, const std::optional<at::Tensor> &k_scale,
                    const std::optional<at::Tensor> &v_scale) {
    auto q_dtype = q.dtype();
    TORCH_CHECK(q_dtype == torch::kFloat16 || q_dtype == torch::kBFloat16,
                "Decoding-Attention only support FP16 and BF16 data type");
    const bool is_bf16 = q_dtype == torch::kBFloat16;
    const int kv8 = kv8_format(q, k);  // 0: 16-bit K/V
    const auto kv_dtype = k.dtype();
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
    const int64_t pack = kv8 == 3 ? 2 : 1;  // K/V elements per tensor element
    TORCH_CHECK(dim % pack == 0 && dim_v % pack == 0, "int4 K/V needs even head dims");
    DA_CHECK_SHAPE(k, total_k, head_k, dim / pack);
    DA_CHECK_SHAPE(cu_seq_k, batch + 1);
    DA_CHECK_CONTIGUOUS(q);
    DA_CHECK_CONTIGUOUS(k);
    TORCH_CHECK(total_q == batch, "one query token per sequence: q.size(0) must equal cu_seq_k.numel() - 1");
    TORCH_CHECK(da_supported_head_dims((size_t)dim, (size_t)dim_v) == 1, "unsupported head dims (dim ", dim,
                ", dim_v ", dim_v, "): supported are (64,64) (96,96) (128,128) (256,256) (576,512)");

    const void *v_ptr = nullptr;
    if (v_.has_value()) {
        const at::Tensor &v = v_.value();
        TORCH_CHECK(v.dtype() == kv_dtype, "key and value must have the same dtype");
        DA_CHECK_DEVICE(v);
        TORCH_CHECK(v.device() == q.device(), "v must be on q's device");
        TORCH_CHECK(v.stride(-1) == 1, "value must have contiguous last dimension");
        DA_CHECK_SHAPE(v, total_k, head_k, dim_v / pack);
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

    const int tok = per_token_pairs(k_scale, v_scale, q, k, kv8);
    TORCH_CHECK(!tok || v_ptr != nullptr, "per-token pairs need a V cache of its own");
    const float *k_scale_ptr = tok ? k_scale.value().data_ptr<float>() : scale_ptr(k_scale, q, head_k, "k_scale", kv8);
    const float *v_scale_ptr = tok ? v_scale.value().data_ptr<float>() : scale_ptr(v_scale, q, head_k, "v_scale", kv8);

    // k.size(0) is the sum of the key lengths: a free host-side hint for sizing the sequence splits
    const size_t ws_bytes =
        kv8 ? (tok == 2 ? (kv8 == 3 ? da_workspace_bytes_int4kv_grp64 : da_workspace_bytes_int8kv_grp64)
               : tok ? (kv8 == 3 ? da_workspace_bytes_int4kv_tok : da_workspace_bytes_int8kv_tok)
                   : kv8 == 3 ? da_workspace_bytes_int4kv : da_workspace_bytes_fp8kv)(
                  (size_t)max_seq_k, (size_t)batch, (size_t)head_q, (size_t)head_k, (size_t)dim, (size_t)dim_v,
                  (size_t)total_k, 0)
            : da_workspace_bytes((size_t)max_seq_k, (size_t)batch, (size_t)head_q, (size_t)head_k, (size_t)dim,
                                 (size_t)dim_v, (size_t)total_k);
    at::Tensor ws;  // from torch's stream-aware caching allocator
    if (ws_bytes > 0) ws = torch::empty({(int64_t)ws_bytes}, q.options().dtype(torch::kUInt8));

    const float scale = softmax_scale.has_value() ? (float)softmax_scale.value() : 0.0f;
    const auto kv8_entry = tok == 2   ? (kv8 == 3 ? da_decoding_attn_int4kv_grp64 : da_decoding_attn_int8kv_grp64)
                           : tok      ? (kv8 == 3 ? da_decoding_attn_int4kv_tok : da_decoding_attn_int8kv_tok)
                           : kv8 == 3 ? da_decoding_attn_int4kv
                                      : (kv8 == 2 ? da_decoding_attn_int8kv : da_decoding_attn_fp8kv);
    const int rc =
        kv8 ? kv8_entry(q.data_ptr(), k.data_ptr(), v_ptr, o.data_ptr(), cu_seq_k.data_ptr<int32_t>(),
                        (size_t)max_seq_k, (size_t)batch, (size_t)head_q, (size_t)head_k, (size_t)dim, (size_t)dim_v,
                        is_alibi ? 1 : 0, is_bf16 ? 1 : 0, scale, slopes_ptr, k_scale_ptr, v_scale_ptr,
                        (size_t)total_k, ws_bytes > 0 ? ws.data_ptr() : nullptr, ws_bytes, (void *)stream)
            : da_decoding_attn_ex(q.data_ptr(), k.data_ptr(), v_ptr, o.data_ptr(), cu_seq_k.data_ptr<int32_t>(),
                                  (size_t)max_seq_k, (size_t)batch, (size_t)head_q, (size_t)head_k, (size_t)dim,
                                  (size_t)dim_v, is_alibi ? 1 : 0, is_bf16 ? 1 : 0, scale, slopes_ptr,
                                  (size_t)total_k, ws_bytes > 0 ? ws.data_ptr() : nullptr, ws_bytes, (void *)stream);
    TORCH_CHECK(rc == DA_OK, "decoding_attn failed (", rc, "): ", da_last_error());
    return o;
}

// Paged K/V: k_pages [pages, page_size, head_k, dim] and v_pages [pages, page_size, head_k, dim_v] (or none: the
// values are the first dim_v columns of each K row), dense within a page, any stride between pages (so the two
// halves of a combined [pages, 2, page_size, head_k, dim] pool can be passed as views).
at::Tensor dmha_fwd_paged(const at::Tensor &q, const at::Tensor &k_pages, const std::optional<at::Tensor> &v_pages_,
                          const std::optional<at::Tensor> &o_, const at::Tensor &block_table,
                          const at::Tensor &seq_lens, const int64_t max_seq_k, const int64_t dim_v, const bool is_alibi,
                          const std::optional<double> softmax_scale, const std::optional<at::Tensor> &alibi_slopes,
                          const int64_t total_k, const std::optional<at::Tensor> &k_scale,
                          const std::optional<at::Tensor> &v_scale) {
    auto q_dtype = q.dtype();
    TORCH_CHECK(q_dtype == torch::kFloat16 || q_dtype == torch::kBFloat16,
                "Decoding-Attention only support FP16 and BF16 data type");
    const bool is_bf16 = q_dtype == torch::kBFloat16;
    const int kv8 = kv8_format(q, k_pages);  // 0: 16-bit K/V
    const auto kv_dtype = k_pages.dtype();
    TORCH_CHECK(block_table.dtype() == torch::kInt32, "block_table must have dtype int32");
    TORCH_CHECK(seq_lens.dtype() == torch::kInt32, "seq_lens must have dtype int32");
    DA_CHECK_DEVICE(q);
    DA_CHECK_DEVICE(k_pages);
    DA_CHECK_DEVICE(block_table);
    DA_CHECK_DEVICE(seq_lens);
    TORCH_CHECK(k_pages.device() == q.device() && block_table.device() == q.device() && seq_lens.device() == q.device(),
                "q, k_pages, block_table and seq_lens must share a device");
    TORCH_CHECK(q.dim() == 3, "q must have three dimensions (batch, heads, dim)");
    TORCH_CHECK(k_pages.dim() == 4, "k_pages must have four dimensions (pages, page_size, heads, dim)");
    TORCH_CHECK(block_table.dim() == 2, "block_table must have two dimensions (batch, max_blocks)");
    DA_CHECK_CONTIGUOUS(q);
    DA_CHECK_CONTIGUOUS(block_table);
    DA_CHECK_CONTIGUOUS(seq_lens);

    const int64_t batch = q.size(0), head_q = q.size(1), dim = q.size(2);
    const int64_t page_size = k_pages.size(1), head_k = k_pages.size(2);
    TORCH_CHECK(batch > 0, "batch size must be positive");
    const int64_t pack = kv8 == 3 ? 2 : 1;  // K/V elements per tensor element
    TORCH_CHECK(dim % pack == 0 && dim_v % pack == 0, "int4 K/V needs even head dims");
    TORCH_CHECK(k_pages.size(3) * pack == dim, "k_pages must have q's head dim");
    TORCH_CHECK(head_q % head_k == 0, "number of heads in key/value must divide number of heads in query");
    DA_CHECK_SHAPE(seq_lens, batch);
    TORCH_CHECK(block_table.size(0) == batch, "block_table must have one row per sequence");
    TORCH_CHECK(da_supported_head_dims((size_t)dim, (size_t)dim_v) == 1, "unsupported head dims (dim ", dim,
                ", dim_v ", dim_v, "): supported are (64,64) (96,96) (128,128) (256,256) (576,512)");
    auto page_dense = [](const at::Tensor &t) {
        return t.stride(3) == 1 && t.stride(2) == t.size(3) && t.stride(1) == t.size(2) * t.size(3);
    };
    TORCH_CHECK(page_dense(k_pages), "k_pages must be dense within a page");

    const void *v_ptr = nullptr;
    int64_t v_stride = 0;
    if (v_pages_.has_value()) {
        const at::Tensor &v = v_pages_.value();
        TORCH_CHECK(v.dtype() == kv_dtype, "key and value must have the same dtype");
        DA_CHECK_DEVICE(v);
        TORCH_CHECK(v.device() == q.device(), "v_pages must be on q's device");
        TORCH_CHECK(v.dim() == 4 && v.size(0) == k_pages.size(0) && v.size(1) == page_size && v.size(2) == head_k &&
                        v.size(3) * pack == dim_v,
                    "v_pages must have shape (pages, page_size, head_k, dim_v)");
        TORCH_CHECK(page_dense(v), "v_pages must be dense within a page");
        v_ptr = v.data_ptr();
        v_stride = v.stride(0) * pack;  // (the C-ABI counts page strides in K/V elements)
    } else {
        TORCH_CHECK(dim_v <= dim, "without v the values are the first dim_v columns of k: dim_v must not exceed dim");
    }

    at::Tensor o;
    if (o_.has_value()) {
        o = o_.value();
        TORCH_CHECK(o.dtype() == q_dtype, "Output must have the same dtype as inputs");
        DA_CHECK_DEVICE(o);
        TORCH_CHECK(o.device() == q.device(), "o must be on q's device");
        DA_CHECK_SHAPE(o, batch, head_q, dim_v);
        DA_CHECK_CONTIGUOUS(o);
    } else {
        o = torch::empty({batch, head_q, dim_v}, q.options());
    }

    const float *slopes_ptr = nullptr;
    if (alibi_slopes.has_value()) {
        const at::Tensor &s = alibi_slopes.value();
        TORCH_CHECK(s.dtype() == torch::kFloat32 && s.is_cuda() && s.device() == q.device() && s.is_contiguous() &&
                        s.numel() == head_q,
                    "alibi_slopes must be a contiguous float32 GPU tensor of head_q values");
        slopes_ptr = s.data_ptr<float>();
    }

    c10::hip::HIPGuardMasqueradingAsCUDA guard(q.device());
    hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(q.device().index()).stream();

    const int tok = per_token_pairs(k_scale, v_scale, q, k_pages, kv8);
    TORCH_CHECK(!tok || v_ptr != nullptr, "per-token pairs need a V cache of its own");
    const float *k_scale_ptr = tok ? k_scale.value().data_ptr<float>() : scale_ptr(k_scale, q, head_k, "k_scale", kv8);
    const float *v_scale_ptr = tok ? v_scale.value().data_ptr<float>() : scale_ptr(v_scale, q, head_k, "v_scale", kv8);
    const size_t hint = total_k > 0 ? (size_t)total_k : 0;
    const size_t ws_bytes =
        kv8 ? (tok == 2 ? (kv8 == 3 ? da_workspace_bytes_int4kv_grp64 : da_workspace_bytes_int8kv_grp64)
               : tok ? (kv8 == 3 ? da_workspace_bytes_int4kv_tok : da_workspace_bytes_int8kv_tok)
                   : kv8 == 3 ? da_workspace_bytes_int4kv : da_workspace_bytes_fp8kv)(
                  (size_t)max_seq_k, (size_t)batch, (size_t)head_q, (size_t)head_k, (size_t)dim, (size_t)dim_v, hint,
                  (size_t)page_size)
            : da_workspace_bytes_paged((size_t)max_seq_k, (size_t)batch, (size_t)head_q, (size_t)head_k, (size_t)dim,
                                       (size_t)dim_v, hint, (size_t)page_size);
    at::Tensor ws;
    if (ws_bytes > 0) ws = torch::empty({(int64_t)ws_bytes}, q.options().dtype(torch::kUInt8));

    const float scale = softmax_scale.has_value() ? (float)softmax_scale.value() : 0.0f;
    const auto kv8_entry = tok == 2   ? (kv8 == 3 ? da_decoding_attn_paged_int4kv_grp64 : da_decoding_attn_paged_int8kv_grp64)
                           : tok      ? (kv8 == 3 ? da_decoding_attn_paged_int4kv_tok : da_decoding_attn_paged_int8kv_tok)
                           : kv8 == 3 ? da_decoding_attn_paged_int4kv
                                      : (kv8 == 2 ? da_decoding_attn_paged_int8kv : da_decoding_attn_paged_fp8kv);
    const int rc =
        kv8 ? kv8_entry(
                  q.data_ptr(), k_pages.data_ptr(), v_ptr, o.data_ptr(), block_table.data_ptr<int32_t>(),
                  seq_lens.data_ptr<int32_t>(), (size_t)max_seq_k, (size_t)batch, (size_t)head_q, (size_t)head_k,
                  (size_t)dim, (size_t)dim_v, (size_t)page_size, (size_t)block_table.size(1),
                  (size_t)(k_pages.stride(0) * pack), (size_t)v_stride, is_alibi ? 1 : 0, is_bf16 ? 1 : 0, scale,
                  slopes_ptr, k_scale_ptr, v_scale_ptr, hint, ws_bytes > 0 ? ws.data_ptr() : nullptr, ws_bytes, (void *)stream)
            : da_decoding_attn_paged(
                  q.data_ptr(), k_pages.data_ptr(), v_ptr, o.data_ptr(), block_table.data_ptr<int32_t>(),
                  seq_lens.data_ptr<int32_t>(), (size_t)max_seq_k, (size_t)batch, (size_t)head_q, (size_t)head_k,
                  (size_t)dim, (size_t)dim_v, (size_t)page_size, (size_t)block_table.size(1),
                  (size_t)k_pages.stride(0), (size_t)v_stride, is_alibi ? 1 : 0, is_bf16 ? 1 : 0, scale, slopes_ptr,
                  hint, ws_bytes > 0 ? ws.data_ptr() : nullptr, ws_bytes, (void *)stream);
    TORCH_CHECK(rc == DA_OK, "decoding_attn (paged) failed (", rc, "): ", da_last_error());
    return o;
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.doc() = "Decoding-Attention for MI355X (gfx950)";
    m.def("fwd", &dmha_fwd, "Forward pass", pybind11::arg("q"), pybind11::arg("k"), pybind11::arg("v_"),
          pybind11::arg("o_"), pybind11::arg("cu_seq_k"), pybind11::arg("max_seq_k"), pybind11::arg("dim_v"),
          pybind11::arg("is_alibi"), pybind11::arg("softmax_scale") = pybind11::none(),
          pybind11::arg("alibi_slopes") = pybind11::none(), pybind11::arg("k_scale") = pybind11::none(),
          pybind11::arg("v_scale") = pybind11::none());
    m.def("fwd_paged", &dmha_fwd_paged, "Forward pass over a paged K/V cache", pybind11::arg("q"),
          pybind11::arg("k_pages"), pybind11::arg("v_pages_"), pybind11::arg("o_"), pybind11::arg("block_table"),
          pybind11::arg("seq_lens"), pybind11::arg("max_seq_k"), pybind11::arg("dim_v"), pybind11::arg("is_alibi"),
          pybind11::arg("softmax_scale") = pybind11::none(), pybind11::arg("alibi_slopes") = pybind11::none(),
          pybind11::arg("total_k") = 0, pybind11::arg("k_scale") = pybind11::none(),
          pybind11::arg("v_scale") = pybind11::none());
}
