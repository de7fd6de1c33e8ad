"""Python face of the decoding-attention op: the reference's `decoding_attn_fwd` and the checks of its
extension function `fwd`, over the C-ABI of libdecoding_attn_hip.so.

`decoding_attn_fwd` keeps the reference's positional signature and return value
(reference decoding_attn/decoding_attn_interface.py:24-53).  `fwd` keeps the argument list, check order and
error type (RuntimeError) of the reference's pybind function `dmha_fwd`
(reference csrc/torch/decoding_torch.cpp:19-80) and adds the checks that function leaves out:
full contiguity (it derives strides from head counts, so a sliced tensor would be mis-read),
total_q == batch (one query token per sequence), supported (dim, dim_v), 16-byte alignment, and a
device guard on q's device.
"""
import math
from typing import Optional

import torch

from . import _lib


def maybe_contiguous(x):
    """Make the tensor dense.  The reference only fixes tensors whose last stride is not 1
    (decoding_attn_interface.py:20-21) and then mis-reads other strided views; here any
    non-contiguous input is copied."""
    return x.contiguous() if x is not None and not x.is_contiguous() else x


def _check(cond, msg):
    if not cond:
        raise RuntimeError(msg)


def fwd(q: torch.Tensor, k: torch.Tensor, v_: Optional[torch.Tensor], o_: Optional[torch.Tensor],
        cu_seq_k: torch.Tensor, max_seq_k: int, dim_v: int, is_alibi: bool, *,
        softmax_scale: Optional[float] = None, alibi_slopes: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Validated launch.  Same checks, in the same order, as reference csrc/torch/decoding_torch.cpp:24-74."""
    lib = _lib.load()
    q_dtype = q.dtype
    _check(q_dtype in (torch.float16, torch.bfloat16), "Decoding-Attention only support FP16 and BF16 data type")
    is_bf16 = q_dtype == torch.bfloat16
    _check(k.dtype == q_dtype, "query and key must have the same dtype")
    _check(cu_seq_k.dtype == torch.int32, "cu_seq_k must have dtype int32")

    _check(q.is_cuda, "q must be on the GPU")
    _check(k.is_cuda, "k must be on the GPU")
    _check(cu_seq_k.is_cuda, "cu_seq_k must be on the GPU")
    _check(k.device == q.device and cu_seq_k.device == q.device, "q, k and cu_seq_k must be on the same device")

    _check(q.dim() == 3 and k.dim() == 3, "q and k must have three dimensions (tokens, heads, dim)")
    _check(q.stride(-1) == 1, "query must have contiguous last dimension")
    _check(k.stride(-1) == 1, "key must have contiguous last dimension")
    _check(cu_seq_k.is_contiguous(), "cu_seq_k must be contiguous")

    batch = cu_seq_k.numel() - 1
    total_q, head_q, dim = q.shape
    total_k, head_k, dim_k = k.shape
    _check(batch > 0, "batch size must be positive")
    _check(dim <= 576, "dim should be at most 576")
    _check(dim_v <= 512, "dim_v should be at most 512")
    _check(head_q % head_k == 0, "number of heads in key/value must divide number of heads in query")

    _check(dim_k == dim, "q and k must have the same head dimension")
    _check(cu_seq_k.dim() == 1, "cu_seq_k must have shape (batch + 1)")
    # beyond the reference: strides are derived from head counts, so the data must be dense
    _check(q.is_contiguous(), "query must be contiguous")
    _check(k.is_contiguous(), "key must be contiguous")
    _check(total_q == batch, "one query token per sequence: q.shape[0] must equal cu_seq_k.numel() - 1")
    _check(bool(lib.da_supported_head_dims(dim, dim_v)),
           f"unsupported head dims (dim {dim}, dim_v {dim_v}): supported are (64,64) (96,96) (128,128) "
           "(256,256) (576,512)")

    v_ptr = None
    if v_ is not None:
        v = v_
        _check(v.dtype == q_dtype, "query and value must have the same dtype")
        _check(v.is_cuda and v.device == q.device, "v must be on the same GPU as q")
        _check(v.stride(-1) == 1, "value must have contiguous last dimension")
        _check(tuple(v.shape) == (total_k, head_k, dim_v), "v must have shape (total_k, head_k, dim_v)")
        _check(v.is_contiguous(), "value must be contiguous")
        v_ptr = v.data_ptr()
    else:
        _check(dim_v <= dim, "without v the values are the first dim_v columns of k: dim_v must not exceed dim")

    if o_ is not None:
        o = o_
        _check(o.dtype == q_dtype, "Output must have the same dtype as inputs")
        _check(o.is_cuda and o.device == q.device, "o must be on the same GPU as q")
        _check(o.stride(-1) == 1, "Output tensor must have contiguous last dimension")
        _check(tuple(o.shape) == (total_q, head_q, dim_v), "o must have shape (total_q, head_q, dim_v)")
        _check(o.is_contiguous(), "Output tensor must be contiguous")
    else:
        o = torch.empty((total_q, head_q, dim_v), dtype=q_dtype, device=q.device)

    slopes_ptr = None
    if alibi_slopes is not None:
        _check(alibi_slopes.dtype == torch.float32 and alibi_slopes.is_cuda and alibi_slopes.is_contiguous()
               and alibi_slopes.numel() == head_q, "alibi_slopes must be a contiguous float32 GPU tensor of head_q values")
        slopes_ptr = alibi_slopes.data_ptr()

    with torch.cuda.device(q.device):
        stream = torch.cuda.current_stream().cuda_stream
        ws_bytes = int(lib.da_workspace_bytes(int(max_seq_k), batch, head_q, head_k, dim, int(dim_v)))
        ws = None
        if ws_bytes:
            # torch's caching allocator is stream-aware, so the partials of back-to-back calls never alias
            ws = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device)
        rc = lib.da_decoding_attn_ex(
            q.data_ptr(), k.data_ptr(), v_ptr, o.data_ptr(), cu_seq_k.data_ptr(), int(max_seq_k), batch, head_q,
            head_k, dim, int(dim_v), int(bool(is_alibi)), int(is_bf16),
            float(softmax_scale) if softmax_scale else 0.0, slopes_ptr,
            ws.data_ptr() if ws is not None else None, ws_bytes, stream)
    _check(rc == _lib.DA_OK, f"decoding_attn failed ({rc}): {_lib.last_error()}")
    return o


def decoding_attn_fwd(q: torch.Tensor, k: torch.Tensor, v: Optional[torch.Tensor], cu_seq_k: torch.Tensor,
                      max_seq_k: int, dim_v: int, is_alibi: bool, *, softmax_scale: Optional[float] = None,
                      alibi_slopes: Optional[torch.Tensor] = None) -> torch.Tensor:
    """
    Arguments:
        q: [total_q, head_q, dim], torch.float16 / torch.bfloat16; one query token per sequence.
        k: [total_k, head_k, dim], same dtype; for MLA the packed latent cache (kv_c and k_pe).
        v: [total_k, head_k, dim_v], same dtype; None for MLA (values are k[..., :dim_v]).
        cu_seq_k: [batch + 1], torch.int32 cumulative key lengths, used to index into k / v.
        max_seq_k: maximum key sequence length in the batch.
        dim_v: head dimension of v.
        is_alibi: whether to add the ALiBi bias slope_h * (j - (len - 1)).
        softmax_scale (keyword only): defaults to 1/sqrt(dim) as in the reference.
        alibi_slopes (keyword only): float32 [head_q] on the GPU; defaults to 2^(-8(h+1)/head_q).
    Return:
        o: [total_q, head_q, dim_v], same dtype as q.
    """
    q, k, v = [maybe_contiguous(x) for x in (q, k, v)]
    return fwd(q, k, v, None, cu_seq_k, max_seq_k, dim_v, is_alibi, softmax_scale=softmax_scale,
               alibi_slopes=alibi_slopes)


def default_softmax_scale(dim: int) -> float:
    return 1.0 / math.sqrt(dim)
