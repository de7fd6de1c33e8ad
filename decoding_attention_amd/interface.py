"""Python face of the decoding-attention op: the reference's `decoding_attn_fwd` over the PyTorch-ROCm
extension module `decoding_attn_hip`, which checks the tensors and calls the C-ABI of libdecoding_attn_hip.so.

`decoding_attn_fwd` keeps the reference's positional signature and return value
(reference decoding_attn/decoding_attn_interface.py:24-53).  `fwd` is the extension function itself; it keeps
the argument list, check order and error type (RuntimeError) of the reference's pybind function `dmha_fwd`
(reference csrc/torch/decoding_torch.cpp:19-80).

There is no fallback: if the extension or the library is not built the import fails with the build command.
"""
import importlib
import os
from typing import Optional

import torch

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
_ext = None


def _extension():
    """The compiled extension module (loaded once)."""
    global _ext
    if _ext is None:
        try:
            _ext = importlib.import_module("decoding_attention_amd.decoding_attn_hip")
        except ImportError as e:
            raise ImportError(
                "the PyTorch-ROCm extension decoding_attention_amd/decoding_attn_hip*.so is not built: run "
                "`python -m decoding_attention_amd.build` and `python -m decoding_attention_amd.build_torch_ext` "
                f"(there is no CPU or pure-PyTorch fallback): {e}") from e
    return _ext


def maybe_contiguous(x):
    """Make the tensor dense.  The reference only fixes tensors whose last stride is not 1
    (decoding_attn_interface.py:20-21) and then mis-reads other strided views; here any
    non-contiguous input is copied."""
    return x.contiguous() if x is not None and not x.is_contiguous() else x


def is_leading_columns_view(v, k) -> bool:
    """True when v is a view of k's own memory that selects the leading columns of every row, as
    `k[..., :dim_v]` does: the values are then read out of the K rows (v = None), which is what the latent form's
    fast kernels need, instead of from a copy."""
    # (the address comparison first: it settles the ordinary case, a V buffer of its own, at once)
    return (v is not None and v.data_ptr() == k.data_ptr() and v.dtype == k.dtype and v.device == k.device and
            v.dim() == k.dim() and v.shape[:-1] == k.shape[:-1] and v.shape[-1] <= k.shape[-1] and
            v.stride() == k.stride())


def fwd(q: torch.Tensor, k: torch.Tensor, v_: Optional[torch.Tensor], o_: Optional[torch.Tensor],
        cu_seq_k: torch.Tensor, max_seq_k: int, dim_v: int, is_alibi: bool, *,
        softmax_scale: Optional[float] = None, alibi_slopes: Optional[torch.Tensor] = None,
        k_scale: Optional[torch.Tensor] = None, v_scale: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The extension's `fwd` (same role as the reference's `decoding_attn_cuda.fwd`)."""
    return _extension().fwd(q, k, v_, o_, cu_seq_k, int(max_seq_k), int(dim_v), bool(is_alibi),
                            None if softmax_scale is None else float(softmax_scale), alibi_slopes, k_scale, v_scale)


def pack_int4(x: torch.Tensor) -> torch.Tensor:
    """Integers in -8 .. 7 (any integer dtype, last dimension even) -> the int4 K/V cache layout: torch.uint8 with
    half the last dimension, element 2 i in the low half of byte i, two's complement."""
    if x.shape[-1] % 2 != 0:
        raise ValueError("the last dimension must be even")
    n = x.to(torch.int16) & 0xF
    return (n[..., 0::2] | (n[..., 1::2] << 4)).to(torch.uint8)


def quantize_int4_per_token(x: torch.Tensor):
    """Asymmetric int4 quantisation with one (scale, zero) pair per row of the last dimension (per token and KV head):
    returns (packed, pairs) with x ~= pairs[..., 0] * (n - pairs[..., 1]), n the integers -8 .. 7 stored in `packed`
    (pack_int4's layout), pairs float32 [..., 2].  The row's minimum maps to -8 and its maximum to 7."""
    xf = x.float()
    lo, hi = xf.amin(dim=-1, keepdim=True), xf.amax(dim=-1, keepdim=True)
    scale = ((hi - lo) / 15.0).clamp_min(1e-8)
    zero = -8.0 - lo / scale
    n = torch.round(xf / scale + zero).clamp(-8, 7).to(torch.int8)
    return pack_int4(n), torch.cat([scale, zero], dim=-1).contiguous()


def quantize_int4_per_group(x: torch.Tensor, group: int = 64):
    """Asymmetric int4 quantisation with one (scale, zero) pair per run of `group` (= 64) elements of the last
    dimension: returns (packed, pairs) with x[..., c] ~= pairs[..., c // 64, 0] * (n[..., c] - pairs[..., c // 64, 1]),
    `packed` in pack_int4's layout, pairs float32 [..., dim / 64, 2]."""
    if group != 64 or x.shape[-1] % 64 != 0:
        raise ValueError("groups of 64 elements, last dimension a multiple of 64")
    xf = x.float().unflatten(-1, (x.shape[-1] // 64, 64))
    lo, hi = xf.amin(dim=-1, keepdim=True), xf.amax(dim=-1, keepdim=True)
    scale = ((hi - lo) / 15.0).clamp_min(1e-8)
    zero = -8.0 - lo / scale
    n = torch.round(xf / scale + zero).clamp(-8, 7).to(torch.int8)
    return pack_int4(n.flatten(-2)), torch.cat([scale, zero], dim=-1).contiguous()


def quantize_int8_per_group(x: torch.Tensor, group: int = 64):
    """The same with eight bits: returns (torch.int8 tensor, pairs [..., dim / 64, 2]), each run's minimum at -128 and
    its maximum at 127."""
    if group != 64 or x.shape[-1] % 64 != 0:
        raise ValueError("groups of 64 elements, last dimension a multiple of 64")
    xf = x.float().unflatten(-1, (x.shape[-1] // 64, 64))
    lo, hi = xf.amin(dim=-1, keepdim=True), xf.amax(dim=-1, keepdim=True)
    scale = ((hi - lo) / 255.0).clamp_min(1e-8)
    zero = -128.0 - lo / scale
    n = torch.round(xf / scale + zero).clamp(-128, 127).to(torch.int8)
    return n.flatten(-2), torch.cat([scale, zero], dim=-1).contiguous()


def quantize_int8_per_token(x: torch.Tensor):
    """The same with eight bits: returns (torch.int8 tensor, pairs) with x ~= pairs[..., 0] * (n - pairs[..., 1]), the
    row's minimum at -128 and its maximum at 127."""
    xf = x.float()
    lo, hi = xf.amin(dim=-1, keepdim=True), xf.amax(dim=-1, keepdim=True)
    scale = ((hi - lo) / 255.0).clamp_min(1e-8)
    zero = -128.0 - lo / scale
    n = torch.round(xf / scale + zero).clamp(-128, 127).to(torch.int8)
    return n, torch.cat([scale, zero], dim=-1).contiguous()


def decoding_attn_fwd(q: torch.Tensor, k: torch.Tensor, v: Optional[torch.Tensor], cu_seq_k: torch.Tensor,
                      max_seq_k: int, dim_v: int, is_alibi: bool, *, softmax_scale: Optional[float] = None,
                      alibi_slopes: Optional[torch.Tensor] = None, k_scale: Optional[torch.Tensor] = None,
                      v_scale: Optional[torch.Tensor] = None) -> torch.Tensor:
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
        k_scale, v_scale (keyword only): k and v may be torch.float8_e4m3fn or torch.int8 (an 8-bit K/V cache; q
            stays 16-bit), or torch.uint8 holding pairs of int4 values (see pack_int4: last dimensions dim / 2 and
            dim_v / 2); these are then float32 [head_k] GPU tensors of de-quantisation factors (default 1):
            K = k_scale * k.  For an int4 or int8 cache they may instead be float32 [total_k, head_k, 2] tensors of
            (scale, zero) pairs, one per token and KV head (quantize_int4_per_token, quantize_int8_per_token):
            K[t, h] = k_scale[t, h, 0] * (k[t, h] - k_scale[t, h, 1]); head dims 64, 128 and 256, v required.
            float32 [total_k, head_k, dim / 64, 2] gives every run of 64 elements of a row its own pair
            (quantize_int4_per_group, quantize_int8_per_group).
    Return:
        o: [total_q, head_q, dim_v], same dtype as q.
    """
    if is_leading_columns_view(v, k) and v.shape[-1] == dim_v:
        v = None  # (the reference's callers pass None themselves: tests/test_decoding_attn.py:45 builds this view)
    q, k, v = [maybe_contiguous(x) for x in (q, k, v)]
    return fwd(q, k, v, None, cu_seq_k, max_seq_k, dim_v, is_alibi, softmax_scale=softmax_scale,
               alibi_slopes=alibi_slopes, k_scale=k_scale, v_scale=v_scale)


def decoding_attn_paged_fwd(q: torch.Tensor, k_pages: torch.Tensor, v_pages: Optional[torch.Tensor],
                            block_table: torch.Tensor, seq_lens: torch.Tensor, max_seq_k: int, dim_v: int,
                            is_alibi: bool, *, softmax_scale: Optional[float] = None,
                            alibi_slopes: Optional[torch.Tensor] = None, total_k: int = 0,
                            out: Optional[torch.Tensor] = None, k_scale: Optional[torch.Tensor] = None,
                            v_scale: Optional[torch.Tensor] = None) -> torch.Tensor:
    """
    The same attention over a paged K/V cache (no counterpart in the reference; the layouts are those of the
    libraries its benchmark compares against, reference benchmarks/python/benchmark_decoding_attn.py:129-151,182-187).

    Arguments:
        q: [batch, head_q, dim], torch.float16 / torch.bfloat16; one query token per sequence.
        k_pages: [pages, page_size, head_k, dim] page pool, dense within a page (any stride between pages).
        v_pages: [pages, page_size, head_k, dim_v] or None for MLA (values are k_pages[..., :dim_v]).
        block_table: [batch, max_blocks], torch.int32 page ids of each sequence in token order.
        seq_lens: [batch], torch.int32 key tokens of each sequence.
        max_seq_k: upper bound of seq_lens (a host integer: nothing here synchronises with the device).
        page_size (from k_pages.shape[1]) must be a power of two.
        total_k (keyword only): sum of seq_lens if the host knows it; only a hint for sizing sequence splits.
        k_scale, v_scale (keyword only): as for decoding_attn_fwd, when the pools are torch.float8_e4m3fn, torch.int8
            or torch.uint8 holding pairs of int4 values (last dimensions dim / 2 and dim_v / 2); per-token
            (scale, zero) pairs of an int4 or int8 cache are float32 [pages, page_size, head_k, 2], pairs per 64
            elements [pages, page_size, head_k, dim / 64, 2].
    Return:
        o: [batch, head_q, dim_v], same dtype as q.
    """
    q = maybe_contiguous(q)
    if is_leading_columns_view(v_pages, k_pages) and v_pages.shape[-1] == dim_v:
        v_pages = None
    return _extension().fwd_paged(q, k_pages, v_pages, out, block_table, seq_lens, int(max_seq_k), int(dim_v),
                                  bool(is_alibi), None if softmax_scale is None else float(softmax_scale),
                                  alibi_slopes, int(total_k), k_scale, v_scale)
