"""TEST INFRASTRUCTURE — Python face of the CPU oracle.

Only tests/, the smoke check and the benchmark's cpu_baseline leg may import this
module; the product package never does and has no CPU fallback.

Two independent statements of the same mathematics live here:

* ``attn_cpu``      — ctypes call into ``liboracle_attn.so`` (oracle/attn_cpu.c), the
  from-scratch restatement of the reference's ``Tester<T>::attn_cpu``
  (reference csrc/common/tester.h:133-259): fp32 accumulation in loop order,
  normalise-then-PV, RNE output cast.
* ``attn_f64``      — textbook ``softmax(q k^T * scale + bias) v`` per (sequence, head)
  in float64 numpy, following the tensor-level recipe of the reference's pytest
  oracle ``torch_attn`` (reference tests/test_decoding_attn.py:35-57: GQA by
  repeating KV heads, ``/sqrt(dim)``, softmax over keys, MLA ``v = k[..., :dim_v]``).
  It is what the tolerance "against an fp32-accumulated result" is checked with and
  it pins ``attn_cpu`` itself.
"""
import ctypes
import math
import os
import subprocess

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle_attn.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile oracle/attn_cpu.c with the committed Makefile."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.check_call(["make", "-s", "-C", _HERE, "liboracle_attn.so"])
    return _LIB_PATH


def _load():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        lib = ctypes.CDLL(_LIB_PATH)
        lib.oracle_attn_cpu.restype = ctypes.c_int
        lib.oracle_attn_cpu.argtypes = [
            ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
            ctypes.c_size_t, ctypes.c_size_t, ctypes.c_size_t, ctypes.c_size_t, ctypes.c_size_t, ctypes.c_size_t,
            ctypes.c_int, ctypes.c_int, ctypes.c_float, ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p,
        ]
        lib.oracle_f32_to_f16.restype = ctypes.c_uint16
        lib.oracle_f32_to_f16.argtypes = [ctypes.c_float]
        lib.oracle_f32_to_bf16.restype = ctypes.c_uint16
        lib.oracle_f32_to_bf16.argtypes = [ctypes.c_float]
        lib.oracle_f16_to_f32.restype = ctypes.c_float
        lib.oracle_f16_to_f32.argtypes = [ctypes.c_uint16]
        lib.oracle_bf16_to_f32.restype = ctypes.c_float
        lib.oracle_bf16_to_f32.argtypes = [ctypes.c_uint16]
        lib.oracle_max_threads.restype = ctypes.c_int
        _lib = lib
    return _lib


def max_threads() -> int:
    return int(_load().oracle_max_threads())


def f32_to_f16_bits(x: float) -> int:
    return int(_load().oracle_f32_to_f16(x))


def f32_to_bf16_bits(x: float) -> int:
    return int(_load().oracle_f32_to_bf16(x))


def f16_bits_to_f32(h: int) -> float:
    return float(_load().oracle_f16_to_f32(h))


def bf16_bits_to_f32(h: int) -> float:
    return float(_load().oracle_bf16_to_f32(h))


def default_slopes(head_q: int) -> np.ndarray:
    """ALiBi slopes of the reference: 1/exp2(8(h+1)/head_q) (csrc/common/tester.h:193)."""
    return np.array([1.0 / 2.0 ** (8.0 * (h + 1) / head_q) for h in range(head_q)], dtype=np.float32)


def attn_cpu(q, k, v, cu_seq_k, max_seq_k, dim_v, is_alibi, softmax_scale=None, alibi_slopes=None, nthreads=1,
             return_f32=False):
    """q [batch, Hq, d], k [total_k, Hk, d], v [total_k, Hk, dv] or None; CPU fp16/bf16 tensors.

    Returns o [batch, Hq, dv] in q's dtype (and the un-rounded fp32 result if asked).
    """
    lib = _load()
    assert q.device.type == "cpu" and q.dtype in (torch.float16, torch.bfloat16)
    q = q.contiguous()
    k = k.contiguous()
    v = v.contiguous() if v is not None else None
    cu = cu_seq_k.to(device="cpu", dtype=torch.int32).contiguous()
    batch = cu.numel() - 1
    head_q, dim = q.shape[1], q.shape[2]
    head_k = k.shape[1]
    o = torch.empty(q.shape[0], head_q, dim_v, dtype=q.dtype)
    o32 = torch.empty(q.shape[0], head_q, dim_v, dtype=torch.float32) if return_f32 else None
    slopes = None
    if alibi_slopes is not None:
        slopes = torch.as_tensor(alibi_slopes, dtype=torch.float32).contiguous()
    rc = lib.oracle_attn_cpu(
        q.data_ptr(), k.data_ptr(), v.data_ptr() if v is not None else None, o.data_ptr(), cu.data_ptr(),
        int(max_seq_k), batch, head_q, head_k, dim, int(dim_v), int(bool(is_alibi)),
        int(q.dtype == torch.bfloat16), float(softmax_scale) if softmax_scale else 0.0,
        slopes.data_ptr() if slopes is not None else None, int(nthreads),
        o32.data_ptr() if o32 is not None else None)
    if rc != 0:
        raise ValueError(f"oracle_attn_cpu rejected its arguments (code {rc})")
    return (o, o32) if return_f32 else o


def attn_f64(q, k, v, cu_seq_k, dim_v, is_alibi, softmax_scale=None, alibi_slopes=None):
    """Float64 textbook attention on the packed layout; returns float64 numpy [batch, Hq, dv]."""
    qn = q.to(torch.float64).numpy()
    kn = k.to(torch.float64).numpy()
    vn = v.to(torch.float64).numpy() if v is not None else kn[..., :dim_v]
    cu = np.asarray(cu_seq_k.cpu().numpy() if torch.is_tensor(cu_seq_k) else cu_seq_k, dtype=np.int64)
    batch = cu.shape[0] - 1
    head_q, dim = qn.shape[1], qn.shape[2]
    head_k = kn.shape[1]
    ratio = head_q // head_k
    scale = float(softmax_scale) if softmax_scale else 1.0 / math.sqrt(dim)
    if alibi_slopes is None:
        slopes = default_slopes(head_q).astype(np.float64)
    else:
        slopes = np.asarray(alibi_slopes, dtype=np.float64)
    out = np.zeros((batch, head_q, dim_v), dtype=np.float64)
    for b in range(batch):
        s0, s1 = int(cu[b]), int(cu[b + 1])
        n = s1 - s0
        if n <= 0:
            continue
        kb = np.repeat(kn[s0:s1], ratio, axis=1)  # [n, Hq, d]
        vb = np.repeat(vn[s0:s1], ratio, axis=1)  # [n, Hq, dv]
        s = np.einsum("hd,nhd->hn", qn[b], kb) * scale
        if is_alibi:
            s = s + slopes[:, None] * (np.arange(n, dtype=np.float64)[None, :] - (n - 1))
        s = s - s.max(axis=1, keepdims=True)
        p = np.exp(s)
        p /= p.sum(axis=1, keepdims=True)
        out[b] = np.einsum("hn,nhd->hd", p, vb)
    return out
