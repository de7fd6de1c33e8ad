"""Writes the small golden fixtures next to this file.

The reference repository holds no golden vectors (its tests draw unseeded random inputs), so these are the
build's own: seeded inputs as raw 16-bit patterns, the CPU oracle's output bits, and the float64 textbook
result that the oracle output was checked against when the fixture was written.

Usage (from the repository root): python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

from decoding_attention_amd import workloads as wl  # noqa: E402
from oracle import oracle  # noqa: E402

CASES = {
    # name: (lens, head_q, head_k, dim, dim_v, dtype, is_alibi)
    "gqa_fp16_d64": ([3, 5], 4, 2, 64, 64, torch.float16, False),
    "gqa_bf16_d128": ([1, 40, 17], 8, 2, 128, 128, torch.bfloat16, False),
    "mqa_alibi_fp16_d128": ([7, 33], 8, 1, 128, 128, torch.float16, True),
    "mha_bf16_d96_with_empty": ([0, 9, 2], 2, 2, 96, 96, torch.bfloat16, False),
    "mla_fp16": ([5, 9], 16, 1, 576, 512, torch.float16, False),
    "mla_bf16_alibi": ([12], 32, 1, 576, 512, torch.bfloat16, True),
}


def build_case(name, spec, seed):
    lens, hq, hk, d, dv, dtype, alibi = spec
    g = torch.Generator().manual_seed(seed)
    lens_t = torch.tensor(lens, dtype=torch.int32)
    total = int(lens_t.sum())
    q = torch.randn(len(lens), hq, d, generator=g).to(dtype)
    k = torch.randn(total, hk, d, generator=g).to(dtype)
    v = None if d != dv else torch.randn(total, hk, dv, generator=g).to(dtype)
    cu = wl.get_cu_seq(lens_t)
    o, o32 = oracle.attn_cpu(q, k, v, cu, max(lens), dv, alibi, return_f32=True)
    ref = oracle.attn_f64(q, k, v, cu, dv, alibi)
    assert np.abs(o32.numpy() - ref).max() < 2e-5, name
    out = {
        "q": q.view(torch.int16).numpy(), "k": k.view(torch.int16).numpy(), "cu_seq_k": cu.numpy(),
        "o": o.view(torch.int16).numpy(), "o_f64": ref, "is_bf16": np.array(dtype == torch.bfloat16),
        "is_alibi": np.array(alibi), "dim_v": np.array(dv),
    }
    if v is not None:
        out["v"] = v.view(torch.int16).numpy()
    return out


def main():
    for i, (name, spec) in enumerate(CASES.items()):
        np.savez_compressed(os.path.join(HERE, name + ".npz"), **build_case(name, spec, 1000 + i))
        print("wrote", name)


if __name__ == "__main__":
    main()
