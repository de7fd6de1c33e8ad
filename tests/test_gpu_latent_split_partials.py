"""Sequence splits of the pipelined (576, 512) kernel: each split's partial output is stored as it lies in the matrix
instruction's registers (blocks of 32 heads) and the merge kernel reads that order back.  The shapes below put every
form of the merge (one lane per element; 2, 4 and 8 lanes sharing an element's splits) on head counts that fill their
last block of 32 partly (100, 65, 96, 129 heads per KV head) and on one and two KV heads, with ragged lengths so that
sequences differ in their number of live splits.

Tolerances as in test_gpu_parity.py (max-abs 2e-3 fp16 / 1e-2 bf16 against the fp32-accumulated oracle).
"""
import pytest
import torch

from decoding_attention_amd import _lib
from decoding_attention_amd import workloads as wl
from gpu_util import TOL, check_against_oracle, run_hip, run_hip_ex, run_oracle, sub_workload

pytestmark = pytest.mark.gpu

# batch, head_q, head_k, seq_k, lanes per element in the merge (the launcher's rule: one lane per element from 2^15
# elements' worth of threads; below that doubled while the splits number 8 x lanes or more)
SHAPES = [
    (20, 129, 1, 1500, 1),
    (32, 128, 1, 1024, 1),
    (16, 100, 1, 2048, 1),
    (4, 192, 2, 3000, 1),
    (1, 128, 1, 1536, 2),
    (1, 192, 2, 1280, 2),
    (2, 100, 1, 2560, 4),
    (1, 200, 2, 8192, 8),
    (2, 65, 1, 4096, 8),
]


def _merge_lanes(batch, head_q, nsplit):
    if batch * head_q * 128 >= (1 << 15):
        return 1
    sg = 1
    while sg < 8 and nsplit >= 8 * sg:
        sg *= 2
    return sg


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["fp16", "bf16"])
@pytest.mark.parametrize("batch,head_q,head_k,seq_k,lanes", SHAPES)
def test_split_partials_at_any_head_count(batch, head_q, head_k, seq_k, lanes, dtype):
    w = wl.make_workload(batch, head_q, head_k, 576, 512, seq_k, dtype, seed=head_q + seq_k, latent=True)
    p = _lib.plan(w.max_seq_k, batch, head_q, head_k, 576, 512, total_k=w.k.shape[0])
    assert p["kind"] == 2 and p["heads_per_group"] == 128 and p["nsplit"] > 1
    assert _merge_lanes(batch, head_q, p["nsplit"]) == lanes
    o = run_hip(w)
    assert torch.isfinite(o.float()).all()
    rows = list(range(batch)) if batch <= 4 else [0, 1, batch // 2, batch - 1]
    _, ref32 = run_oracle(sub_workload(w, rows))
    err = (o[rows].float() - ref32).abs().max().item()
    assert err <= TOL[dtype], f"max-abs {err:.3e}"


@pytest.mark.parametrize("head_q,head_k", [(100, 1), (192, 2)])
def test_ragged_lengths_leave_some_splits_empty(head_q, head_k):
    """Lengths from one token to the maximum: short sequences have fewer live splits than the plan, and the slots of
    the dead ones hold whatever an earlier call left there (the workspace is filled with NaN patterns first)."""
    lens = torch.tensor([1, 31, 32, 33, 700, 2048, 0, 1500, 257, 1024, 2047, 90], dtype=torch.int32)
    g = torch.Generator().manual_seed(5)
    total = int(lens.sum())
    q = torch.randn(len(lens), head_q, 576, generator=g).to(torch.float16)
    k = torch.randn(total, head_k, 576, generator=g).to(torch.float16)
    w = wl.Workload("ragged_splits", q, k, None, wl.get_cu_seq(lens), int(lens.max()), 512, False, lens.tolist())
    p = _lib.plan(w.max_seq_k, len(lens), head_q, head_k, 576, 512)
    assert p["kind"] == 2 and p["nsplit"] > 1
    o = run_hip_ex(w, 0, fill=0xFF)
    check_against_oracle(w, o)
    assert (o[6].float() == 0).all()
