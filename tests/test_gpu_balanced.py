"""Balanced grid of the grouped-head kernel: when the caller gives the total token count of a ragged packed batch,
every work-group takes an equal share of the concatenated tokens, across sequence boundaries.  The results must
match the oracle exactly as the fixed-split grid's do, whatever the lengths are: empty sequences anywhere, many
short sequences inside one share, one sequence over many shares, and a hint that is too small or too large.
"""
import pytest
import torch

from decoding_attention_amd import _lib
from decoding_attention_amd import workloads as wl
from tests.gpu_util import TOL, check_against_oracle, run_hip_ex

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _workload(lens, hq, hk, dim, dtype, seed, is_alibi=False):
    g = torch.Generator().manual_seed(seed)
    lens = torch.tensor(lens, dtype=torch.int32)
    total = int(lens.sum())
    q = torch.randn(len(lens), hq, dim, generator=g).to(dtype)
    k = torch.randn(total, hk, dim, generator=g).to(dtype)
    v = torch.randn(total, hk, dim, generator=g).to(dtype)
    return wl.Workload("balanced", q, k, v, wl.get_cu_seq(lens), int(lens.max()), dim, is_alibi, lens.tolist())


def _run_ex(w, hint):
    return run_hip_ex(w, hint)


def _is_balanced(w, hint):
    """The planner chose equal token shares: its split length is the share, not a divisor of max_seq_k."""
    b, hq, d = w.q.shape
    hk = w.k.shape[1]
    with_hint = _lib.plan(w.max_seq_k, b, hq, hk, d, d, True, hint)
    return with_hint["kind"] == 3 and with_hint["nsplit"] * with_hint["chunk"] >= w.max_seq_k + with_hint["chunk"]


MIXED = [0, 0, 1, 5000, 0, 37, 2048, 1, 8191, 64, 0, 3000, 333, 4096, 31, 33, 0]


@pytest.mark.parametrize("hq,hk", [(32, 8), (32, 2), (32, 1), (12, 4), (8, 1)])
@pytest.mark.parametrize("dim,dtype", [(128, torch.bfloat16), (64, torch.float16)])
def test_mixed_lengths(hq, hk, dim, dtype):
    w = _workload(MIXED, hq, hk, dim, dtype, seed=hq + hk + dim)
    total = int(w.k.shape[0])
    assert _is_balanced(w, total)
    o = _run_ex(w, total)
    check_against_oracle(w, o)
    for b, n in enumerate(w.lengths):
        if n == 0:
            assert torch.count_nonzero(o[b]) == 0  # an empty sequence yields a zero row


def test_many_short_sequences_share_a_work_group():
    g = torch.Generator().manual_seed(5)
    lens = torch.randint(64, 140, (300,), generator=g).tolist()
    lens[17] = 6000  # keeps max_seq_k far above the mean, so the batch counts as ragged
    w = _workload(lens, 32, 8, 128, torch.float16, seed=6)
    total = int(w.k.shape[0])
    assert _is_balanced(w, total)
    check_against_oracle(w, _run_ex(w, total))


def test_alibi_and_long_sequence_over_many_shares():
    w = _workload([16384, 100, 0, 777, 50, 2000], 32, 8, 128, torch.float16, seed=9, is_alibi=True)
    total = int(w.k.shape[0])
    assert _is_balanced(w, total)
    check_against_oracle(w, _run_ex(w, total))


@pytest.mark.parametrize("factor", [0.6, 1.0, 1.5])
def test_hint_need_not_be_exact(factor):
    """A hint below the true count leaves the remainder to the last work-group; one above it leaves shares empty."""
    w = _workload(MIXED, 32, 8, 128, torch.bfloat16, seed=12)
    hint = int(int(w.k.shape[0]) * factor)
    assert _is_balanced(w, hint)
    check_against_oracle(w, _run_ex(w, hint))


def test_same_result_as_fixed_splits_up_to_summation_order():
    w = _workload(MIXED, 32, 8, 128, torch.bfloat16, seed=13)
    total = int(w.k.shape[0])
    a = _run_ex(w, total).float()
    b = _run_ex(w, 0).float()  # no hint: fixed splits of every sequence
    assert (a - b).abs().max().item() <= TOL[torch.bfloat16]
