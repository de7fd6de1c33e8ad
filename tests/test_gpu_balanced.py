"""Balanced grid of the grouped-head kernel: for a packed batch that the token count shows to be ragged, and for a
large batch given without a count, every work-group takes an equal share of the concatenated tokens (derived on the
device from cu_seq_k[batch]), across sequence boundaries.  The results must
match the oracle exactly as the fixed-split grid's do, whatever the lengths are: empty sequences anywhere, many
short sequences inside one share, one sequence over many shares, and a hint that is too small or too large.
"""
import os
import subprocess
import sys

import pytest
import torch

from decoding_attention_amd import _lib, decoding_attn_paged_fwd
from decoding_attention_amd import workloads as wl
from tests.gpu_util import TOL, check_against_oracle, run_hip_ex, sub_workload

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
    """The planner chose equal token shares of the concatenated sequences."""
    b, hq, d = w.q.shape
    hk = w.k.shape[1]
    return _lib.plan(w.max_seq_k, b, hq, hk, d, w.dim_v, True, hint)["balanced"]


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


@pytest.mark.parametrize("seed", range(8))
def test_random_ragged_batches(seed):
    """Random batch size, head grouping and lengths (zeros included, one long sequence so that the batch counts as
    ragged); every row against the oracle for small batches, a sample of rows for large ones."""
    g = torch.Generator().manual_seed(1000 + seed)
    batch = int(torch.randint(2, 700, (1,), generator=g))
    hq, hk = [(32, 8), (16, 16), (32, 1), (24, 4), (32, 2), (16, 4), (64, 8), (12, 12)][seed]
    dim, dtype = [(128, torch.float16), (64, torch.bfloat16), (128, torch.bfloat16), (96, torch.float16)][seed % 4]
    hi = int(torch.randint(80, 400, (1,), generator=g))
    lens = torch.randint(0, hi, (batch,), generator=g)
    lens[torch.rand(batch, generator=g) < 0.1] = 0
    lens[int(torch.randint(0, batch, (1,), generator=g))] = max(10 * hi, 3000)
    if int(lens.sum()) < 64 * batch:
        lens += 64
    w = _workload(lens.tolist(), hq, hk, dim, dtype, seed=2000 + seed, is_alibi=bool(seed & 1))
    total = int(w.k.shape[0])
    if not _is_balanced(w, total):
        pytest.skip("the planner kept fixed splits for this shape (VALU sweep)")
    o = _run_ex(w, total)
    assert torch.isfinite(o.float()).all()
    rows = list(range(batch)) if batch <= 64 else sorted(set(torch.randint(0, batch, (48,), generator=g).tolist()) |
                                                         {0, batch - 1, int(lens.argmax())})
    check_against_oracle(sub_workload(w, rows), o[rows])
    empty = [b for b in range(batch) if w.lengths[b] == 0]
    assert all(torch.count_nonzero(o[b]) == 0 for b in empty)


def test_paged_small_cases_in_a_process_with_the_size_threshold_off():
    """Paged K/V takes the balanced grid only from 512 MB of K/V (it costs one more small kernel); the edge cases
    are small, so they run in a process of their own that loads the library with that threshold at zero."""
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, DA_FLAT_PAGED_MIN_MB="0")
    r = subprocess.run([sys.executable, os.path.join(root, "tests", "paged_balanced_cases.py")], env=env, cwd=root,
                       capture_output=True, text=True, timeout=600)
    assert r.returncode == 0 and "all ok" in r.stdout, r.stdout[-2000:] + r.stderr[-4000:]


def test_paged_large_ragged_batch_takes_the_balanced_grid():
    """A ragged paged batch above the size threshold (0.6 GB of K/V): balanced plan, spot-checked against the oracle."""
    g = torch.Generator().manual_seed(21)
    lens = torch.randint(1, 16385, (18,), generator=g).tolist()
    lens[0], lens[5] = 16384, 0
    w = _workload(lens, 32, 8, 128, torch.bfloat16, seed=22)
    total, b = int(w.k.shape[0]), len(lens)
    assert total * 8 * 256 * 2 >= 512e6
    lib = _lib.load()
    flat = lib.da_workspace_bytes_paged(w.max_seq_k, b, 32, 8, 128, 128, total, 64)
    assert _lib.plan(w.max_seq_k, b, 32, 8, 128, 128, total_k=total, page_size=64)["balanced"]
    # a partial slot per (share, sequence) pair that can occur, then the sequences' positions
    slots, rest = divmod(flat - ((b + 1) * 4 + 15) // 16 * 16, 32 * (128 + 2) * 4)
    assert rest == 0 and b < slots <= 256 + b
    pk = wl.to_pages(w, 64, seed=3).to(DEV)
    wd = w.to(DEV)
    o = decoding_attn_paged_fwd(wd.q, pk.k_pages, pk.v_pages, pk.block_table, pk.seq_lens, w.max_seq_k, w.dim_v,
                                False, total_k=total).cpu()
    assert torch.isfinite(o.float()).all()
    assert torch.count_nonzero(o[5]) == 0
    rows = [0, 1, 7, 17]
    sub = sub_workload(w, rows)
    check_against_oracle(sub, o[rows])


@pytest.mark.parametrize("hq,hk,dim,dtype", [(32, 8, 128, torch.bfloat16), (32, 1, 128, torch.float16),
                                             (16, 4, 64, torch.float16)])
def test_large_batch_without_a_token_count_takes_the_balanced_grid(hq, hk, dim, dtype):
    """The reference's signature carries no token count (csrc/ops/decoding_attn.h:29-30): a batch large enough for
    whole shares takes the balanced grid all the same, the share derived on the device.  Ragged lengths with empty
    sequences, every row against the oracle, through da_decoding_attn itself; and a workspace poisoned with NaN
    (stale slots must never be read) through da_decoding_attn_ex with hint 0."""
    g = torch.Generator().manual_seed(31)
    lens = torch.randint(1, 8193, (40,), generator=g).tolist()
    lens[3], lens[17], lens[39] = 0, 8192, 1
    w = _workload(lens, hq, hk, dim, dtype, seed=32)
    b = len(lens)
    assert _lib.plan(w.max_seq_k, b, hq, hk, dim, dim)["balanced"]
    lib = _lib.load()
    wd = w.to(DEV)
    o = torch.full((b, hq, dim), float("nan"), dtype=dtype, device=DEV)
    rc = lib.da_decoding_attn(wd.q.data_ptr(), wd.k.data_ptr(), wd.v.data_ptr(), o.data_ptr(), wd.cu_seq_k.data_ptr(),
                              w.max_seq_k, b, hq, hk, dim, dim, 0, int(dtype == torch.bfloat16),
                              torch.cuda.current_stream().cuda_stream)
    assert rc == 0, _lib.last_error()
    torch.cuda.synchronize()
    check_against_oracle(w, o.cpu())
    assert torch.count_nonzero(o[3]) == 0
    o2 = run_hip_ex(w, 0, fill=0xFF)
    assert torch.equal(o2.view(torch.int16), o.cpu().view(torch.int16))
