"""Small paged cases of the balanced grid, run as a script in a process of its own (tests/test_gpu_balanced.py starts
it once): the library reads its tunables when it is loaded, and these cases need DA_FLAT_PAGED_MIN_MB=0 so that
paged K/V of a few megabytes takes the balanced grid, which by default only large ragged batches do."""
import os
import sys

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

from decoding_attention_amd import _lib, decoding_attn_paged_fwd  # noqa: E402
from decoding_attention_amd import workloads as wl  # noqa: E402
from tests.gpu_util import check_against_oracle  # noqa: E402

DEV = "cuda:0"
MIXED = [0, 0, 1, 5000, 0, 37, 2048, 1, 8191, 64, 0, 3000, 333, 4096, 31, 33, 0]


def workload(lens, hq, hk, dim, dtype, seed, is_alibi=False):
    g = torch.Generator().manual_seed(seed)
    lens = torch.tensor(lens, dtype=torch.int32)
    total = int(lens.sum())
    q = torch.randn(len(lens), hq, dim, generator=g).to(dtype)
    k = torch.randn(total, hk, dim, generator=g).to(dtype)
    v = torch.randn(total, hk, dim, generator=g).to(dtype)
    return wl.Workload("paged_balanced", q, k, v, wl.get_cu_seq(lens), int(lens.max()), dim, is_alibi, lens.tolist())


def run_case(name, w, page_size, hint):
    b, hq, d = w.q.shape
    hk = w.k.shape[1]
    lib = _lib.load()
    # the paged plan is the balanced one: its workspace holds one more share than max_seq_k fills, plus the positions
    fixed = lib.da_workspace_bytes_paged(w.max_seq_k, b, hq, hk, d, w.dim_v, 0, page_size)
    flat = lib.da_workspace_bytes_paged(w.max_seq_k, b, hq, hk, d, w.dim_v, hint, page_size)
    assert flat != fixed and flat % 16 == 0, (name, fixed, flat)
    pk = wl.to_pages(w, page_size, seed=3).to(DEV)
    wd = w.to(DEV)
    o = decoding_attn_paged_fwd(wd.q, pk.k_pages, pk.v_pages, pk.block_table, pk.seq_lens, w.max_seq_k, w.dim_v,
                                w.is_alibi, total_k=hint)
    torch.cuda.synchronize()
    o = o.cpu()
    assert torch.isfinite(o.float()).all(), name  # unused pool rows are NaN
    check_against_oracle(w, o)
    for i, n in enumerate(w.lengths):
        if n == 0:
            assert torch.count_nonzero(o[i]) == 0, name
    print("ok", name, flush=True)


def main():
    assert os.environ.get("DA_FLAT_PAGED_MIN_MB") == "0"
    for hq, hk in [(32, 8), (32, 2), (32, 1)]:
        for page_size in (32, 64, 256):
            w = workload(MIXED, hq, hk, 128, torch.bfloat16, seed=hq + hk + page_size)
            run_case(f"mixed hq{hq} hk{hk} page{page_size}", w, page_size, int(w.k.shape[0]))
    w = workload(MIXED, 16, 4, 64, torch.float16, seed=77, is_alibi=True)
    run_case("mixed d64 alibi", w, 64, int(w.k.shape[0]))
    g = torch.Generator().manual_seed(5)
    lens = torch.randint(64, 140, (300,), generator=g).tolist()
    lens[17] = 6000
    w = workload(lens, 32, 8, 128, torch.float16, seed=6)
    run_case("many short sequences", w, 32, int(w.k.shape[0]))
    w = workload(MIXED, 32, 8, 128, torch.bfloat16, seed=12)
    for factor in (0.6, 1.5):  # a hint that is not the true count only balances worse
        run_case(f"hint x{factor}", w, 64, int(int(w.k.shape[0]) * factor))
    print("all ok", flush=True)


if __name__ == "__main__":
    main()
