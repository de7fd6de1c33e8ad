"""The latent form (576, 512) with 16 query heads or fewer, as a tensor-parallel shard of an MLA model has them: it
runs on the grouped-head kernel (K rows loaded once, their value columns parked in LDS from the K registers).  Every
layout and cache format of that kernel against float64 attention, and against the latent kernel's result for the
same inputs (17 heads and more take that one)."""
import pytest
import torch

from decoding_attention_amd import _lib, decoding_attn_fwd, decoding_attn_paged_fwd
from decoding_attention_amd import workloads as wl
from oracle import oracle
from tests.gpu_util import TOL, check_against_oracle, run_hip

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _latent(batch, head_q, seq_k, dtype, seed, is_alibi=False, varlen=True):
    return wl.make_workload(batch, head_q, 1, 576, 512, seq_k, dtype, seed=seed, varlen=varlen, is_alibi=is_alibi,
                            latent=True)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("head_q", [1, 5, 8, 16])
@pytest.mark.parametrize("batch,seq_k,is_alibi", [(1, 1, False), (3, 97, True), (5, 1500, False), (2, 5000, True)])
def test_packed(head_q, batch, seq_k, is_alibi, dtype):
    w = _latent(batch, head_q, seq_k, dtype, seed=head_q + seq_k, is_alibi=is_alibi)
    assert _lib.plan(w.max_seq_k, batch, head_q, 1, 576, 512)["kind"] == 3
    check_against_oracle(w, run_hip(w))


def test_the_first_16_heads_of_a_larger_model_give_the_same_rows():
    """Heads are independent: the shard's result is the first rows of the full model's (latent kernel) up to the
    order of summation."""
    full = _latent(4, 64, 1200, torch.float16, seed=3, varlen=False)
    o_full = run_hip(full)
    # ALiBi off, so the head count does not enter the arithmetic of a head
    shard = wl.Workload("shard", full.q[:, :16].contiguous(), full.k, None, full.cu_seq_k, full.max_seq_k, 512, False,
                        full.lengths)
    o_shard = run_hip(shard)
    assert (o_shard.float() - o_full[:, :16].float()).abs().max().item() <= 2 ** -10


@pytest.mark.parametrize("page_size", [1, 4, 16, 32, 64])
@pytest.mark.parametrize("fmt", ["f16", "fp8", "int8"])
def test_paged_and_8_bit(page_size, fmt):
    w = _latent(5, 16, 1100, torch.float16, seed=21 + page_size)
    kw = {}
    k_true, k_store = w.k.float(), w.k
    if fmt != "f16":
        ks = torch.tensor([0.03])
        if fmt == "fp8":
            k_store = (w.k.float() / ks).to(torch.float8_e4m3fn)
        else:
            k_store = torch.round(w.k.float() / ks).clamp(-128, 127).to(torch.int8)
        k_true = k_store.float() * ks
        kw = dict(k_scale=ks.to(DEV), v_scale=ks.to(DEV))
    ref = torch.from_numpy(oracle.attn_f64(w.q, k_true, None, w.cu_seq_k, 512, False)).float()
    raw = k_store if fmt == "f16" else k_store.view(torch.uint8)
    src = wl.Workload(w.name, w.q, raw, None, w.cu_seq_k, w.max_seq_k, 512, False, w.lengths)
    pk = wl.to_pages(src, page_size, seed=2, poison=fmt == "f16").to(DEV)
    pages = pk.k_pages if fmt == "f16" else pk.k_pages.view(k_store.dtype)
    o_paged = decoding_attn_paged_fwd(w.q.to(DEV), pages, None, pk.block_table, pk.seq_lens, w.max_seq_k, 512, False,
                                      **kw).cpu()
    o_packed = decoding_attn_fwd(w.q.to(DEV), k_store.to(DEV), None, w.cu_seq_k.to(DEV), w.max_seq_k, 512, False,
                                 **kw).cpu()
    assert (o_packed.float() - ref).abs().max().item() <= TOL[torch.float16]
    assert (o_paged.float() - ref).abs().max().item() <= TOL[torch.float16]


def test_ragged_batch_with_token_count_takes_the_balanced_grid():
    lens = [0, 3000, 17, 0, 900, 6000, 64, 1, 2500, 333]
    g = torch.Generator().manual_seed(5)
    total = sum(lens)
    lens_t = torch.tensor(lens, dtype=torch.int32)
    q = torch.randn(len(lens), 16, 576, generator=g).to(torch.bfloat16)
    k = torch.randn(total, 1, 576, generator=g).to(torch.bfloat16)
    w = wl.Workload("ragged", q, k, None, wl.get_cu_seq(lens_t), max(lens), 512, False, lens)
    plan = _lib.plan(w.max_seq_k, len(lens), 16, 1, 576, 512, True, total)
    assert plan["kind"] == 3 and plan["balanced"]  # equal shares
    o = decoding_attn_fwd(q.to(DEV), k.to(DEV), None, w.cu_seq_k.to(DEV), w.max_seq_k, 512, False).cpu()
    check_against_oracle(w, o)
    for b, n in enumerate(lens):
        if n == 0:
            assert torch.count_nonzero(o[b]) == 0


@pytest.mark.parametrize("head_q", [16, 128])
def test_value_passed_as_a_view_of_the_key_rows(head_q):
    """`v = k[..., :512]` is the aliasing the latent kernels are built on: same bits as v = None, not a copy that
    would take the slow path for a distinct V buffer."""
    w = _latent(3, head_q, 900, torch.float16, seed=44)
    q, k, cu = w.q.to(DEV), w.k.to(DEV), w.cu_seq_k.to(DEV)
    o_none = decoding_attn_fwd(q, k, None, cu, w.max_seq_k, 512, False)
    o_view = decoding_attn_fwd(q, k, k[..., :512], cu, w.max_seq_k, 512, False)
    assert torch.equal(o_none.view(torch.int16), o_view.view(torch.int16))
    o_copy = decoding_attn_fwd(q, k, k[..., :512].contiguous(), cu, w.max_seq_k, 512, False)  # a distinct buffer
    assert (o_copy.float() - o_none.float()).abs().max().item() <= 2 ** -10


@pytest.mark.parametrize("head_q", [20, 40, 100, 128])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_small_problems_of_any_head_count_as_groups_of_16(head_q, dtype):
    """Small latent problems run on the grouped kernel whatever the head count, ceil(heads / 16) groups per sequence,
    the last one partly idle when 16 does not divide the head count (65 heads and more: only sequences short enough
    to stay unsplit, the pipelined latent kernel takes the rest)."""
    w = _latent(3, head_q, 600 if head_q <= 64 else 200, dtype, seed=head_q, is_alibi=head_q == 40)
    assert _lib.plan(w.max_seq_k, 3, head_q, 1, 576, 512)["kind"] == 3
    check_against_oracle(w, run_hip(w))
