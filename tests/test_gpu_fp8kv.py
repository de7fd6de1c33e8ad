"""FP8 (e4m3) K/V cache: q and o stay 16-bit, K/V are one byte per element with per-KV-head scales.

FP8 values convert exactly to fp16/bf16, so with unit scales the FP8 call must agree with the 16-bit call on the
same (FP8-representable) values up to the order of fp32 summation; with scales it is checked against float64
attention on the de-quantised inputs at the usual tolerance.
"""
import pytest
import torch

from decoding_attention_amd import _lib, decoding_attn_fwd, decoding_attn_paged_fwd
from decoding_attention_amd import workloads as wl
from oracle import oracle
from tests.gpu_util import TOL

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
FP8 = torch.float8_e4m3fn


def _quantise(x, scale):
    """x / scale[head] rounded to FP8; scale is a float32 [head_k] tensor."""
    return (x.float() / scale.view(1, -1, 1)).to(FP8)


def _case(batch, head_q, head_k, dim, dim_v, seq_k, dtype, *, latent=False, is_alibi=False, unit=False, seed=3):
    w = wl.make_workload(batch, head_q, head_k, dim, dim_v, seq_k, dtype, seed=seed, varlen=True, is_alibi=is_alibi,
                         latent=latent if latent else None)
    g = torch.Generator().manual_seed(seed + 100)
    if unit:
        ks = torch.ones(head_k)
        vs = torch.ones(head_k)
    else:
        ks = 0.015 + 0.015 * torch.rand(head_k, generator=g)  # N(0,1) data over 0.015..0.03 stays inside +-448
        vs = 0.015 + 0.015 * torch.rand(head_k, generator=g)
    k8 = _quantise(w.k, ks)
    v8 = None if w.v is None else _quantise(w.v, vs)
    return w, k8, v8, ks, vs


def _reference(w, k8, v8, ks, vs):
    k_deq = k8.float() * ks.view(1, -1, 1)
    if v8 is None:
        # V is the leading columns of the de-quantised K (one scale serves both)
        return oracle.attn_f64(w.q, k_deq, None, w.cu_seq_k, w.dim_v, w.is_alibi)
    v_deq = v8.float() * vs.view(1, -1, 1)
    return oracle.attn_f64(w.q, k_deq, v_deq, w.cu_seq_k, w.dim_v, w.is_alibi)


def _run(w, k8, v8, ks, vs, scales=True):
    kw = dict(k_scale=ks.to(DEV), v_scale=vs.to(DEV)) if scales else {}
    o = decoding_attn_fwd(w.q.to(DEV), k8.to(DEV), None if v8 is None else v8.to(DEV), w.cu_seq_k.to(DEV),
                          w.max_seq_k, w.dim_v, w.is_alibi, **kw)
    torch.cuda.synchronize()
    return o.cpu()


SHAPES = [
    # batch, head_q, head_k, dim, dim_v, seq_k
    (5, 8, 8, 128, 128, 700),      # MHA: VALU sweep
    (3, 4, 2, 64, 64, 333),        # ratio 2: VALU sweep
    (6, 32, 8, 128, 128, 1500),    # GQA: grouped MFMA, one wave per KV head
    (4, 32, 1, 128, 128, 1200),    # MQA: grouped MFMA, 32 heads per group, waves split the tokens
    (3, 16, 4, 64, 64, 900),       # GQA d64
    (2, 16, 4, 256, 256, 500),     # GQA d256
    (3, 12, 4, 96, 96, 400),       # d96: no FP8 form of the grouped kernel, VALU sweep
]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", SHAPES)
def test_fp8_kv_with_scales_matches_float64_attention(shape, dtype):
    w, k8, v8, ks, vs = _case(*shape, dtype)
    o = _run(w, k8, v8, ks, vs)
    ref = torch.from_numpy(_reference(w, k8, v8, ks, vs)).float()
    assert torch.isfinite(o.float()).all()
    err = (o.float() - ref).abs().max().item()
    assert err <= TOL[dtype], f"max-abs {err:.3e}"


@pytest.mark.parametrize("shape", [SHAPES[0], SHAPES[2], SHAPES[3]])
def test_unit_scales_agree_with_the_16_bit_path_on_the_same_values(shape):
    """The FP8 values, widened on the host, through the 16-bit entry point: same numbers up to summation order."""
    w, k8, v8, ks, vs = _case(*shape, torch.float16, unit=True)
    o8 = _run(w, k8, v8, ks, vs, scales=False)
    o16 = decoding_attn_fwd(w.q.to(DEV), k8.to(torch.float16).to(DEV), v8.to(torch.float16).to(DEV),
                            w.cu_seq_k.to(DEV), w.max_seq_k, w.dim_v, w.is_alibi).cpu()
    assert (o8.float() - o16.float()).abs().max().item() <= 2 ** -9  # a few fp16 ulps of O(1) values


def test_alibi_and_softmax_scale_with_fp8_kv():
    w, k8, v8, ks, vs = _case(4, 32, 1, 128, 128, 800, torch.float16, is_alibi=True)
    o = decoding_attn_fwd(w.q.to(DEV), k8.to(DEV), v8.to(DEV), w.cu_seq_k.to(DEV), w.max_seq_k, 128, True,
                          softmax_scale=0.05, k_scale=ks.to(DEV), v_scale=vs.to(DEV)).cpu()
    ref = oracle.attn_f64(w.q, k8.float() * ks.view(1, -1, 1), v8.float() * vs.view(1, -1, 1), w.cu_seq_k, 128, True,
                          softmax_scale=0.05)
    assert (o.float() - torch.from_numpy(ref).float()).abs().max().item() <= TOL[torch.float16]


@pytest.mark.parametrize("batch,head_q,seq_k,dtype,is_alibi", [
    (2, 16, 300, torch.float16, False),     # one wave of 32 heads, half of them idle
    (3, 64, 700, torch.bfloat16, False),    # two waves
    (5, 128, 1500, torch.float16, False),   # four waves, several splits
    (4, 128, 900, torch.bfloat16, True),
    (1, 128, 5000, torch.float16, False),   # one long sequence: many short splits
    (7, 32, 97, torch.float16, True),       # shorter than four tiles
])
def test_latent_form_with_fp8_cache(batch, head_q, seq_k, dtype, is_alibi):
    """(576, 512) with V = K[..., :512]: the latent MFMA kernel over FP8 tiles converted in LDS (one scale for K
    and V, as they are one buffer)."""
    w, k8, _, ks, _ = _case(batch, head_q, 1, 576, 512, seq_k, dtype, latent=True, is_alibi=is_alibi, seed=seq_k)
    o = decoding_attn_fwd(w.q.to(DEV), k8.to(DEV), None, w.cu_seq_k.to(DEV), w.max_seq_k, 512, is_alibi,
                          k_scale=ks.to(DEV), v_scale=ks.to(DEV)).cpu()
    ref = torch.from_numpy(_reference(w, k8, None, ks, ks)).float()
    assert (o.float() - ref).abs().max().item() <= TOL[dtype]


@pytest.mark.parametrize("batch,head_q,seq_k", [(300, 64, 600), (6, 64, 3000), (6, 128, 3000)])
def test_latent_fp8_unit_scales_equal_the_16_bit_call(batch, head_q, seq_k):
    """FP8 values convert exactly and the tiles are converted before any arithmetic: with unit scales the FP8 call
    is the 16-bit call on the same values.  Up to 64 heads both run the same kernel, and where neither call splits
    its sequences (300 sequences of 600 tokens) in the same order of operations: same bits.  Where they split, the
    two plans cut the sequences differently (the 16-bit form runs two work-groups to a CU) and the partials are
    rounded to 16 bits, and with 128 heads the 16-bit call runs on the software-pipelined kernel: equal within the
    output tolerance."""
    # (large enough for the planner to pick the latent kernel, whose property this is)
    w, k8, _, ks, _ = _case(batch, head_q, 1, 576, 512, seq_k, torch.float16, latent=True, unit=True, seed=9)
    plan = _lib.plan(w.max_seq_k, batch, head_q, 1, 576, 512, total_k=w.k.shape[0])
    assert plan["kind"] == 2
    k16 = k8.to(torch.float16).to(DEV)
    args = (w.cu_seq_k.to(DEV), w.max_seq_k, 512, False)
    o8 = decoding_attn_fwd(w.q.to(DEV), k8.to(DEV), None, *args, k_scale=ks.to(DEV), v_scale=ks.to(DEV))
    o16 = decoding_attn_fwd(w.q.to(DEV), k16, None, *args)
    if batch == 300:
        assert plan["nsplit"] == 1
        assert torch.equal(o8.view(torch.int16), o16.view(torch.int16))
    else:
        assert (o8.float() - o16.float()).abs().max().item() <= TOL[torch.float16]


@pytest.mark.parametrize("page_size", [1, 4, 16, 32, 64])
def test_latent_paged_fp8(page_size):
    w, k8, _, ks, _ = _case(5, 128, 1, 576, 512, 1100, torch.float16, latent=True, seed=21)
    w8 = wl.Workload(w.name, w.q, k8.view(torch.uint8), None, w.cu_seq_k, w.max_seq_k, w.dim_v, w.is_alibi, w.lengths)
    pk = wl.to_pages(w8, page_size, seed=2, poison=False).to(DEV)
    o = decoding_attn_paged_fwd(w.q.to(DEV), pk.k_pages.view(FP8), None, pk.block_table, pk.seq_lens, w.max_seq_k,
                                512, False, k_scale=ks.to(DEV), v_scale=ks.to(DEV)).cpu()
    ref = torch.from_numpy(_reference(w, k8, None, ks, ks)).float()
    assert (o.float() - ref).abs().max().item() <= TOL[torch.float16]


@pytest.mark.parametrize("page_size", [1, 8, 16, 64])
def test_paged_fp8_kv(page_size):
    w, k8, v8, ks, vs = _case(6, 32, 8, 128, 128, 1100, torch.bfloat16)
    w8 = wl.Workload(w.name, w.q, k8.view(torch.uint8), v8.view(torch.uint8), w.cu_seq_k, w.max_seq_k, w.dim_v,
                     w.is_alibi, w.lengths)
    pk = wl.to_pages(w8, page_size, seed=2, poison=False).to(DEV)
    o = decoding_attn_paged_fwd(w.q.to(DEV), pk.k_pages.view(FP8), pk.v_pages.view(FP8), pk.block_table, pk.seq_lens,
                                w.max_seq_k, 128, False, k_scale=ks.to(DEV), v_scale=vs.to(DEV)).cpu()
    ref = torch.from_numpy(_reference(w, k8, v8, ks, vs)).float()
    assert (o.float() - ref).abs().max().item() <= TOL[torch.bfloat16]


def test_full_size_gqa_fp8_spot_checked():
    """The benchmark shape with an FP8 cache; a sample of sequences against float64."""
    w, k8, v8, ks, vs = _case(64, 32, 8, 128, 128, 4096, torch.bfloat16)
    o = _run(w, k8, v8, ks, vs)
    cu = w.cu_seq_k.tolist()
    for b in (0, 17, 63):
        sub = wl.Workload("sub", w.q[b:b + 1], w.k[cu[b]:cu[b + 1]], w.v[cu[b]:cu[b + 1]],
                          torch.tensor([0, cu[b + 1] - cu[b]], dtype=torch.int32), w.max_seq_k, 128, False,
                          [cu[b + 1] - cu[b]])
        ref = torch.from_numpy(_reference(sub, k8[cu[b]:cu[b + 1]], v8[cu[b]:cu[b + 1]], ks, vs)).float()
        assert (o[b:b + 1].float() - ref).abs().max().item() <= TOL[torch.bfloat16]


def test_argument_errors():
    w, k8, v8, ks, vs = _case(2, 8, 8, 128, 128, 100, torch.float16)
    q, cu = w.q.to(DEV), w.cu_seq_k.to(DEV)
    with pytest.raises(RuntimeError, match="same dtype"):
        decoding_attn_fwd(q, k8.to(DEV), w.v.to(DEV), cu, w.max_seq_k, 128, False)
    with pytest.raises(RuntimeError, match="K/V cache only"):
        decoding_attn_fwd(q, w.k.to(DEV), w.v.to(DEV), cu, w.max_seq_k, 128, False, k_scale=ks.to(DEV))
    with pytest.raises(RuntimeError, match="head_k values"):
        decoding_attn_fwd(q, k8.to(DEV), v8.to(DEV), cu, w.max_seq_k, 128, False, k_scale=ks[:3].to(DEV))
    assert _lib.load().da_workspace_bytes_fp8kv(8192, 1, 32, 8, 128, 128, 0, 0) > 0
