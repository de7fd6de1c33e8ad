"""int8 K/V cache: q and o stay 16-bit, K/V are two's-complement bytes with one symmetric scale per KV head.

Every int8 value converts exactly to fp16 and to bf16, so with unit scales the int8 call must agree with the 16-bit
call on the same integers (bit for bit where the kernel converts whole tiles before any arithmetic); with scales it
is checked against float64 attention on the de-quantised inputs at the usual tolerance.
"""
import pytest
import torch

from decoding_attention_amd import _lib, decoding_attn_fwd, decoding_attn_paged_fwd
from decoding_attention_amd import workloads as wl
from oracle import oracle
from tests.gpu_util import TOL

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _quantise(x, scale):
    """round(x / scale[head]) clamped to int8; scale is a float32 [head_k] tensor."""
    return torch.round(x.float() / scale.view(1, -1, 1)).clamp(-128, 127).to(torch.int8)


def _case(batch, head_q, head_k, dim, dim_v, seq_k, dtype, *, latent=False, is_alibi=False, unit=False, seed=3):
    w = wl.make_workload(batch, head_q, head_k, dim, dim_v, seq_k, dtype, seed=seed, varlen=True, is_alibi=is_alibi,
                         latent=latent if latent else None)
    g = torch.Generator().manual_seed(seed + 100)
    if unit:
        # integers of small magnitude as they are (scores stay moderate), plus both ends of the range
        ks = torch.ones(head_k)
        vs = torch.ones(head_k)
        k8 = torch.round(w.k.float() * 1.5).clamp(-128, 127).to(torch.int8)
        v8 = None if w.v is None else torch.round(w.v.float() * 40).clamp(-128, 127).to(torch.int8)
        k8.view(-1)[::97] = 5
        k8.view(-1)[3::1013] = -6
        if v8 is not None:
            v8.view(-1)[::89] = -128
            v8.view(-1)[1::89] = 127
        return w, k8, v8, ks, vs
    ks = (3.0 + torch.rand(head_k, generator=g)) / 127  # N(0,1) data: 3..4 sigma at full scale, the rest clamps
    vs = (3.0 + torch.rand(head_k, generator=g)) / 127
    k8 = _quantise(w.k, ks)
    v8 = None if w.v is None else _quantise(w.v, vs)
    return w, k8, v8, ks, vs


def _reference(w, k8, v8, ks, vs, **kw):
    k_deq = k8.float() * ks.view(1, -1, 1)
    v_deq = None if v8 is None else v8.float() * vs.view(1, -1, 1)  # None: V is the leading columns of K
    return torch.from_numpy(oracle.attn_f64(w.q, k_deq, v_deq, w.cu_seq_k, w.dim_v, w.is_alibi, **kw)).float()


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
    (3, 12, 4, 96, 96, 400),       # d96: no 8-bit form of the grouped kernel, VALU sweep
    (2, 32, 32, 256, 256, 300),    # MHA d256
]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", SHAPES)
def test_int8_kv_with_scales_matches_float64_attention(shape, dtype):
    w, k8, v8, ks, vs = _case(*shape, dtype)
    o = _run(w, k8, v8, ks, vs)
    assert torch.isfinite(o.float()).all()
    err = (o.float() - _reference(w, k8, v8, ks, vs)).abs().max().item()
    assert err <= TOL[dtype], f"max-abs {err:.3e}"


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", [SHAPES[0], SHAPES[2], SHAPES[3], SHAPES[6]])
def test_unit_scales_agree_with_the_16_bit_path_on_the_same_integers(shape, dtype):
    """The integers, widened on the host (exact in both 16-bit types), through the 16-bit entry point: the same
    numbers up to the order of summation.  Both ends of the int8 range are among the values."""
    w, k8, v8, ks, vs = _case(*shape, dtype, unit=True)
    o8 = _run(w, k8, v8, ks, vs, scales=False)
    o16 = decoding_attn_fwd(w.q.to(DEV), k8.to(dtype).to(DEV), v8.to(dtype).to(DEV), w.cu_seq_k.to(DEV), w.max_seq_k,
                            w.dim_v, w.is_alibi).cpu()
    assert torch.equal(k8.to(dtype).float(), k8.float())  # widening is exact
    scale = max(1.0, o16.float().abs().max().item())
    assert (o8.float() - o16.float()).abs().max().item() <= (2 ** -9 if dtype == torch.float16 else 2 ** -6) * scale


def test_alibi_and_softmax_scale_with_int8_kv():
    w, k8, v8, ks, vs = _case(4, 32, 1, 128, 128, 800, torch.float16, is_alibi=True)
    o = decoding_attn_fwd(w.q.to(DEV), k8.to(DEV), v8.to(DEV), w.cu_seq_k.to(DEV), w.max_seq_k, 128, True,
                          softmax_scale=0.05, k_scale=ks.to(DEV), v_scale=vs.to(DEV)).cpu()
    ref = _reference(w, k8, v8, ks, vs, softmax_scale=0.05)
    assert (o.float() - ref).abs().max().item() <= TOL[torch.float16]


@pytest.mark.parametrize("batch,head_q,seq_k,dtype,is_alibi", [
    (2, 16, 300, torch.float16, False),     # one wave of 32 heads, half of them idle
    (3, 64, 700, torch.bfloat16, False),    # two waves
    (5, 128, 1500, torch.float16, False),   # four waves, several splits
    (4, 128, 900, torch.bfloat16, True),
    (1, 128, 5000, torch.bfloat16, False),  # one long sequence: many short splits
    (7, 32, 97, torch.float16, True),       # shorter than four tiles
])
def test_latent_form_with_int8_cache(batch, head_q, seq_k, dtype, is_alibi):
    """(576, 512) with V = K[..., :512]: the latent MFMA kernel over int8 tiles converted in LDS (one scale for K
    and V, as they are one buffer)."""
    w, k8, _, ks, _ = _case(batch, head_q, 1, 576, 512, seq_k, dtype, latent=True, is_alibi=is_alibi, seed=seq_k)
    o = decoding_attn_fwd(w.q.to(DEV), k8.to(DEV), None, w.cu_seq_k.to(DEV), w.max_seq_k, 512, is_alibi,
                          k_scale=ks.to(DEV), v_scale=ks.to(DEV)).cpu()
    assert (o.float() - _reference(w, k8, None, ks, ks)).abs().max().item() <= TOL[dtype]


@pytest.mark.parametrize("batch,head_q,seq_k", [(300, 64, 600), (6, 64, 3000), (6, 128, 3000)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_latent_int8_unit_scales_equal_the_16_bit_call(dtype, batch, head_q, seq_k):
    """The tiles are converted, exactly, before any arithmetic: with unit scales the int8 call is the 16-bit call on
    the same integers.  Up to 64 heads both run the same kernel, and where neither call splits its sequences (300
    sequences of up to 600 tokens) in the same order of operations: same bits.  Where they split, the two plans cut
    the sequences differently and the partials are rounded to 16 bits, and with 128 heads the 16-bit call runs on the
    software-pipelined kernel: equal within the output tolerance.  All 256 byte values occur."""
    # (large enough for the planner to pick the latent kernel, whose property this is)
    w = wl.make_workload(batch, head_q, 1, 576, 512, seq_k, dtype, seed=9, varlen=True, latent=True)
    plan = _lib.plan(w.max_seq_k, batch, head_q, 1, 576, 512, total_k=w.k.shape[0])
    assert plan["kind"] == 2
    g = torch.Generator().manual_seed(10)
    k8 = torch.round(torch.randn(w.k.shape, generator=g) * 0.7).to(torch.int8)
    k8.view(-1)[::211] = torch.arange(-128, 128, dtype=torch.int8).repeat(k8.numel() // 211 // 256 + 1)[
        :k8.view(-1)[::211].numel()]
    assert len(torch.unique(k8)) == 256
    args = (w.cu_seq_k.to(DEV), w.max_seq_k, 512, False)
    o8 = decoding_attn_fwd(w.q.to(DEV), k8.to(DEV), None, *args)
    o16 = decoding_attn_fwd(w.q.to(DEV), k8.to(dtype).to(DEV), None, *args)
    assert torch.isfinite(o8.float()).all()
    if batch == 300:
        assert plan["nsplit"] == 1
        assert torch.equal(o8.view(torch.int16), o16.view(torch.int16))
    else:
        # (integer values up to 128 in magnitude: outputs of order 1, so the tolerance is relative)
        scale = max(1.0, o16.float().abs().max().item())
        assert (o8.float() - o16.float()).abs().max().item() <= TOL[dtype] * scale


@pytest.mark.parametrize("page_size", [1, 4, 16, 32, 64])
def test_latent_paged_int8(page_size):
    w, k8, _, ks, _ = _case(5, 128, 1, 576, 512, 1100, torch.float16, latent=True, seed=21)
    w8 = wl.Workload(w.name, w.q, k8.view(torch.uint8), None, w.cu_seq_k, w.max_seq_k, w.dim_v, w.is_alibi, w.lengths)
    pk = wl.to_pages(w8, page_size, seed=2, poison=False).to(DEV)
    o = decoding_attn_paged_fwd(w.q.to(DEV), pk.k_pages.view(torch.int8), None, pk.block_table, pk.seq_lens,
                                w.max_seq_k, 512, False, k_scale=ks.to(DEV), v_scale=ks.to(DEV)).cpu()
    assert (o.float() - _reference(w, k8, None, ks, ks)).abs().max().item() <= TOL[torch.float16]


@pytest.mark.parametrize("page_size", [1, 8, 16, 64])
def test_paged_int8_kv(page_size):
    w, k8, v8, ks, vs = _case(6, 32, 8, 128, 128, 1100, torch.bfloat16)
    w8 = wl.Workload(w.name, w.q, k8.view(torch.uint8), v8.view(torch.uint8), w.cu_seq_k, w.max_seq_k, w.dim_v,
                     w.is_alibi, w.lengths)
    pk = wl.to_pages(w8, page_size, seed=2, poison=False).to(DEV)
    o = decoding_attn_paged_fwd(w.q.to(DEV), pk.k_pages.view(torch.int8), pk.v_pages.view(torch.int8), pk.block_table,
                                pk.seq_lens, w.max_seq_k, 128, False, k_scale=ks.to(DEV), v_scale=vs.to(DEV)).cpu()
    assert (o.float() - _reference(w, k8, v8, ks, vs)).abs().max().item() <= TOL[torch.bfloat16]


def test_full_size_gqa_int8_spot_checked():
    """The benchmark shape with an int8 cache; a sample of sequences against float64."""
    w, k8, v8, ks, vs = _case(64, 32, 8, 128, 128, 4096, torch.bfloat16)
    o = _run(w, k8, v8, ks, vs)
    cu = w.cu_seq_k.tolist()
    for b in (0, 17, 63):
        sub = wl.Workload("sub", w.q[b:b + 1], w.k[cu[b]:cu[b + 1]], w.v[cu[b]:cu[b + 1]],
                          torch.tensor([0, cu[b + 1] - cu[b]], dtype=torch.int32), w.max_seq_k, 128, False,
                          [cu[b + 1] - cu[b]])
        ref = _reference(sub, k8[cu[b]:cu[b + 1]], v8[cu[b]:cu[b + 1]], ks, vs)
        assert (o[b:b + 1].float() - ref).abs().max().item() <= TOL[torch.bfloat16]


def test_argument_errors():
    w, k8, v8, ks, vs = _case(2, 8, 8, 128, 128, 100, torch.float16)
    q, cu = w.q.to(DEV), w.cu_seq_k.to(DEV)
    with pytest.raises(RuntimeError, match="same dtype"):
        decoding_attn_fwd(q, k8.to(DEV), w.v.to(DEV), cu, w.max_seq_k, 128, False)
    with pytest.raises(RuntimeError, match="same dtype"):
        decoding_attn_fwd(q, k8.to(DEV), v8.view(torch.float8_e4m3fn).to(DEV), cu, w.max_seq_k, 128, False)
    with pytest.raises(RuntimeError, match="head_k values"):
        decoding_attn_fwd(q, k8.to(DEV), v8.to(DEV), cu, w.max_seq_k, 128, False, k_scale=ks[:3].to(DEV))
    lib = _lib.load()
    assert lib.da_workspace_bytes_int8kv(8192, 1, 32, 8, 128, 128, 0, 0) == \
        lib.da_workspace_bytes_fp8kv(8192, 1, 32, 8, 128, 128, 0, 0) > 0
