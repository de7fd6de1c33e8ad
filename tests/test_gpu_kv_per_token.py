"""int4 and int8 K/V caches with a (scale, zero) pair per (token, KV head): K[t, h, c] = scale[t, h] * (n[t, h, c] -
zero[t, h]), n the stored integer (-8 .. 7, or -128 .. 127), and V likewise.  q and o stay 16-bit.

The kernel never builds the de-quantised rows: its matrix instructions run on the integers and the factors enter the
score tile, the probabilities and a per-head correction at the end.  It is therefore checked against float64 attention
on the de-quantised inputs (max-abs 2e-3 fp16 / 1e-2 bf16, the tolerances of test_gpu_parity.py), and against two
properties that a wrong sign or a dropped term in that algebra breaks: shifting every integer and its zero point by the
same amount changes nothing, and zero points of 0 with one scale per head reduce to the per-head int4 call.
"""
import pytest
import torch

from decoding_attention_amd import (_lib, decoding_attn_fwd, decoding_attn_paged_fwd, pack_int4,
                                    quantize_int4_per_token, quantize_int8_per_token)
from decoding_attention_amd import workloads as wl
from oracle import oracle
from tests.gpu_util import TOL, sub_workload

DEV = "cuda:0"


def _unpack(p):
    lo = (p & 15).to(torch.int16)
    hi = (p >> 4).to(torch.int16)
    n = torch.stack([lo, hi], dim=-1).flatten(-2)
    return torch.where(n >= 8, n - 16, n).to(torch.int8)


def _ints(cache, bits):
    """The stored integers of a cache tensor."""
    return _unpack(cache) if bits == 4 else cache


def _cache(ints, bits):
    return pack_int4(ints) if bits == 4 else ints.to(torch.int8)


def test_quantize_int8_per_token_round_trip():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(29, 2, 128, generator=g) * 3 + torch.randn(29, 2, 1, generator=g)
    n, pairs = quantize_int8_per_token(x)
    assert n.dtype == torch.int8 and n.shape == x.shape and pairs.shape == (29, 2, 2)
    assert (n.amin(-1) == -128).all() and (n.amax(-1) == 127).all()
    back = pairs[..., :1] * (n.float() - pairs[..., 1:])
    assert ((back - x).abs() <= pairs[..., :1] * 0.5001).all()


def test_quantize_int4_per_token_round_trip():
    """Row minimum -> -8, row maximum -> 7, reconstruction within half a step, pairs shaped like the rows."""
    g = torch.Generator().manual_seed(0)
    x = torch.randn(37, 3, 64, generator=g) * torch.rand(37, 3, 1, generator=g) * 4 + torch.randn(37, 3, 1, generator=g)
    packed, pairs = quantize_int4_per_token(x)
    assert packed.dtype == torch.uint8 and packed.shape == (37, 3, 32) and pairs.shape == (37, 3, 2)
    n = _unpack(packed)
    assert int(n.min()) == -8 and int(n.max()) == 7
    assert (n.amin(-1) == -8).all() and (n.amax(-1) == 7).all()
    back = pairs[..., :1] * (n.float() - pairs[..., 1:])
    assert ((back - x).abs() <= pairs[..., :1] * 0.5001).all()


def _case(batch, head_q, head_k, dim, seq_k, dtype, *, is_alibi=False, seed=3, varlen=True, bits=4):
    w = wl.make_workload(batch, head_q, head_k, dim, dim, seq_k, dtype, seed=seed, varlen=varlen, is_alibi=is_alibi)
    g = torch.Generator().manual_seed(seed + 50)
    # rows of different spread and offset, so that scales and zero points differ from token to token and head to head
    k = w.k.float() * (0.5 + torch.rand(w.k.shape[0], head_k, 1, generator=g)) + torch.randn(w.k.shape[0], head_k, 1, generator=g)
    v = w.v.float() * (0.5 + torch.rand(w.v.shape[0], head_k, 1, generator=g)) + 0.5 * torch.randn(w.v.shape[0], head_k, 1, generator=g)
    quant = quantize_int4_per_token if bits == 4 else quantize_int8_per_token
    k4, kp = quant(k)
    v4, vp = quant(v)
    return w, k4, v4, kp, vp


def _dequant(cache, pairs):
    ints = _unpack(cache) if cache.dtype == torch.uint8 else cache
    return pairs[..., :1].double() * (ints.double() - pairs[..., 1:].double())


def _reference(w, k4, v4, kp, vp, **kw):
    return torch.from_numpy(oracle.attn_f64(w.q, _dequant(k4, kp), _dequant(v4, vp), w.cu_seq_k, w.dim_v, w.is_alibi,
                                            **kw)).float()


def _run(w, k4, v4, kp, vp, **extra):
    o = decoding_attn_fwd(w.q.to(DEV), k4.to(DEV), v4.to(DEV), w.cu_seq_k.to(DEV), w.max_seq_k, w.dim_v, w.is_alibi,
                          k_scale=kp.to(DEV), v_scale=vp.to(DEV), **extra)
    torch.cuda.synchronize()
    return o.cpu()


SHAPES = [
    # batch, head_q, head_k, dim, seq_k
    (5, 8, 8, 128, 700),       # MHA: one live head per group, one wave per KV head
    (3, 4, 2, 64, 333),        # ratio 2, two KV heads: the four waves share a KV head's tokens
    (6, 32, 8, 128, 1500),     # GQA, one wave per KV head
    (4, 32, 1, 128, 1200),     # MQA: 32 heads per group
    (3, 16, 4, 64, 900),       # d 64
    (2, 16, 4, 256, 500),      # d 256
    (2, 32, 32, 256, 300),     # MHA d 256
    (1, 8, 2, 128, 1),         # a single token
    (64, 32, 8, 128, 2048),    # a full grid, split sequences (ragged: the balanced grid)
]


@pytest.mark.gpu
@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", SHAPES)
def test_per_token_cache_matches_float64_attention(shape, dtype, bits):
    w, k4, v4, kp, vp = _case(*shape, dtype, bits=bits)
    o = _run(w, k4, v4, kp, vp)
    assert torch.isfinite(o.float()).all()
    if w.batch > 8:  # the large case: sampled sequences against float64
        rows = [0, 1, w.batch // 2, w.batch - 1]
        cu = w.cu_seq_k.tolist()
        cat = lambda t: torch.cat([t[cu[b]:cu[b + 1]] for b in rows])  # noqa: E731
        err = (o[rows].float() - _reference(sub_workload(w, rows), cat(k4), cat(v4), cat(kp), cat(vp))).abs().max().item()
    else:
        err = (o.float() - _reference(w, k4, v4, kp, vp)).abs().max().item()
    assert err <= TOL[dtype], f"max-abs {err:.3e}"


@pytest.mark.gpu
def test_uniform_batch_with_fixed_splits():
    """Equal lengths: the planner keeps fixed splits (the ragged case above takes the balanced grid)."""
    w, k4, v4, kp, vp = _case(16, 32, 8, 128, 4096, torch.bfloat16, varlen=False, seed=9)
    plan = _lib.plan(4096, 16, 32, 8, 128, 128, total_k=16 * 4096, kv_bits=_lib.KV_BITS_INT4_PER_TOKEN)
    assert plan["kind"] == 3 and plan["nsplit"] > 1 and not plan["balanced"]
    o = _run(w, k4, v4, kp, vp)
    rows = [0, 7, 15]
    cu = w.cu_seq_k.tolist()
    cat = lambda t: torch.cat([t[cu[b]:cu[b + 1]] for b in rows])  # noqa: E731
    err = (o[rows].float() - _reference(sub_workload(w, rows), cat(k4), cat(v4), cat(kp), cat(vp))).abs().max().item()
    assert err <= TOL[torch.bfloat16]


@pytest.mark.gpu
@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_shifting_integers_and_zero_points_together_changes_nothing(dtype, bits):
    """scale * ((n + 1) - (zero + 1)) is the same row: a sign error or a dropped zero-point term on either side of the
    kernel's algebra (score tile, per-head correction) shows as a difference of the size of the values."""
    w, k4, v4, kp, vp = _case(4, 32, 8, 128, 900, dtype, seed=17, is_alibi=True, bits=bits)
    top = 6 if bits == 4 else 126
    nk, nv = _ints(k4, bits).clamp(max=top), _ints(v4, bits).clamp(max=top)
    a = _run(w, _cache(nk, bits), _cache(nv, bits), kp, vp)
    shift = torch.tensor([0.0, 1.0])
    b = _run(w, _cache(nk + 1, bits), _cache(nv + 1, bits), kp + shift, vp + shift)
    ref = _reference(w, _cache(nk, bits), _cache(nv, bits), kp, vp)
    assert (a.float() - ref).abs().max().item() <= TOL[dtype]
    assert (b.float() - ref).abs().max().item() <= TOL[dtype]
    assert ref.abs().max().item() > 50 * TOL[dtype]  # the check has teeth: the values are far above the tolerance


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_rows_with_a_scale_of_zero(dtype):
    """A constant row may come with a scale of exactly zero: it is a row of zeros, and its probability still counts."""
    w, k4, v4, kp, vp = _case(3, 16, 4, 128, 400, dtype, seed=41)
    g = torch.Generator().manual_seed(4)
    kp[torch.rand(kp.shape[:2], generator=g) < 0.2, 0] = 0.0
    vp[torch.rand(vp.shape[:2], generator=g) < 0.2, 0] = 0.0
    o = _run(w, k4, v4, kp, vp)
    assert torch.isfinite(o.float()).all()
    assert (o.float() - _reference(w, k4, v4, kp, vp)).abs().max().item() <= TOL[dtype]


@pytest.mark.gpu
def test_zero_points_of_zero_reduce_to_the_per_head_call():
    w = wl.make_workload(5, 32, 8, 128, 128, 1100, torch.float16, seed=23, varlen=True)
    ks, vs = torch.full((8,), 3.0 / 7), torch.linspace(0.3, 0.5, 8)
    nk = torch.round(w.k.float() / ks.view(1, -1, 1)).clamp(-8, 7).to(torch.int8)
    nv = torch.round(w.v.float() / vs.view(1, -1, 1)).clamp(-8, 7).to(torch.int8)
    pairs = lambda s: torch.stack([s.expand(w.k.shape[0], 8), torch.zeros(w.k.shape[0], 8)], dim=-1).contiguous()  # noqa: E731
    per_token = _run(w, pack_int4(nk), pack_int4(nv), pairs(ks), pairs(vs))
    per_head = _run(w, pack_int4(nk), pack_int4(nv), ks, vs)
    assert (per_token.float() - per_head.float()).abs().max().item() <= 2 ** -10


@pytest.mark.gpu
@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("shape", [SHAPES[0], SHAPES[2], SHAPES[3]])
def test_paged_pools(shape, bits):
    """Pairs in pools of their own, [pages, page_size, head_k, 2], addressed through the same block table: float64
    attention on the de-quantised rows, and the same bits at every page size (64: one lookup per tile, 16: one per
    run of 16 tokens, 4 and 1: one per row)."""
    w, k4, v4, kp, vp = _case(*shape, torch.float16, seed=21, bits=bits)
    w4 = wl.Workload(w.name, w.q, k4, v4, w.cu_seq_k, w.max_seq_k, w.dim_v, w.is_alibi, w.lengths)
    wp = wl.Workload(w.name, w.q, kp, vp, w.cu_seq_k, w.max_seq_k, w.dim_v, w.is_alibi, w.lengths)
    outs = {}
    for page_size in (64, 16, 4, 1):
        pk = wl.to_pages(w4, page_size, seed=2, poison=False).to(DEV)
        pp = wl.to_pages(wp, page_size, seed=2).to(DEV)  # (same seed: same page numbering; unused entries are NaN)
        assert torch.equal(pk.block_table, pp.block_table)
        outs[page_size] = decoding_attn_paged_fwd(w.q.to(DEV), pk.k_pages, pk.v_pages, pk.block_table, pk.seq_lens,
                                                  w.max_seq_k, w.dim_v, False, k_scale=pp.k_pages,
                                                  v_scale=pp.v_pages).cpu()
    assert (outs[64].float() - _reference(w, k4, v4, kp, vp)).abs().max().item() <= TOL[torch.float16]
    for page_size in (16, 4, 1):
        assert torch.equal(outs[page_size].view(torch.int16), outs[64].view(torch.int16)), page_size


@pytest.mark.gpu
def test_argument_errors():
    w, k4, v4, kp, vp = _case(2, 8, 2, 128, 100, torch.float16)
    q, cu = w.q.to(DEV), w.cu_seq_k.to(DEV)
    with pytest.raises(RuntimeError, match="both K and V"):
        decoding_attn_fwd(q, k4.to(DEV), v4.to(DEV), cu, w.max_seq_k, 128, False, k_scale=kp.to(DEV))
    with pytest.raises(RuntimeError, match="int4 or int8 K/V cache only"):
        decoding_attn_fwd(q, w.k.to(torch.float8_e4m3fn).to(DEV), w.v.to(torch.float8_e4m3fn).to(DEV), cu, w.max_seq_k,
                          128, False, k_scale=kp.to(DEV), v_scale=vp.to(DEV))
    with pytest.raises(RuntimeError, match="leading dimensions"):
        decoding_attn_fwd(q, k4.to(DEV), v4.to(DEV), cu, w.max_seq_k, 128, False, k_scale=kp[:-1].to(DEV),
                          v_scale=vp[:-1].to(DEV))
    w96 = wl.make_workload(2, 6, 2, 96, 96, 64, torch.float16, seed=1)
    k96, p96 = quantize_int4_per_token(w96.k)
    with pytest.raises(RuntimeError, match="head dims"):
        decoding_attn_fwd(w96.q.to(DEV), k96.to(DEV), k96.to(DEV), w96.cu_seq_k.to(DEV), 64, 96, False,
                          k_scale=p96.to(DEV), v_scale=p96.to(DEV))
