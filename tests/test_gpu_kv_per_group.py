"""int4 and int8 K/V caches with a (scale, zero) pair per run of 64 elements of every (token, KV head) row:
K[t, h, c] = scale[t, h, c // 64] * (n[t, h, c] - zero[t, h, c // 64]), V likewise.  q and o stay 16-bit.

As for the per-token form the kernel works on the integers, so it is checked against float64 attention on the
de-quantised inputs (max-abs 2e-3 fp16 / 1e-2 bf16, the tolerances of test_gpu_parity.py, relative to the largest
output where that exceeds 1).  The inputs give every run of a row its own spread and offset, so a kernel that took
another run's pair would miss by the size of the values.
Two properties pin the run numbering on their own: exchanging the runs of V (integers and pairs) exchanges the output's
column runs bit for bit, and exchanging the runs of K together with those of q changes nothing; equal pairs in every
run reduce to the per-token call.
"""
import pytest
import torch

from decoding_attention_amd import (_lib, decoding_attn_fwd, decoding_attn_paged_fwd, quantize_int4_per_group,
                                    quantize_int4_per_token, quantize_int8_per_group, quantize_int8_per_token)
from decoding_attention_amd import workloads as wl
from oracle import oracle
from tests.gpu_util import TOL, sub_workload
from tests.test_gpu_kv_per_token import _unpack

DEV = "cuda:0"


def test_quantize_int4_per_group_round_trip():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(23, 3, 4, 64, generator=g) * (0.2 + 4 * torch.rand(23, 3, 4, 1, generator=g))
    x = (x + 2 * torch.randn(23, 3, 4, 1, generator=g)).flatten(-2)
    packed, pairs = quantize_int4_per_group(x)
    assert packed.dtype == torch.uint8 and packed.shape == (23, 3, 128) and pairs.shape == (23, 3, 4, 2)
    n = _unpack(packed).unflatten(-1, (4, 64))
    assert (n.amin(-1) == -8).all() and (n.amax(-1) == 7).all()
    back = pairs[..., :1] * (n.float() - pairs[..., 1:])
    assert ((back - x.unflatten(-1, (4, 64))).abs() <= pairs[..., :1] * 0.5001).all()
    with pytest.raises(ValueError):
        quantize_int4_per_group(torch.zeros(2, 96))


def test_quantize_int8_per_group_round_trip():
    g = torch.Generator().manual_seed(2)
    x = (torch.randn(11, 2, 2, 64, generator=g) * 3 + torch.randn(11, 2, 2, 1, generator=g)).flatten(-2)
    n, pairs = quantize_int8_per_group(x)
    assert n.dtype == torch.int8 and n.shape == x.shape and pairs.shape == (11, 2, 2, 2)
    runs = n.unflatten(-1, (2, 64))
    assert (runs.amin(-1) == -128).all() and (runs.amax(-1) == 127).all()
    back = pairs[..., :1] * (runs.float() - pairs[..., 1:])
    assert ((back - x.unflatten(-1, (2, 64))).abs() <= pairs[..., :1] * 0.5001).all()


def _case(batch, head_q, head_k, dim, seq_k, dtype, *, is_alibi=False, seed=3, varlen=True, bits=4):
    w = wl.make_workload(batch, head_q, head_k, dim, dim, seq_k, dtype, seed=seed, varlen=varlen, is_alibi=is_alibi)
    g = torch.Generator().manual_seed(seed + 70)
    rows, ng = w.k.shape[0], dim // 64

    def spread(x, offset):  # every run of 64 of every row: its own spread and offset
        x = x.float().unflatten(-1, (ng, 64))
        x = x * (0.3 + 1.5 * torch.rand(rows, head_k, ng, 1, generator=g)) + offset * torch.randn(rows, head_k, ng, 1, generator=g)
        return x.flatten(-2)

    quant = quantize_int4_per_group if bits == 4 else quantize_int8_per_group
    k4, kp = quant(spread(w.k, 1.0))
    v4, vp = quant(spread(w.v, 0.5))
    return w, k4, v4, kp, vp


def _dequant(cache, pairs):
    n = (_unpack(cache) if cache.dtype == torch.uint8 else cache).double().unflatten(-1, (pairs.shape[-2], 64))
    return (pairs[..., :1].double() * (n - pairs[..., 1:].double())).flatten(-2)


def _reference(w, k4, v4, kp, vp):
    return torch.from_numpy(oracle.attn_f64(w.q, _dequant(k4, kp), _dequant(v4, vp), w.cu_seq_k, w.dim_v,
                                            w.is_alibi)).float()


def _run(w, k4, v4, kp, vp, q=None):
    o = decoding_attn_fwd((w.q if q is None else q).to(DEV), k4.to(DEV), v4.to(DEV), w.cu_seq_k.to(DEV), w.max_seq_k,
                          w.dim_v, w.is_alibi, k_scale=kp.to(DEV), v_scale=vp.to(DEV))
    torch.cuda.synchronize()
    return o.cpu()


SHAPES = [
    # batch, head_q, head_k, dim, seq_k
    (5, 8, 8, 128, 700),       # MHA: one live head per group, one wave per KV head
    (3, 4, 2, 128, 333),       # ratio 2, two KV heads: the four waves share a KV head's tokens
    (6, 32, 8, 128, 1500),     # GQA, one wave per KV head
    (4, 32, 1, 128, 1200),     # MQA: 32 heads per group
    (3, 16, 4, 64, 900),       # d 64: one run per row, the per-token kernel
    (2, 16, 4, 256, 500),      # d 256: four runs
    (2, 32, 1, 256, 400),      # d 256, 32 heads over one KV head: two groups of 16
    (2, 32, 32, 256, 300),     # MHA d 256
    (1, 8, 2, 128, 1),         # a single token
    (64, 32, 8, 128, 2048),    # a full grid, split sequences (ragged: the balanced grid)
]


@pytest.mark.gpu
@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", SHAPES)
def test_per_group_cache_matches_float64_attention(shape, dtype, bits):
    w, k4, v4, kp, vp = _case(*shape, dtype, is_alibi=shape[0] == 6, bits=bits)
    o = _run(w, k4, v4, kp, vp)
    assert torch.isfinite(o.float()).all()
    if w.batch > 8:  # the large case: sampled sequences against float64
        rows = [0, 1, w.batch // 2, w.batch - 1]
        cu = w.cu_seq_k.tolist()
        cat = lambda t: torch.cat([t[cu[b]:cu[b + 1]] for b in rows])  # noqa: E731
        ref = _reference(sub_workload(w, rows), cat(k4), cat(v4), cat(kp), cat(vp))
        err = (o[rows].float() - ref).abs().max().item()
    else:
        ref = _reference(w, k4, v4, kp, vp)
        err = (o.float() - ref).abs().max().item()
    # (outputs reach 2 to 5 here, where rounding the exact result to 16 bits already costs half the tolerance or
    # more: the tolerance is taken relative to the largest output)
    top = ref.abs().max().item()
    assert err <= TOL[dtype] * max(1.0, top), f"max-abs {err:.3e}, largest output {top:.2f}"
    assert top > 20 * TOL[dtype]


@pytest.mark.gpu
@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_runs_with_a_scale_of_zero(dtype, bits):
    """A constant run may come with a scale of exactly zero: a run of zeros, whose row still counts in the sums."""
    w, k4, v4, kp, vp = _case(3, 16, 4, 128, 400, dtype, seed=41, bits=bits)
    g = torch.Generator().manual_seed(4)
    kp[torch.rand(kp.shape[:3], generator=g) < 0.2, 0] = 0.0
    vp[torch.rand(vp.shape[:3], generator=g) < 0.2, 0] = 0.0
    o = _run(w, k4, v4, kp, vp)
    assert torch.isfinite(o.float()).all()
    assert (o.float() - _reference(w, k4, v4, kp, vp)).abs().max().item() <= TOL[dtype]


def _swap_runs(x, ng, unit):
    """Runs of `unit` entries of the last dimension in reverse order."""
    return x.unflatten(-1, (ng, unit)).flip(-2).flatten(-2)


@pytest.mark.gpu
@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("dim", [128, 256])
def test_exchanging_runs(dim, bits):
    w, k4, v4, kp, vp = _case(3, 16, 4, dim, 600, torch.float16, seed=31, bits=bits)
    ng = dim // 64
    unit = 32 if bits == 4 else 64  # cache entries per run
    base = _run(w, k4, v4, kp, vp)
    # V: the output's column runs follow, bit for bit (each run's columns see the same arithmetic wherever they sit)
    o = _run(w, k4, _swap_runs(v4, ng, unit), kp, vp.flip(-2).contiguous())
    assert torch.equal(_swap_runs(o, ng, 64).view(torch.int16), base.view(torch.int16))
    # K with q: the same scores (summed over the runs in another order)
    o = _run(w, _swap_runs(k4, ng, unit), v4, kp.flip(-2).contiguous(), vp, q=_swap_runs(w.q, ng, 64))
    assert (o.float() - base.float()).abs().max().item() <= TOL[torch.float16] / 4


@pytest.mark.gpu
@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_equal_pairs_in_every_run_reduce_to_the_per_token_call(dtype, bits):
    w = wl.make_workload(4, 32, 8, 128, 128, 1000, dtype, seed=5, varlen=True)
    quant = quantize_int4_per_token if bits == 4 else quantize_int8_per_token
    k4, kp = quant(w.k)
    v4, vp = quant(w.v)
    per_token = _run(w, k4, v4, kp, vp)
    twice = lambda p: p.unsqueeze(-2).expand(-1, -1, 2, -1).contiguous()  # noqa: E731
    per_group = _run(w, k4, v4, twice(kp), twice(vp))
    assert (per_group.float() - per_token.float()).abs().max().item() <= TOL[dtype] / 4


@pytest.mark.gpu
@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("shape", [SHAPES[0], SHAPES[2], SHAPES[5]])
def test_paged_pools(shape, bits):
    """Pairs in pools of their own, [pages, page_size, head_k, dim / 64, 2], addressed through the same block table:
    float64 attention on the de-quantised rows at 64-token pages, and the same bits at every page size."""
    w, k4, v4, kp, vp = _case(*shape, torch.float16, seed=21, bits=bits)
    w4 = wl.Workload(w.name, w.q, k4, v4, w.cu_seq_k, w.max_seq_k, w.dim_v, w.is_alibi, w.lengths)
    flat = lambda p: p.flatten(-2)  # noqa: E731  (to_pages handles [rows, head_k, x])
    wp = wl.Workload(w.name, w.q, flat(kp), flat(vp), w.cu_seq_k, w.max_seq_k, w.dim_v, w.is_alibi, w.lengths)
    ng = shape[3] // 64
    outs = {}
    for page_size in (64, 16, 4, 1):
        pk = wl.to_pages(w4, page_size, seed=2, poison=False).to(DEV)
        pp = wl.to_pages(wp, page_size, seed=2).to(DEV)  # (same seed: same page numbering; unused entries are NaN)
        assert torch.equal(pk.block_table, pp.block_table)
        outs[page_size] = decoding_attn_paged_fwd(w.q.to(DEV), pk.k_pages, pk.v_pages, pk.block_table, pk.seq_lens,
                                                  w.max_seq_k, w.dim_v, False,
                                                  k_scale=pp.k_pages.unflatten(-1, (ng, 2)),
                                                  v_scale=pp.v_pages.unflatten(-1, (ng, 2))).cpu()
    assert (outs[64].float() - _reference(w, k4, v4, kp, vp)).abs().max().item() <= TOL[torch.float16]
    for page_size in (16, 4, 1):
        assert torch.equal(outs[page_size].view(torch.int16), outs[64].view(torch.int16)), page_size


def test_plan_takes_sixteen_heads_a_group_at_256():
    """Four sets of factors for 32 heads do not fit a wave's registers: d = 256 runs as groups of 16 heads."""
    assert _lib.plan(1024, 8, 32, 1, 256, 256, kv_bits=_lib.KV_BITS_INT4_GROUP64)["heads_per_group"] == 16
    assert _lib.plan(1024, 8, 32, 1, 256, 256, kv_bits=_lib.KV_BITS_INT8_GROUP64)["heads_per_group"] == 16
    assert _lib.plan(1024, 8, 32, 1, 256, 256, kv_bits=_lib.KV_BITS_INT4_PER_TOKEN)["heads_per_group"] == 32
    assert _lib.plan(1024, 8, 32, 1, 128, 128, kv_bits=_lib.KV_BITS_INT4_GROUP64)["heads_per_group"] == 32


@pytest.mark.gpu
def test_argument_errors():
    w, k4, v4, kp, vp = _case(2, 8, 2, 128, 100, torch.float16)
    q, cu = w.q.to(DEV), w.cu_seq_k.to(DEV)
    k8 = _unpack(k4).float().to(torch.float8_e4m3fn).to(DEV)
    with pytest.raises(RuntimeError, match="int4 or int8 K/V cache only"):
        decoding_attn_fwd(q, k8, k8, cu, w.max_seq_k, 128, False, k_scale=kp.to(DEV), v_scale=vp.to(DEV))
    with pytest.raises(RuntimeError, match="same form"):
        decoding_attn_fwd(q, k4.to(DEV), v4.to(DEV), cu, w.max_seq_k, 128, False, k_scale=kp.to(DEV),
                          v_scale=vp[:, :, 0].contiguous().to(DEV))
    with pytest.raises(RuntimeError, match="dim / 64"):
        decoding_attn_fwd(q, k4.to(DEV), v4.to(DEV), cu, w.max_seq_k, 128, False, k_scale=kp[:, :, :1].contiguous().to(DEV),
                          v_scale=vp[:, :, :1].contiguous().to(DEV))
