"""int4 K/V cache: q and o stay 16-bit, K/V are two's-complement four-bit integers (-8 .. 7), two to a byte (element
2 i in the low half of byte i), with one symmetric scale per KV head.

Every value converts exactly to fp16 and to bf16; the call is checked against float64 attention on the de-quantised
inputs at the usual tolerance (max-abs 2e-3 fp16 / 1e-2 bf16) and against the int8 call on the same integers (the same
bits on the VALU sweep, within a quarter of the tolerance on the grouped kernel, whose int4 conversion adds a bias
that its sums take out again).  The packing
helper is checked on the CPU against a per-element restatement of the layout.
"""
import pytest
import torch

from decoding_attention_amd import _lib, decoding_attn_fwd, decoding_attn_paged_fwd, pack_int4
from decoding_attention_amd import workloads as wl
from oracle import oracle
from tests.gpu_util import TOL, sub_workload

DEV = "cuda:0"


def test_pack_int4_layout():
    """Element 2 i in bits 0 .. 3 of byte i, element 2 i + 1 in bits 4 .. 7, two's complement; all 16 values."""
    x = torch.tensor([[-8, -7, -1, 0, 1, 7, 3, -4], [5, -8, 7, 7, -1, -1, 0, 0]], dtype=torch.int8)
    p = pack_int4(x)
    assert p.dtype == torch.uint8 and p.shape == (2, 4)
    for r in range(2):
        for i in range(4):
            lo, hi = int(p[r, i]) & 15, int(p[r, i]) >> 4
            assert (lo - 16 if lo >= 8 else lo) == int(x[r, 2 * i])
            assert (hi - 16 if hi >= 8 else hi) == int(x[r, 2 * i + 1])
    with pytest.raises(ValueError):
        pack_int4(torch.zeros(3, 5, dtype=torch.int8))


def _quantise(x, scale):
    """round(x / scale[head]) clamped to -8 .. 7; scale is a float32 [head_k] tensor."""
    return torch.round(x.float() / scale.view(1, -1, 1)).clamp(-8, 7).to(torch.int8)


def _case(batch, head_q, head_k, dim, dim_v, seq_k, dtype, *, latent=False, is_alibi=False, seed=3):
    w = wl.make_workload(batch, head_q, head_k, dim, dim_v, seq_k, dtype, seed=seed, varlen=True, is_alibi=is_alibi,
                         latent=latent if latent else None)
    g = torch.Generator().manual_seed(seed + 100)
    ks = (2.5 + torch.rand(head_k, generator=g)) / 7  # N(0,1) data: 2.5 .. 3.5 sigma at full scale, the rest clamps
    vs = (2.5 + torch.rand(head_k, generator=g)) / 7
    k4 = _quantise(w.k, ks)
    v4 = None if w.v is None else _quantise(w.v, vs)
    # every value of the range occurs
    k4.view(-1)[:16] = torch.arange(-8, 8, dtype=torch.int8)
    return w, k4, v4, ks, vs


def _reference(w, k4, v4, ks, vs, **kw):
    k_deq = k4.float() * ks.view(1, -1, 1)
    v_deq = None if v4 is None else v4.float() * vs.view(1, -1, 1)  # None: V is the leading columns of K
    return torch.from_numpy(oracle.attn_f64(w.q, k_deq, v_deq, w.cu_seq_k, w.dim_v, w.is_alibi, **kw)).float()


def _run(w, k4, v4, ks, vs, scales=True, **extra):
    kw = dict(k_scale=ks.to(DEV), v_scale=vs.to(DEV)) if scales else {}
    kw.update(extra)
    o = decoding_attn_fwd(w.q.to(DEV), pack_int4(k4).to(DEV), None if v4 is None else pack_int4(v4).to(DEV),
                          w.cu_seq_k.to(DEV), w.max_seq_k, w.dim_v, w.is_alibi, **kw)
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
    (64, 32, 8, 128, 128, 2048),   # a full grid of the grouped kernel, split sequences
]


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", SHAPES)
def test_int4_kv_with_scales_matches_float64_attention(shape, dtype):
    w, k4, v4, ks, vs = _case(*shape, dtype)
    o = _run(w, k4, v4, ks, vs)
    assert torch.isfinite(o.float()).all()
    rows = list(range(w.batch)) if w.batch <= 8 else [0, 1, w.batch // 2, w.batch - 1]
    if w.batch > 8:  # the large case: sampled sequences against float64
        cu = w.cu_seq_k.tolist()
        ws = sub_workload(w, rows)
        k4s = torch.cat([k4[cu[b]:cu[b + 1]] for b in rows])
        v4s = torch.cat([v4[cu[b]:cu[b + 1]] for b in rows])
        err = (o[rows].float() - _reference(ws, k4s, v4s, ks, vs)).abs().max().item()
    else:
        err = (o.float() - _reference(w, k4, v4, ks, vs)).abs().max().item()
    assert err <= TOL[dtype], f"max-abs {err:.3e}"


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", [SHAPES[0], SHAPES[2], SHAPES[3], SHAPES[5], SHAPES[6]])
def test_int4_equals_int8_on_the_same_integers(shape, dtype):
    """The same integers as an int8 cache.  On the VALU sweep the nibbles are widened to sixteen times their value, a
    power of two divided out of the per-head factors: the same bits as the int8 call.  On the grouped kernel the
    nibbles enter the matrix instructions with a bias that the kernel takes out of its sums again (exact products,
    fp32 sums in another order): a quarter of the acceptance tolerance."""
    w, k4, v4, ks, vs = _case(*shape, dtype)
    o4 = _run(w, k4, v4, ks, vs)
    o8 = decoding_attn_fwd(w.q.to(DEV), k4.to(DEV), v4.to(DEV), w.cu_seq_k.to(DEV), w.max_seq_k, w.dim_v, w.is_alibi,
                           k_scale=ks.to(DEV), v_scale=vs.to(DEV)).cpu()
    batch, head_q, head_k, dim, dim_v, _ = shape
    kind = _lib.plan(w.max_seq_k, batch, head_q, head_k, dim, dim_v, total_k=int(k4.shape[0]), kv_bits=4)["kind"]
    if kind == 1:
        assert torch.equal(o4.view(torch.int16), o8.view(torch.int16))
    else:
        assert (o4.float() - o8.float()).abs().max().item() <= TOL[dtype] / 4


@pytest.mark.gpu
@pytest.mark.parametrize("dim", [64, 128])
def test_mha_over_int4_takes_the_grouped_kernel_from_2_17_rows(dim):
    """One query head per KV head: the matrix kernel (one live head in sixteen) still beats the VALU sweep's
    nibble conversion once the problem is large enough for its launch to pay."""
    assert _lib.plan(256, 40, 32, 32, dim, dim, total_k=40 * 256, kv_bits=4)["kind"] == 3
    assert _lib.plan(256, 8, 32, 32, dim, dim, total_k=8 * 256, kv_bits=4)["kind"] == 1
    assert _lib.plan(256, 40, 32, 32, dim, dim, total_k=40 * 256, kv_bits=8)["kind"] == 1
    w, k4, v4, ks, vs = _case(40, 32, 32, dim, dim, 256, torch.float16, seed=31)
    o = _run(w, k4, v4, ks, vs)
    rows = [0, 13, 39]
    cu = w.cu_seq_k.tolist()
    k4s = torch.cat([k4[cu[b]:cu[b + 1]] for b in rows])
    v4s = torch.cat([v4[cu[b]:cu[b + 1]] for b in rows])
    err = (o[rows].float() - _reference(sub_workload(w, rows), k4s, v4s, ks, vs)).abs().max().item()
    assert torch.isfinite(o.float()).all() and err <= TOL[torch.float16]


@pytest.mark.gpu
def test_alibi_and_softmax_scale_with_int4_kv():
    w, k4, v4, ks, vs = _case(4, 32, 1, 128, 128, 800, torch.float16, is_alibi=True)
    o = _run(w, k4, v4, ks, vs, softmax_scale=0.05)
    ref = _reference(w, k4, v4, ks, vs, softmax_scale=0.05)
    assert (o.float() - ref).abs().max().item() <= TOL[torch.float16]


@pytest.mark.gpu
@pytest.mark.parametrize("batch,head_q,seq_k", [(3, 8, 700), (3, 16, 700), (3, 32, 700), (3, 100, 700), (16, 128, 2048)])
def test_latent_form_with_int4_cache(batch, head_q, seq_k):
    """(576, 512) with V = K[..., :512]: the grouped kernel's latent form, ceil(heads / 16) groups per sequence, at
    every head count and size (the latent kernel has no int4 form)."""
    w, k4, _, ks, _ = _case(batch, head_q, 1, 576, 512, seq_k, torch.float16, latent=True, seed=head_q)
    o = _run(w, k4, None, ks, ks)
    rows = list(range(min(batch, 4)))
    cu = w.cu_seq_k.tolist()
    ws = sub_workload(w, rows)
    k4s = torch.cat([k4[cu[b]:cu[b + 1]] for b in rows])
    assert torch.isfinite(o.float()).all()
    assert (o[rows].float() - _reference(ws, k4s, None, ks, ks)).abs().max().item() <= TOL[torch.float16]


@pytest.mark.gpu
@pytest.mark.parametrize("page_size", [1, 8, 16, 64])
@pytest.mark.parametrize("shape", [SHAPES[0], SHAPES[2], SHAPES[3]])
def test_paged_int4(shape, page_size):
    """Page pools of packed nibbles (page strides are counted in elements, two to a byte)."""
    w, k4, v4, ks, vs = _case(*shape, torch.float16, seed=21)
    w4 = wl.Workload(w.name, w.q, pack_int4(k4), pack_int4(v4), w.cu_seq_k, w.max_seq_k, w.dim_v, w.is_alibi, w.lengths)
    pk = wl.to_pages(w4, page_size, seed=2, poison=False).to(DEV)
    o = decoding_attn_paged_fwd(w.q.to(DEV), pk.k_pages, pk.v_pages, pk.block_table, pk.seq_lens, w.max_seq_k,
                                w.dim_v, False, k_scale=ks.to(DEV), v_scale=vs.to(DEV)).cpu()
    assert (o.float() - _reference(w, k4, v4, ks, vs)).abs().max().item() <= TOL[torch.float16]
