"""Pins the CPU oracle (oracle/attn_cpu.c) without the reference: the reference holds no golden
vectors, so every check here is against something the mathematics fixes — a float64 textbook
attention, torch's own CPU attention, head-expansion / slicing identities, closed forms and
round-to-nearest-even tie cases — each chosen so that a dropped term, a wrong index or a wrong sign
fails at least one of them."""
import math

import numpy as np
import pytest
import torch

from decoding_attention_amd.workloads import get_cu_seq, make_workload
from oracle import oracle

DTYPES = [torch.float16, torch.bfloat16]
TOL = {torch.float16: 2e-3, torch.bfloat16: 1e-2}


def _run(w, **kw):
    return oracle.attn_cpu(w.q, w.k, w.v, w.cu_seq_k, w.max_seq_k, w.dim_v, w.is_alibi, **kw)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hq,hk,d", [(4, 4, 64), (8, 2, 128), (6, 3, 96), (4, 1, 256)])
def test_fp32_result_matches_float64_textbook(dtype, hq, hk, d):
    w = make_workload(3, hq, hk, d, d, 37, dtype, seed=1, varlen=True)
    o, o32 = _run(w, return_f32=True)
    ref = oracle.attn_f64(w.q, w.k, w.v, w.cu_seq_k, w.dim_v, False)
    # fp32 accumulation over <= 256 + 37 terms: 1e-5 is far below the output rounding step
    assert np.abs(o32.numpy().astype(np.float64) - ref).max() < 1e-5
    assert np.abs(o.to(torch.float64).numpy() - ref).max() <= TOL[dtype]


@pytest.mark.parametrize("dtype", DTYPES)
def test_matches_torch_sdpa_cpu(dtype):
    w = make_workload(2, 8, 8, 64, 64, 50, dtype, seed=2)
    _, o32 = _run(w, return_f32=True)
    q4 = w.q.float().reshape(2, 1, 8, 64).transpose(1, 2)
    k4 = w.k.float().reshape(2, 50, 8, 64).transpose(1, 2)
    v4 = w.v.float().reshape(2, 50, 8, 64).transpose(1, 2)
    ref = torch.nn.functional.scaled_dot_product_attention(q4, k4, v4).transpose(1, 2).reshape(2, 8, 64)
    assert (o32 - ref).abs().max().item() < 1e-5


def test_reference_test_recipe_mean_abs_bar():
    """The reference's own test recipe (GQA by repeat_interleave, matmul, softmax, matmul in the input
    dtype; tests/test_decoding_attn.py:35-57) and its bar (mean abs diff <= 5e-3, :94)."""
    for dtype in DTYPES:
        w = make_workload(2, 32, 8, 128, 128, 128, dtype, seed=3)
        o = _run(w)
        q4 = w.q.reshape(2, 1, 32, 128).transpose(1, 2)
        k4 = w.k.reshape(2, 128, 8, 128).transpose(1, 2).repeat_interleave(4, dim=1)
        v4 = w.v.reshape(2, 128, 8, 128).transpose(1, 2).repeat_interleave(4, dim=1)
        s = torch.matmul(q4, k4.transpose(-2, -1)) / math.sqrt(128)
        p = torch.nn.functional.softmax(s, dim=-1)
        ref = torch.matmul(p, v4).transpose(1, 2).reshape(2, 32, 128)
        assert (ref.float() - o.float()).abs().mean().item() <= 5e-3


@pytest.mark.parametrize("dtype", DTYPES)
def test_gqa_equals_mha_on_repeated_heads(dtype):
    w = make_workload(2, 8, 2, 64, 64, 19, dtype, seed=4)
    o = _run(w)
    k_rep = w.k.repeat_interleave(4, dim=1)
    v_rep = w.v.repeat_interleave(4, dim=1)
    o_mha = oracle.attn_cpu(w.q, k_rep, v_rep, w.cu_seq_k, w.max_seq_k, 64, False)
    assert torch.equal(o.view(torch.int16), o_mha.view(torch.int16))


@pytest.mark.parametrize("dtype", DTYPES)
def test_latent_equals_mqa_with_sliced_values(dtype):
    w = make_workload(2, 16, 1, 576, 512, 23, dtype, seed=5)
    assert w.v is None
    o = _run(w)
    assert o.shape == (2, 16, 512)
    v = w.k[..., :512].contiguous()
    o_sep = oracle.attn_cpu(w.q, w.k, v, w.cu_seq_k, w.max_seq_k, 512, False)
    assert torch.equal(o.view(torch.int16), o_sep.view(torch.int16))
    ref = oracle.attn_f64(w.q, w.k, None, w.cu_seq_k, 512, False)
    assert np.abs(o.to(torch.float64).numpy() - ref).max() <= TOL[dtype]


def test_varlen_equals_per_sequence_runs_and_is_independent():
    w = make_workload(5, 4, 2, 64, 64, 40, torch.float16, seed=6, varlen=True)
    o = _run(w)
    cu = w.cu_seq_k.tolist()
    for b in range(5):
        kb, vb = w.k[cu[b]:cu[b + 1]], w.v[cu[b]:cu[b + 1]]
        ob = oracle.attn_cpu(w.q[b:b + 1], kb, vb, torch.tensor([0, kb.shape[0]], dtype=torch.int32), kb.shape[0],
                             64, False)
        assert torch.equal(ob.view(torch.int16), o[b:b + 1].view(torch.int16))
    # changing one sequence's keys must not touch another sequence's output
    k2 = w.k.clone()
    k2[cu[2]:cu[3]] = -k2[cu[2]:cu[3]]
    o2 = oracle.attn_cpu(w.q, k2, w.v, w.cu_seq_k, w.max_seq_k, 64, False)
    for b in (0, 1, 3, 4):
        assert torch.equal(o2[b].view(torch.int16), o[b].view(torch.int16))
    assert not torch.equal(o2[2].view(torch.int16), o[2].view(torch.int16))


def test_alibi_closed_form_geometric_series():
    """q = 0 and ALiBi on: p_j is proportional to exp(slope*(j-(n-1))), a geometric series; with V[j] = one-hot
    style ramps the output has a closed form."""
    n, hq, d = 33, 8, 64
    q = torch.zeros(1, hq, d, dtype=torch.float16)
    k = torch.randn(n, 1, d, generator=torch.Generator().manual_seed(7)).to(torch.float16)
    v = torch.zeros(n, 1, d, dtype=torch.float16)
    v[:, 0, 0] = 1.0                                      # column 0: sum of p = 1
    v[:, 0, 1] = torch.arange(n, dtype=torch.float32).to(torch.float16)  # column 1: E[j]
    v[n - 1, 0, 2] = 1.0                                  # column 2: p_{n-1}
    cu = torch.tensor([0, n], dtype=torch.int32)
    _, o32 = oracle.attn_cpu(q, k, v, cu, n, d, True, return_f32=True)
    for h in range(hq):
        slope = 2.0 ** (-8.0 * (h + 1) / hq)
        r = math.exp(-slope)  # p_{n-1-i} proportional to r^i
        z = (1 - r ** n) / (1 - r)
        e_j = sum((n - 1 - i) * r ** i for i in range(n)) / z
        assert abs(o32[0, h, 0].item() - 1.0) < 1e-5
        assert abs(o32[0, h, 1].item() - e_j) < 1e-3 * max(1.0, e_j)
        assert abs(o32[0, h, 2].item() - 1.0 / z) < 1e-5


def test_alibi_matches_float64_and_custom_slopes():
    w = make_workload(2, 8, 2, 64, 64, 29, torch.float16, seed=8, varlen=True, is_alibi=True)
    _, o32 = _run(w, return_f32=True)
    ref = oracle.attn_f64(w.q, w.k, w.v, w.cu_seq_k, 64, True)
    assert np.abs(o32.numpy() - ref).max() < 1e-5
    slopes = np.linspace(0.01, 0.5, 8).astype(np.float32)
    _, o32s = _run(w, alibi_slopes=slopes, return_f32=True)
    refs = oracle.attn_f64(w.q, w.k, w.v, w.cu_seq_k, 64, True, alibi_slopes=slopes)
    assert np.abs(o32s.numpy() - refs).max() < 1e-5
    assert np.abs(refs - ref).max() > 1e-3  # the slopes matter


def test_softmax_scale_argument_and_linearity_in_q():
    w = make_workload(2, 4, 4, 64, 64, 21, torch.float16, seed=9)
    _, o_a = _run(w, softmax_scale=0.25, return_f32=True)
    q2 = (w.q.float() * 2).to(torch.float16)  # exact in fp16
    _, o_b = oracle.attn_cpu(q2, w.k, w.v, w.cu_seq_k, w.max_seq_k, 64, False, softmax_scale=0.125,
                             return_f32=True)
    assert (o_a - o_b).abs().max().item() < 1e-5
    ref = oracle.attn_f64(w.q, w.k, w.v, w.cu_seq_k, 64, False, softmax_scale=0.25)
    assert np.abs(o_a.numpy() - ref).max() < 1e-5


@pytest.mark.parametrize("dtype", DTYPES)
def test_special_cases(dtype):
    g = torch.Generator().manual_seed(10)
    d = 64
    # len == 1: the output is V[0], bit for bit
    q = torch.randn(3, 2, d, generator=g).to(dtype)
    k = torch.randn(3, 2, d, generator=g).to(dtype)
    v = torch.randn(3, 2, d, generator=g).to(dtype)
    cu = torch.tensor([0, 1, 2, 3], dtype=torch.int32)
    o = oracle.attn_cpu(q, k, v, cu, 1, d, False)
    assert torch.equal(o.view(torch.int16), v.view(torch.int16))
    # q == 0: uniform weights, the output is the mean of V
    n = 16
    q0 = torch.zeros(1, 2, d, dtype=dtype)
    k = torch.randn(n, 2, d, generator=g).to(dtype)
    v = torch.randn(n, 2, d, generator=g).to(dtype)
    cu = torch.tensor([0, n], dtype=torch.int32)
    _, o32 = oracle.attn_cpu(q0, k, v, cu, n, d, False, return_f32=True)
    assert (o32[0] - v.float().mean(dim=0)).abs().max().item() < 1e-6
    # one key = large multiple of q: the softmax picks that row
    qv = torch.randn(1, 2, d, generator=g).to(dtype)
    k2 = k.clone()
    k2[5] = (qv[0].float() * 8).to(dtype)
    _, o32 = oracle.attn_cpu(qv, k2, v, cu, n, d, False, return_f32=True)
    assert (o32[0] - v[5].float()).abs().max().item() < 1e-3
    # empty sequence: zeros (documented choice; the reference leaves the row untouched)
    cu = torch.tensor([0, 0, n], dtype=torch.int32)
    q2 = torch.randn(2, 2, d, generator=g).to(dtype)
    o = oracle.attn_cpu(q2, k, v, cu, n, d, False)
    assert (o[0].float() == 0).all() and o[1].float().abs().max() > 0


def test_output_rounding_is_nearest_even():
    # hand-picked ties and neighbours; torch's casts are the library reference for RNE
    vals = [1.0, 1.0 + 2 ** -11, 1.0 + 2 ** -11 + 2 ** -20, 1.0 + 3 * 2 ** -11, 65504.0, 65519.9, 65520.0, 1e-8,
            2 ** -24, 2 ** -25, 2 ** -25 + 2 ** -40, 3 * 2 ** -25, -0.3333333, 6.1e-5, 5.9604645e-8, 1e5,
            1.0 + 2 ** -8, 1.0 + 2 ** -8 + 2 ** -16, 1.0 + 3 * 2 ** -8, 3.3895314e38, float("inf"), -float("inf")]
    rng = np.random.default_rng(0)
    vals += list(rng.standard_normal(2000).astype(np.float32))
    vals += list((rng.standard_normal(500) * 1e-6).astype(np.float32))
    for x in vals:
        x = float(np.float32(x))
        t = torch.tensor([x], dtype=torch.float32)
        h = t.to(torch.float16).view(torch.int16).item() & 0xFFFF
        b = t.to(torch.bfloat16).view(torch.int16).item() & 0xFFFF
        assert oracle.f32_to_f16_bits(x) == h, x
        assert oracle.f32_to_bf16_bits(x) == b, x
    for bits in list(range(0, 0x7C01)) + [0x8000, 0xFBFF, 0x83FF]:
        f = oracle.f16_bits_to_f32(bits)
        want = torch.tensor([bits], dtype=torch.int32).to(torch.int16).view(torch.float16).float().item()
        assert f == want
    for bits in (0x3F80, 0x0001, 0x7F7F, 0xC2F7, 0x0080):
        want = torch.tensor([bits if bits < 0x8000 else bits - 0x10000], dtype=torch.int16).view(torch.bfloat16)
        assert oracle.bf16_bits_to_f32(bits) == want.float().item()


def test_threads_do_not_change_bits():
    w = make_workload(4, 8, 2, 128, 128, 64, torch.bfloat16, seed=11, varlen=True)
    o1 = _run(w, nthreads=1)
    o4 = _run(w, nthreads=4)
    assert torch.equal(o1.view(torch.int16), o4.view(torch.int16))


def test_rejects_what_the_reference_rejects():
    w = make_workload(1, 4, 4, 64, 64, 8, torch.float16, seed=12)
    with pytest.raises(ValueError):
        oracle.attn_cpu(w.q, w.k[:, :3].contiguous(), w.v[:, :3].contiguous(), w.cu_seq_k, 8, 64, False)


def test_get_cu_seq_layout():
    cu = get_cu_seq(torch.tensor([3, 5, 1], dtype=torch.int32))
    assert cu.dtype == torch.int32 and cu.tolist() == [0, 3, 8, 9]
