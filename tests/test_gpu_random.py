"""Randomised differential test: every path of the library (packed with and without the token-count hint, paged with
pages of 1..128 tokens, FP8 and int8 caches, the latent form, ALiBi, ragged and empty sequences) against float64
attention on a sample of rows.  Shapes, layouts and options are drawn from a fixed seed, so a failure names its case.

The tolerance is the acceptance bar scaled by the magnitude of the result: a bf16 output of magnitude 2..4 is only
representable to 0.0078, so the absolute bar of 1e-2 is widened in proportion when |o| > 1.
"""
import random

import pytest
import torch

from decoding_attention_amd import (decoding_attn_fwd, decoding_attn_paged_fwd, pack_int4, quantize_int4_per_group,
                                    quantize_int4_per_token, quantize_int8_per_group, quantize_int8_per_token)
from decoding_attention_amd import workloads as wl
from oracle import oracle
from tests.gpu_util import TOL, run_hip_ex, sub_workload

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
FP8 = torch.float8_e4m3fn
HEADS = [(32, 8), (32, 32), (32, 1), (8, 2), (28, 4), (16, 16), (64, 8), (12, 4), (40, 8), (4, 1), (6, 3), (64, 2)]
CASES_PER_CHUNK = 12


def _one_case(rng, seed, case, int4=False, per_token=False, per64=False):
    """int4: the case runs over an int4 cache (whatever format the draws below pick; the stream of draws is the same
    either way, so the other cases do not move).  per_token (4 or 8): an int4 or int8 cache with a (scale, zero) pair
    per token and KV head (never the latent form, never d = 96, which those entry points do not serve); with per64 the
    pairs are per run of 64 elements of each row."""
    latent = rng.random() < 0.3 and not per_token
    dtype = rng.choice([torch.float16, torch.bfloat16])
    if latent:
        hq, hk, d, dv = rng.choice([16, 32, 64, 128, 96, 8]), 1, 576, 512
    else:
        hq, hk = rng.choice(HEADS)
        d = dv = rng.choice([64, 96, 128, 256])
        if per_token and d == 96:
            d = dv = 128
    batch = rng.choice([1, 2, 3, 5, 8, 17, 40, 90])
    maxlen = rng.choice([5, 33, 100, 300, 777, 1500, 3000, 6000])
    if batch * maxlen * hk * d > 1.5e8:
        maxlen = max(5, int(1.5e8 / (batch * hk * d)))
    g = torch.Generator().manual_seed(seed * 100003 + case)
    mode = rng.choice(["fixed", "ragged", "ragged0"])
    if mode == "fixed":
        lens = torch.full((batch,), maxlen, dtype=torch.int32)
    else:
        lens = torch.randint(1, maxlen + 1, (batch,), generator=g, dtype=torch.int32)
        if mode == "ragged0" and batch > 1:
            lens[torch.rand(batch, generator=g) < 0.2] = 0
        if int(lens.max()) == 0:
            lens[0] = maxlen
    alibi = rng.random() < 0.3
    total = int(lens.sum())
    q = torch.randn(batch, hq, d, generator=g).to(dtype)
    k = torch.randn(total, hk, d, generator=g).to(dtype)
    v = None if latent else torch.randn(total, hk, dv, generator=g).to(dtype)
    fp8 = rng.random() < 0.35
    layout = rng.choice(["packed", "packed_nohint", "paged"])
    page = rng.choice([1, 8, 16, 32, 64, 128])
    int8 = fp8 and rng.random() < 0.4  # the 8-bit cache holds int8 instead of FP8
    kv8_dtype = torch.int8 if int8 else FP8
    if int4 or per_token:
        fp8, int8, kv8_dtype = True, True, torch.int8 if per_token == 8 else torch.uint8
    desc = (f"seed {seed} case {case}: latent={latent} {hq}/{hk} d{d} {dtype} b{batch} max{maxlen} {mode} "
            f"alibi={alibi} fp8={fp8} int8={int8} {layout} page={page} total={total}")
    kw, k8, v8 = {}, None, None
    k_true, v_true = k.float(), None if v is None else v.float()
    if per_token:
        # rows of different spread and offset: the pairs differ from token to token and head to head
        runs = d // 64 if per64 else 1  # (per64: every run of 64 elements likewise)
        shape = (total, hk, runs, 1)
        k = (k.float().unflatten(-1, (runs, -1)) * (0.5 + torch.rand(shape, generator=g))
             + torch.randn(shape, generator=g)).flatten(-2)
        v = (v.float().unflatten(-1, (runs, -1)) * (0.5 + torch.rand(shape, generator=g))
             + 0.5 * torch.randn(shape, generator=g)).flatten(-2)
        quant = {(8, False): quantize_int8_per_token, (4, False): quantize_int4_per_token,
                 (4, True): quantize_int4_per_group, (8, True): quantize_int8_per_group}[(per_token, per64)]
        k8, kpairs = quant(k)
        v8, vpairs = quant(v)
        if not per64:
            kpairs, vpairs = kpairs.unsqueeze(-2), vpairs.unsqueeze(-2)  # [total, hk, runs, 2] from here on

        def unpack(p4):
            if per_token == 8:
                return p4.double()
            n = torch.stack([(p4 & 15).to(torch.int16), (p4 >> 4).to(torch.int16)], dim=-1).flatten(-2)
            return torch.where(n >= 8, n - 16, n).double()

        k_true = (kpairs[..., :1].double() * (unpack(k8).unflatten(-1, (runs, -1)) - kpairs[..., 1:].double())).flatten(-2)
        v_true = (vpairs[..., :1].double() * (unpack(v8).unflatten(-1, (runs, -1)) - vpairs[..., 1:].double())).flatten(-2)
        as_passed = (lambda t: t) if per64 else (lambda t: t.squeeze(-2))  # noqa: E731
        kw = dict(k_scale=as_passed(kpairs).to(DEV), v_scale=as_passed(vpairs).to(DEV))
    elif fp8:
        def quantise(x, scale):
            y = x.float() / scale.view(1, -1, 1)
            if int4:
                return torch.round(y).clamp(-8, 7).to(torch.int8)
            return torch.round(y).clamp(-128, 127).to(torch.int8) if int8 else y.to(FP8)

        ks = 0.015 + 0.015 * torch.rand(hk, generator=g)
        vs = ks if latent else 0.015 + 0.015 * torch.rand(hk, generator=g)
        if int4:
            ks, vs = ks * 20, vs * 20  # sixteen levels over about three standard deviations
        k8 = quantise(k, ks)
        k_true = k8.float() * ks.view(1, -1, 1)
        if v is not None:
            v8 = quantise(v, vs)
            v_true = v8.float() * vs.view(1, -1, 1)
        kw = dict(k_scale=ks.to(DEV), v_scale=vs.to(DEV))
        if int4:  # from here on the cache is its packed bytes
            k8 = pack_int4(k8)
            v8 = None if v8 is None else pack_int4(v8)
    cu = wl.get_cu_seq(lens)
    max_seq_k = int(lens.max())
    if layout == "paged":
        src = wl.Workload("p", q, k8.view(torch.uint8) if fp8 else k,
                          None if v is None else (v8.view(torch.uint8) if fp8 else v), cu, max_seq_k, dv, alibi,
                          lens.tolist())
        pk = wl.to_pages(src, page, seed=case, poison=not fp8).to(DEV)
        if per_token:  # the pairs in pools of their own, numbered like the pages (same seed)
            pp = wl.to_pages(wl.Workload("pp", q, kpairs.flatten(-2), vpairs.flatten(-2), cu, max_seq_k, dv, alibi,
                                         lens.tolist()), page, seed=case).to(DEV)
            kw = dict(k_scale=as_passed(pp.k_pages.unflatten(-1, (runs, 2))),
                      v_scale=as_passed(pp.v_pages.unflatten(-1, (runs, 2))))
        kp = pk.k_pages.view(kv8_dtype) if fp8 else pk.k_pages
        vp = None if pk.v_pages is None else (pk.v_pages.view(kv8_dtype) if fp8 else pk.v_pages)
        o = decoding_attn_paged_fwd(q.to(DEV), kp, vp, pk.block_table, pk.seq_lens, max_seq_k, dv, alibi,
                                    total_k=rng.choice([0, total]), **kw)
    elif layout == "packed_nohint" and not fp8:
        o = run_hip_ex(wl.Workload("x", q, k, v, cu, max_seq_k, dv, alibi, lens.tolist()), 0)
    else:
        o = decoding_attn_fwd(q.to(DEV), (k8 if fp8 else k).to(DEV),
                              None if v is None else (v8 if fp8 else v).to(DEV), cu.to(DEV), max_seq_k, dv, alibi, **kw)
    torch.cuda.synchronize()
    o = o.cpu()
    assert torch.isfinite(o.float()).all(), desc
    rows = list(range(batch)) if batch <= 8 else sorted(set(rng.sample(range(batch), 8)) | {int(lens.argmax())})
    sub = sub_workload(wl.Workload("o", q.float(), k_true, v_true, cu, max_seq_k, dv, alibi, lens.tolist()), rows)
    ref = torch.from_numpy(oracle.attn_f64(sub.q, sub.k, sub.v, sub.cu_seq_k, dv, alibi)).float()
    err = (o[rows].float() - ref).abs().max().item()
    assert err <= TOL[dtype] * max(1.0, ref.abs().max().item()), f"{desc}: max-abs {err:.3e}"
    for b in range(batch):
        if int(lens[b]) == 0:
            assert torch.count_nonzero(o[b]) == 0, desc


@pytest.mark.parametrize("chunk", range(3))
def test_random_cases_over_an_int4_cache(chunk):
    seed = 11
    rng = random.Random(seed * 1000 + chunk)
    for i in range(CASES_PER_CHUNK):
        _one_case(rng, seed, chunk * CASES_PER_CHUNK + i, int4=True)


@pytest.mark.parametrize("chunk", range(3))
def test_random_cases_over_an_int4_cache_with_per_token_pairs(chunk):
    seed = 13
    rng = random.Random(seed * 1000 + chunk)
    for i in range(CASES_PER_CHUNK):
        _one_case(rng, seed, chunk * CASES_PER_CHUNK + i, per_token=4)


@pytest.mark.parametrize("chunk", range(2))
def test_random_cases_over_an_int8_cache_with_per_token_pairs(chunk):
    seed = 17
    rng = random.Random(seed * 1000 + chunk)
    for i in range(CASES_PER_CHUNK):
        _one_case(rng, seed, chunk * CASES_PER_CHUNK + i, per_token=8)


@pytest.mark.parametrize("chunk", range(8))
def test_random_cases(chunk):
    seed = 7
    rng = random.Random(seed * 1000 + chunk)
    for i in range(CASES_PER_CHUNK):
        _one_case(rng, seed, chunk * CASES_PER_CHUNK + i)


@pytest.mark.parametrize("chunk", range(3))
def test_random_cases_over_an_int4_cache_with_pairs_per_64_elements(chunk):
    seed = 19
    rng = random.Random(seed * 1000 + chunk)
    for i in range(CASES_PER_CHUNK):
        _one_case(rng, seed, chunk * CASES_PER_CHUNK + i, per_token=4, per64=True)


@pytest.mark.parametrize("chunk", range(2))
def test_random_cases_over_an_int8_cache_with_pairs_per_64_elements(chunk):
    seed = 23
    rng = random.Random(seed * 1000 + chunk)
    for i in range(CASES_PER_CHUNK):
        _one_case(rng, seed, chunk * CASES_PER_CHUNK + i, per_token=8, per64=True)
