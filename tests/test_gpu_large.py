"""K/V buffers beyond 4 GiB: byte offsets past 2^32 in every kernel's addressing.

The inputs are drawn on the GPU (drawing 4 G elements on the host would dominate the test); the sequences that are
checked are copied back and go through the CPU oracle.
"""
import pytest
import torch

from decoding_attention_amd import _lib, decoding_attn_fwd
from decoding_attention_amd import workloads as wl
from tests.gpu_util import check_against_oracle

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _check_rows(q, k, v, cu, o, rows, dim_v, name):
    cu_l = cu.tolist()
    ks = [k[cu_l[b]:cu_l[b + 1]].cpu() for b in rows]
    vs = None if v is None else [v[cu_l[b]:cu_l[b + 1]].cpu() for b in rows]
    lens = torch.tensor([x.shape[0] for x in ks], dtype=torch.int32)
    w = wl.Workload(name, q[rows].cpu(), torch.cat(ks), None if vs is None else torch.cat(vs), wl.get_cu_seq(lens),
                    int(lens.max()), dim_v, False, lens.tolist())
    check_against_oracle(w, o[rows].cpu())


@pytest.mark.parametrize("kind", ["gqa", "mha", "mla"])
def test_offsets_beyond_4_gib(kind):
    g = torch.Generator(device=DEV).manual_seed(5)
    if kind == "gqa":      # grouped MFMA kernel: 2 x 5.4 GB
        batch, hq, hk, d, dv, sk, dtype = 320, 32, 8, 128, 128, 8192, torch.bfloat16
    elif kind == "mha":    # VALU sweep (short sequences): 2 x 5.4 GB
        batch, hq, hk, d, dv, sk, dtype = 10240, 32, 32, 128, 128, 64, torch.float16
    else:                  # latent MFMA kernel: 4.8 GB
        batch, hq, hk, d, dv, sk, dtype = 512, 128, 1, 576, 512, 8192, torch.float16
    total = batch * sk
    assert total * hk * d * 2 > (1 << 32)
    q = torch.randn(batch, hq, d, generator=g, device=DEV, dtype=dtype)
    k = torch.randn(total, hk, d, generator=g, device=DEV, dtype=dtype)
    v = None if kind == "mla" else torch.randn(total, hk, dv, generator=g, device=DEV, dtype=dtype)
    cu = torch.arange(batch + 1, dtype=torch.int32) * sk
    assert _lib.plan(sk, batch, hq, hk, d, dv)["kind"] == {"gqa": 3, "mha": 1, "mla": 2}[kind]
    o = decoding_attn_fwd(q, k, v, cu.to(DEV), sk, dv, False)
    torch.cuda.synchronize()
    assert torch.isfinite(o.float()).all()
    # first, last, and the sequences on either side of the 4 GiB byte offset
    edge = (1 << 32) // (sk * hk * d * 2)
    _check_rows(q, k, v, cu, o, [0, edge - 1, edge, edge + 1, batch - 1], dv, "large_" + kind)


@pytest.mark.parametrize("kind", ["mha_ragged", "gqa_paged"])
def test_batch_beyond_one_grid_axis(kind):
    """70 000 sequences, more than a grid axis numbers (65 535; the reference numbers sequences along grid.x and has no
    such limit, csrc/kernel/decoding_attn/decoding_fwd_launch_template.h:18): the call runs as two launches.  Every row
    finite, rows on both sides of the seam and at both ends against the oracle; packed ragged MHA and paged GQA."""
    from decoding_attention_amd import decoding_attn_paged_fwd

    g = torch.Generator(device="cpu").manual_seed(9)
    batch = 70000
    seam = 65528
    rows = [0, 1, seam - 1, seam, seam + 1, batch - 1]
    if kind == "mha_ragged":
        hq, hk, d, sk, dtype = 8, 8, 64, 24, torch.float16
        lens = torch.randint(0, sk + 1, (batch,), generator=g, dtype=torch.int32)
        lens[seam] = sk
        cu = wl.get_cu_seq(lens)
        total = int(cu[-1])
        gd = torch.Generator(device=DEV).manual_seed(9)
        q = torch.randn(batch, hq, d, generator=gd, device=DEV, dtype=dtype)
        k = torch.randn(total, hk, d, generator=gd, device=DEV, dtype=dtype)
        v = torch.randn(total, hk, d, generator=gd, device=DEV, dtype=dtype)
        o = decoding_attn_fwd(q, k, v, cu.to(DEV), sk, d, False)
        torch.cuda.synchronize()
        assert torch.isfinite(o.float()).all()
        assert (o[lens.to(DEV) == 0] == 0).all()  # empty sequences: zero rows
        rows = [b for b in rows if lens[b] > 0]
        _check_rows(q, k, v, cu, o, rows, d, "batch70000_mha")
    else:
        hq, hk, d, sk, dtype, page = 16, 4, 128, 40, torch.bfloat16, 16
        lens = torch.randint(1, sk + 1, (batch,), generator=g, dtype=torch.int32)
        max_blocks = (sk + page - 1) // page
        npages = batch * max_blocks
        gd = torch.Generator(device=DEV).manual_seed(10)
        q = torch.randn(batch, hq, d, generator=gd, device=DEV, dtype=dtype)
        k_pages = torch.randn(npages, page, hk, d, generator=gd, device=DEV, dtype=dtype)
        v_pages = torch.randn(npages, page, hk, d, generator=gd, device=DEV, dtype=dtype)
        table = torch.randperm(npages, generator=g).to(torch.int32).reshape(batch, max_blocks)
        o = decoding_attn_paged_fwd(q, k_pages, v_pages, table.to(DEV), lens.to(DEV), sk, d, False)
        torch.cuda.synchronize()
        assert torch.isfinite(o.float()).all()
        ks, vs = [], []
        for b in rows:
            n = int(lens[b])
            pages = table[b, : (n + page - 1) // page].long().to(DEV)
            ks.append(k_pages[pages].reshape(-1, hk, d)[:n].cpu())
            vs.append(v_pages[pages].reshape(-1, hk, d)[:n].cpu())
        sub = torch.tensor([int(lens[b]) for b in rows], dtype=torch.int32)
        w = wl.Workload("batch70000_paged", q[rows].cpu(), torch.cat(ks), torch.cat(vs), wl.get_cu_seq(sub), int(sub.max()),
                        d, False, sub.tolist())
        check_against_oracle(w, o[rows].cpu())


def test_batch_beyond_one_grid_axis_with_per_token_pairs():
    """The same seam with an int4 cache whose rows carry their own (scale, zero) pairs: the second launch addresses
    the packed rows and their pairs by absolute row number, q and o by the run's first sequence."""
    from decoding_attention_amd import quantize_int4_per_token
    from oracle import oracle

    g = torch.Generator(device="cpu").manual_seed(19)
    batch, seam, hq, hk, d, sk = 70000, 65528, 8, 2, 64, 20
    lens = torch.randint(1, sk + 1, (batch,), generator=g, dtype=torch.int32)
    cu = wl.get_cu_seq(lens)
    total = int(cu[-1])
    gd = torch.Generator(device=DEV).manual_seed(19)
    q = torch.randn(batch, hq, d, generator=gd, device=DEV, dtype=torch.float16)
    k = torch.randn(total, hk, d, generator=gd, device=DEV) * 2 + 0.5
    v = torch.randn(total, hk, d, generator=gd, device=DEV) - 0.3
    k4, kp = quantize_int4_per_token(k)
    v4, vp = quantize_int4_per_token(v)
    o = decoding_attn_fwd(q, k4, v4, cu.to(DEV), sk, d, False, k_scale=kp, v_scale=vp)
    torch.cuda.synchronize()
    assert torch.isfinite(o.float()).all()

    def unpack(p4):
        n = torch.stack([(p4 & 15).to(torch.int16), (p4 >> 4).to(torch.int16)], dim=-1).flatten(-2)
        return torch.where(n >= 8, n - 16, n).double()

    rows = [0, 1, seam - 1, seam, seam + 1, batch - 1]
    cu_l = cu.tolist()
    sel = torch.cat([torch.arange(cu_l[b], cu_l[b + 1]) for b in rows]).to(DEV)
    kd = (kp[sel][..., :1].double() * (unpack(k4[sel]) - kp[sel][..., 1:].double())).cpu()
    vd = (vp[sel][..., :1].double() * (unpack(v4[sel]) - vp[sel][..., 1:].double())).cpu()
    sub = torch.tensor([int(lens[b]) for b in rows], dtype=torch.int32)
    ref = torch.from_numpy(oracle.attn_f64(q[rows].cpu(), kd, vd, wl.get_cu_seq(sub), d, False)).float()
    assert (o[rows].cpu().float() - ref).abs().max().item() <= 2e-3
