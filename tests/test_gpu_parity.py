"""GPU parity: the HIP path, called through the C-ABI, against the CPU oracle on the same seeded inputs.

Tolerances: max-abs <= 2e-3 (fp16) / 1e-2 (bf16) against the oracle's fp32-accumulated result, and the
reference's own bar (mean-abs <= 5e-3, reference tests/test_decoding_attn.py:94,128) against its rounded
output.  The case matrices re-author the reference's pytest grids (tests/test_decoding_attn.py:61-66,97-103)
and add what they leave out: variable lengths, ALiBi, MQA, empty and ragged sequences.
"""
import pytest
import torch

from decoding_attention_amd import _lib, decoding_attn_fwd, fwd
from decoding_attention_amd import workloads as wl
from gpu_util import TOL, check_against_oracle, run_hip, run_hip_ex, run_oracle, sub_workload

pytestmark = pytest.mark.gpu
DTYPES = [torch.float16, torch.bfloat16]


def _name(dtype):
    return "bf16" if dtype == torch.bfloat16 else "fp16"


def test_config0_mha_cpu_case():
    w = wl.config_mha_cpu_case()
    check_against_oracle(w, run_hip(w))


@pytest.mark.parametrize("dtype", DTYPES, ids=_name)
@pytest.mark.parametrize("seq_k", [1, 128, 512])
@pytest.mark.parametrize("batch", [1, 2, 16])
@pytest.mark.parametrize("dim", [64, 96, 128, 256])
@pytest.mark.parametrize("head_k", [8, 32])
@pytest.mark.parametrize("head_q", [32, 64])
def test_reference_grid_mha_gqa(head_q, head_k, dim, batch, seq_k, dtype):
    w = wl.make_workload(batch, head_q, head_k, dim, dim, seq_k, dtype, seed=head_q + head_k + dim + batch + seq_k)
    check_against_oracle(w, run_hip(w))


@pytest.mark.parametrize("dtype", DTYPES, ids=_name)
@pytest.mark.parametrize("seq_k", [1, 128, 512])
@pytest.mark.parametrize("batch", [1, 2, 16])
@pytest.mark.parametrize("head_q", [16, 32, 64, 128])
def test_reference_grid_mla(head_q, batch, seq_k, dtype):
    w = wl.config_mla(batch, seq_k, seed=head_q + batch + seq_k, dtype=dtype, head_q=head_q)
    check_against_oracle(w, run_hip(w))


@pytest.mark.parametrize("batch,seq_k", [(1, 128), (8, 128), (32, 128), (128, 128), (512, 128), (1, 512), (1, 1536),
                                          (1, 4096), (1, 6144), (2, 4096), (1, 8192)])
def test_config1_mha_sweep_points(batch, seq_k):
    """Every point of the two sweeps (batch 2048 below), every row against the oracle."""
    w = wl.config_mha_sweep(batch, seq_k)
    check_against_oracle(w, run_hip(w))


def test_config1_mha_sweep_batch_2048():
    """The largest point of the batch sweep: all 2048 x 32 rows finite, every 16th sequence against the oracle."""
    w = wl.config_mha_sweep(2048, 128)
    o = run_hip(w)
    assert torch.isfinite(o.float()).all()
    rows = list(range(0, 2048, 16)) + [2047]
    _, ref32 = run_oracle(sub_workload(w, rows))
    assert (o[rows].float() - ref32).abs().max().item() <= TOL[torch.float16]


def test_config2_gqa_varlen_scaled():
    w = wl.config_gqa_varlen(seed=1, batch=16, max_len=2048)
    check_against_oracle(w, run_hip(w))


def test_config2_gqa_varlen_full_size_every_row():
    """BASELINE's ragged batch (64 sequences of 1..8192 tokens, balanced grid): every row against the oracle."""
    w = wl.config_gqa_varlen(seed=0)
    check_against_oracle(w, run_hip(w))


def test_config2_gqa_varlen_full_size_without_token_count():
    """The same batch as a caller of the reference-signature entry sees it planned (no token count: fixed splits)."""
    w = wl.config_gqa_varlen(seed=0)
    check_against_oracle(w, run_hip_ex(w, 0))


def test_config2_gqa_fixed_4096_every_row():
    w = wl.config_gqa_fixed(seed=0)
    check_against_oracle(w, run_hip(w))


@pytest.mark.parametrize("batch", [40, 48, 100])
def test_gqa_batches_that_refill_the_grid(batch):
    """Batch sizes whose first plan fills its last round of CUs poorly and is re-planned: every row."""
    w = wl.config_gqa_fixed(seed=batch, batch=batch)
    check_against_oracle(w, run_hip(w))


def test_config3_mqa_alibi_scaled_and_full():
    w = wl.config_mqa_alibi(seed=2, batch=4, seq_k=1024)
    check_against_oracle(w, run_hip(w))
    w = wl.config_mqa_alibi(seed=0)  # BASELINE's shape (batch 32, 4096 tokens): every row
    check_against_oracle(w, run_hip(w))


@pytest.mark.parametrize("batch,seq_k", [(1, 4096), (16, 512), (16, 1024), (16, 2048), (16, 4096), (2, 16384)])
def test_config4_mla_points(batch, seq_k):
    """Points of BASELINE's two latent sweeps that the oracle does whole in seconds: every row."""
    w = wl.config_mla(batch, seq_k)
    check_against_oracle(w, run_hip(w))


@pytest.mark.parametrize("dtype", DTYPES, ids=_name)
def test_latent_kernel_every_trip_count(dtype):
    """256 unsplit sequences of 129 .. 420 tokens, 128 heads: one work-group per sequence, so every count of whole
    tiles from 4 to 13 occurs with and without a partial last tile, on both sides of where the pipelined kernel's
    steady-state loop (pairs of trips) starts and hands over to its general loop.  Every 5th sequence and the ten
    shortest and longest against the oracle, every row finite."""
    lens = torch.tensor([129 + (i * 37) % 292 for i in range(256)], dtype=torch.int32)
    g = torch.Generator().manual_seed(17)
    total = int(lens.sum())
    q = torch.randn(256, 128, 576, generator=g).to(dtype)
    k = torch.randn(total, 1, 576, generator=g).to(dtype)
    w = wl.Workload("trip_counts", q, k, None, wl.get_cu_seq(lens), int(lens.max()), 512, False, lens.tolist())
    p = _lib.plan(w.max_seq_k, 256, 128, 1, 576, 512, total_k=total)
    assert (p["kind"], p["nsplit"], p["heads_per_group"]) == (2, 1, 128)
    assert {int(n) // 32 for n in lens.tolist()} >= set(range(4, 14))
    o = run_hip(w)
    assert torch.isfinite(o.float()).all()
    order = sorted(range(256), key=lambda i: int(lens[i]))
    rows = sorted(set(list(range(0, 256, 5)) + order[:10] + order[-10:]))
    _, ref32 = run_oracle(sub_workload(w, rows))
    assert (o[rows].float() - ref32).abs().max().item() <= TOL[dtype]


@pytest.mark.parametrize("batch,seq_k,step", [(16, 8192, 3), (16, 16384, 5), (128, 4096, 16)])
def test_config4_mla_large_points(batch, seq_k, step):
    """The largest points of the two sweeps: every output finite, every step-th sequence (and the last) against the
    oracle."""
    w = wl.config_mla(batch, seq_k)
    o = run_hip(w)
    assert torch.isfinite(o.float()).all()
    rows = sorted(set(range(0, batch, step)) | {batch - 1})
    _, ref32 = run_oracle(sub_workload(w, rows))
    assert (o[rows].float() - ref32).abs().max().item() <= TOL[torch.float16]


def test_config4_mla_b64_full_size_every_row():
    """BASELINE's headline latent shape (batch 64, 4096 tokens, 4 sequence splits of 16-bit partials): every row."""
    w = wl.config_mla(64, 4096)
    check_against_oracle(w, run_hip(w))


def test_config4_mla_b64_bf16_every_row():
    w = wl.config_mla(64, 4096, dtype=torch.bfloat16)
    check_against_oracle(w, run_hip(w))


@pytest.mark.parametrize("dtype", DTYPES, ids=_name)
@pytest.mark.parametrize("hq,hk", [(8, 8), (8, 4), (12, 4), (8, 1), (32, 1), (20, 4), (48, 8)])
def test_head_group_shapes(hq, hk, dtype):
    """Group sizes 1, 2, 3, 4, 5, 6, 8, 32 (3, 5 and 6 leave a partly idle work-group)."""
    w = wl.make_workload(3, hq, hk, 128, 128, 333, dtype, seed=hq * 7 + hk, varlen=True)
    check_against_oracle(w, run_hip(w))


@pytest.mark.parametrize("dim", [64, 128, 256])
@pytest.mark.parametrize("hq,hk", [(33, 1), (40, 1), (64, 1), (128, 1), (80, 2), (144, 4)])
def test_more_than_32_query_heads_per_kv_head(hq, hk, dim):
    """Groups beyond the 32 heads one work-group serves: several work-groups per KV head, the last partly idle."""
    dtype = torch.bfloat16 if (hq + dim) % 3 == 0 else torch.float16
    w = wl.make_workload(3, hq, hk, dim, dim, 700, dtype, seed=hq + dim, varlen=True, is_alibi=hq == 40)
    check_against_oracle(w, run_hip(w))


@pytest.mark.parametrize("dim", [64, 96, 128, 256])
def test_ragged_lengths_with_empty_and_single(dim):
    lens = torch.tensor([0, 1, 2, 63, 64, 65, 127, 129, 0, 700, 1, 0], dtype=torch.int32)
    g = torch.Generator().manual_seed(dim)
    total = int(lens.sum())
    q = torch.randn(len(lens), 8, dim, generator=g).to(torch.float16)
    k = torch.randn(total, 2, dim, generator=g).to(torch.float16)
    v = torch.randn(total, 2, dim, generator=g).to(torch.float16)
    w = wl.Workload("ragged", q, k, v, wl.get_cu_seq(lens), int(lens.max()), dim, False, lens.tolist())
    o = run_hip(w)
    check_against_oracle(w, o)
    for b, n in enumerate(lens.tolist()):
        if n == 0:
            assert (o[b].float() == 0).all()  # documented: an empty sequence yields zeros
        if n == 1:
            start = int(w.cu_seq_k[b])
            assert torch.equal(o[b].view(torch.int16), v[start].repeat_interleave(4, dim=0).view(torch.int16))


def test_ragged_mla_with_empty():
    lens = torch.tensor([0, 1, 65, 300, 0, 1031], dtype=torch.int32)
    g = torch.Generator().manual_seed(5)
    total = int(lens.sum())
    q = torch.randn(len(lens), 128, 576, generator=g).to(torch.bfloat16)
    k = torch.randn(total, 1, 576, generator=g).to(torch.bfloat16)
    w = wl.Workload("ragged_mla", q, k, None, wl.get_cu_seq(lens), int(lens.max()), 512, False, lens.tolist())
    o = run_hip(w)
    check_against_oracle(w, o)
    assert (o[0].float() == 0).all() and (o[4].float() == 0).all()
    assert torch.equal(o[1, 7].view(torch.int16), k[0, 0, :512].view(torch.int16))


def test_split_and_unsplit_agree():
    """One sequence alone is split many ways; inside a large batch it is not.  Both must match the oracle
    and each other."""
    big = wl.make_workload(256, 32, 8, 128, 128, 2048, torch.float16, seed=21)
    p_big = _lib.plan(2048, 256, 32, 8, 128, 128, total_k=256 * 2048)  # (the Python face passes the token count)
    o_big = run_hip(big)
    one = sub_workload(big, [3])
    p_one = _lib.plan(2048, 1, 32, 8, 128, 128)
    assert p_one["nsplit"] > p_big["nsplit"]
    o_one = run_hip(one)
    _, ref32 = run_oracle(one)
    assert (o_one.float() - ref32).abs().max().item() <= TOL[torch.float16]
    assert (o_big[3:4].float() - ref32).abs().max().item() <= TOL[torch.float16]
    assert (o_big[3:4].float() - o_one.float()).abs().max().item() <= 1e-3


def test_repeated_calls_are_bit_identical():
    for w in (wl.config_mha_sweep(1, 4096), wl.config_mla(2, 1024), wl.config_gqa_varlen(seed=4, batch=8, max_len=1024)):
        a = run_hip(w)
        b = run_hip(w)
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))


def test_alibi_default_and_custom_slopes():
    w = wl.make_workload(3, 16, 4, 128, 128, 777, torch.float16, seed=31, varlen=True, is_alibi=True)
    check_against_oracle(w, run_hip(w))
    slopes = torch.linspace(0.01, 0.7, 16, dtype=torch.float32)
    o = run_hip(w, alibi_slopes=slopes.cuda())
    check_against_oracle(w, o, alibi_slopes=slopes.numpy())
    w2 = wl.make_workload(2, 128, 1, 576, 512, 300, torch.float16, seed=32, is_alibi=True, latent=True)
    check_against_oracle(w2, run_hip(w2))


def test_softmax_scale_argument():
    w = wl.make_workload(2, 8, 2, 64, 64, 200, torch.bfloat16, seed=33)
    o = run_hip(w, softmax_scale=0.3)
    check_against_oracle(w, o, softmax_scale=0.3)


def test_max_seq_k_larger_than_needed_and_output_argument():
    w = wl.make_workload(4, 32, 8, 128, 128, 300, torch.float16, seed=34, varlen=True)
    dev = torch.device("cuda:0")
    wd = w.to(dev)
    o_buf = torch.full((4, 32, 128), 7.0, dtype=torch.float16, device=dev)
    out = fwd(wd.q, wd.k, wd.v, o_buf, wd.cu_seq_k, 5000, 128, False)
    torch.cuda.synchronize()
    assert out.data_ptr() == o_buf.data_ptr()
    check_against_oracle(w, out.cpu())


def test_non_contiguous_inputs_are_copied_not_misread():
    w = wl.make_workload(2, 8, 8, 64, 64, 50, torch.float16, seed=35)
    dev = torch.device("cuda:0")
    k_wide = torch.zeros(100, 8, 128, dtype=torch.float16, device=dev)
    k_wide[:, :, :64] = w.k.to(dev)
    k_view = k_wide[:, :, :64]          # unit last stride, but not dense: the reference would mis-read it
    v_t = w.v.to(dev).transpose(0, 1).contiguous().transpose(0, 1)  # last stride 1, rows permuted in memory
    o = decoding_attn_fwd(w.q.to(dev), k_view, v_t, w.cu_seq_k.to(dev), 50, 64, False)
    torch.cuda.synchronize()
    check_against_oracle(w, o.cpu())


def test_non_default_stream():
    w = wl.config_mha_sweep(1, 2048)
    dev = torch.device("cuda:0")
    wd = w.to(dev)
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        o = decoding_attn_fwd(wd.q, wd.k, wd.v, wd.cu_seq_k, wd.max_seq_k, 128, False)
    s.synchronize()
    check_against_oracle(w, o.cpu())


def test_reference_signature_entry_point_with_library_workspace():
    """da_decoding_attn (the reference's argument list, library-owned workspace) on a split shape."""
    lib = _lib.load()
    w = wl.config_mha_sweep(1, 4096)
    assert _lib.plan(4096, 1, 32, 32, 128, 128)["nsplit"] > 1
    dev = torch.device("cuda:0")
    wd = w.to(dev)
    o = torch.empty(1, 32, 128, dtype=torch.float16, device=dev)
    for _ in range(2):
        rc = lib.da_decoding_attn(wd.q.data_ptr(), wd.k.data_ptr(), wd.v.data_ptr(), o.data_ptr(),
                                  wd.cu_seq_k.data_ptr(), 4096, 1, 32, 32, 128, 128, 0, 0,
                                  torch.cuda.current_stream().cuda_stream)
        assert rc == 0, _lib.last_error()
    torch.cuda.synchronize()
    check_against_oracle(w, o.cpu())


def test_reference_signature_entry_point_takes_the_plan_of_a_uniform_batch():
    """BASELINE's GQA shape (batch 64 x 4096 tokens, 32/8 heads) through da_decoding_attn, which is told no token
    count: the same cut as the counted call (four splits of 1024 tokens), so the same bits and the same time as the
    Python face; and the library's cached workspace can be released and is allocated again on the next call."""
    lib = _lib.load()
    w = wl.config_gqa_fixed(seed=0)
    dev = torch.device("cuda:0")
    wd = w.to(dev)
    o = torch.full((64, 32, 128), float("nan"), dtype=w.q.dtype, device=dev)
    stream = torch.cuda.current_stream().cuda_stream

    def ref_sig():
        rc = lib.da_decoding_attn(wd.q.data_ptr(), wd.k.data_ptr(), wd.v.data_ptr(), o.data_ptr(),
                                  wd.cu_seq_k.data_ptr(), 4096, 64, 32, 8, 128, 128, 0,
                                  int(w.q.dtype == torch.bfloat16), stream)
        assert rc == 0, _lib.last_error()

    def python_face():
        return decoding_attn_fwd(wd.q, wd.k, wd.v, wd.cu_seq_k, wd.max_seq_k, 128, False)

    ref_sig()
    o_face = python_face()
    torch.cuda.synchronize()
    assert torch.equal(o, o_face)

    def us_per_call(fn, reps=100):
        for _ in range(10):
            fn()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(reps):
            fn()
        b.record()
        b.synchronize()
        return a.elapsed_time(b) * 1000.0 / reps

    t_ref, t_face = us_per_call(ref_sig), us_per_call(python_face)
    print(f"GQA b64 sk4096: da_decoding_attn {t_ref:.1f} us/call, Python face {t_face:.1f} us/call")
    # (the same plan gives the same bits above; the times are printed for the record and bound nothing: a parity suite
    # must not depend on the power state of the box)

    torch.cuda.synchronize()
    assert lib.da_release_workspaces() == 0, _lib.last_error()
    o.fill_(float("nan"))
    ref_sig()
    torch.cuda.synchronize()
    assert torch.equal(o, o_face)


def test_total_k_hint_changes_the_plan_not_the_result():
    """A ragged batch through da_decoding_attn_ex with and without the token-count hint; both match the oracle."""
    lib = _lib.load()
    dev = torch.device("cuda:0")
    b = 64
    w = wl.make_workload(b, 32, 8, 128, 128, 2048, torch.bfloat16, seed=11, varlen=True)
    total, sk = int(w.k.shape[0]), int(w.max_seq_k)
    # (with the count: equal shares of the concatenated tokens; without: this small batch keeps fixed splits)
    assert _lib.plan(sk, b, 32, 8, 128, 128, True, total)["balanced"] and not _lib.plan(sk, b, 32, 8, 128, 128, True)["balanced"]
    wd = w.to(dev)
    for hint in (0, total):
        n = lib.da_workspace_bytes(sk, b, 32, 8, 128, 128, hint)
        ws = torch.empty(n, dtype=torch.uint8, device=dev)
        o = torch.full((b, 32, 128), float("nan"), dtype=torch.bfloat16, device=dev)
        rc = lib.da_decoding_attn_ex(wd.q.data_ptr(), wd.k.data_ptr(), wd.v.data_ptr(), o.data_ptr(),
                                     wd.cu_seq_k.data_ptr(), sk, b, 32, 8, 128, 128, 0, 1, 0.0, None, hint,
                                     ws.data_ptr(), n, None)
        assert rc == 0, _lib.last_error()
        torch.cuda.synchronize()
        check_against_oracle(w, o.cpu())


def test_gpu_side_argument_errors():
    lib = _lib.load()
    dev = torch.device("cuda:0")
    w = wl.config_mha_sweep(1, 4096).to(dev)
    o = torch.empty(1, 32, 128, dtype=torch.float16, device=dev)
    small = torch.empty(64, dtype=torch.uint8, device=dev)
    rc = lib.da_decoding_attn_ex(w.q.data_ptr(), w.k.data_ptr(), w.v.data_ptr(), o.data_ptr(), w.cu_seq_k.data_ptr(),
                                 4096, 1, 32, 32, 128, 128, 0, 0, 0.0, None, 0, small.data_ptr(), 64, None)
    assert rc == _lib.DA_ERR_WORKSPACE and "workspace" in _lib.last_error()
    with pytest.raises(RuntimeError, match="one query token per sequence"):
        fwd(torch.cat([w.q, w.q]), w.k, w.v, None, w.cu_seq_k, 4096, 128, False)
    with pytest.raises(RuntimeError, match="shape"):
        fwd(w.q, w.k, w.v[:-1], None, w.cu_seq_k, 4096, 128, False)
    with pytest.raises(RuntimeError, match="unsupported head dims"):
        fwd(w.q[..., :80].contiguous(), w.k[..., :80].contiguous(), None, None, w.cu_seq_k, 4096, 80, False)
    with pytest.raises(RuntimeError, match="batch size must be positive"):
        fwd(w.q[:0], w.k, w.v, None, w.cu_seq_k[:1], 4096, 128, False)


def test_full_size_properties_gqa():
    """Size-independent properties at the benchmark shape: q = 0 gives the mean of V; constant V comes back."""
    dev = torch.device("cuda:0")
    b, hq, hk, d, sk = 64, 32, 8, 128, 4096
    g = torch.Generator().manual_seed(41)
    k = torch.randn(b * sk, hk, d, generator=g).to(torch.bfloat16).to(dev)
    v = torch.randn(b * sk, hk, d, generator=g).to(torch.bfloat16).to(dev)
    cu = wl.get_cu_seq(torch.full((b,), sk, dtype=torch.int32)).to(dev)
    q0 = torch.zeros(b, hq, d, dtype=torch.bfloat16, device=dev)
    o = decoding_attn_fwd(q0, k, v, cu, sk, d, False).float()
    mean_v = v.float().reshape(b, sk, hk, d).mean(dim=1).repeat_interleave(hq // hk, dim=1)
    assert (o - mean_v).abs().max().item() <= 2e-3  # |mean| ~ 0.016, bf16 rounding step there is 6e-5
    q = torch.randn(b, hq, d, generator=g).to(torch.bfloat16).to(dev)
    vc = torch.full_like(v, 0.375)
    o = decoding_attn_fwd(q, k, vc, cu, sk, d, False).float()
    assert (o - 0.375).abs().max().item() <= 2e-3
