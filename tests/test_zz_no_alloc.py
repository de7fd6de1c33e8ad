"""The entry point that allocates nothing (da_decoding_attn_noalloc: split partials in a static device array) against
da_decoding_attn_ex with a caller-owned workspace: same kernels, same plan, so the outputs must be equal bit for bit.
Two calls in a row share the array, the second with a smaller input (stale partials of the first must not leak in)."""
import pytest
import torch

from decoding_attention_amd import _lib
from decoding_attention_amd import workloads as wl

pytestmark = pytest.mark.gpu


def _call(lib, fn_noalloc, w, dev):
    wd = w.to(dev)
    b, hq, d = w.q.shape
    hk = w.k.shape[1]
    total_k = w.k.shape[0]
    bf16 = int(w.q.dtype == torch.bfloat16)
    stream = torch.cuda.current_stream().cuda_stream
    v_ptr = None if wd.v is None else wd.v.data_ptr()
    o = torch.full((b, hq, w.dim_v), float("nan"), dtype=w.q.dtype, device=dev)
    if fn_noalloc:
        rc = lib.da_decoding_attn_noalloc(wd.q.data_ptr(), wd.k.data_ptr(), v_ptr, o.data_ptr(), wd.cu_seq_k.data_ptr(),
                                          w.max_seq_k, b, hq, hk, d, w.dim_v, int(w.is_alibi), bf16, 0.0, None, total_k,
                                          stream)
    else:
        n = lib.da_workspace_bytes(w.max_seq_k, b, hq, hk, d, w.dim_v, total_k)
        ws = torch.empty(max(n, 16), dtype=torch.uint8, device=dev)
        rc = lib.da_decoding_attn_ex(wd.q.data_ptr(), wd.k.data_ptr(), v_ptr, o.data_ptr(), wd.cu_seq_k.data_ptr(),
                                     w.max_seq_k, b, hq, hk, d, w.dim_v, int(w.is_alibi), bf16, 0.0, None, total_k,
                                     ws.data_ptr(), n, stream)
    assert rc == 0, _lib.last_error()
    torch.cuda.synchronize()
    return o.cpu()


def test_noalloc_matches_ex_on_two_calls_in_a_row():
    lib = _lib.load()
    dev = torch.device("cuda:0")
    assert lib.da_noalloc_workspace_limit() == 80 << 20
    # (each pair: a larger call, then a smaller one on the same static array)
    cases = [
        wl.make_workload(8, 32, 8, 128, 128, 2048, torch.bfloat16, seed=3),               # grouped kernel, split
        wl.make_workload(3, 32, 8, 128, 128, 700, torch.bfloat16, seed=4, varlen=True),
        wl.config_mla(16, 4096),                                                          # latent kernel, 16 splits
        wl.config_mla(2, 1000, seed=5),
        wl.config_mqa_alibi(batch=4, seq_k=4096),                                         # ALiBi, split
        wl.make_workload(2, 32, 32, 128, 128, 1536, torch.float16, seed=6),               # VALU sweep, split
    ]
    for w in cases:
        want = _call(lib, False, w, dev)
        got = _call(lib, True, w, dev)
        assert torch.isfinite(got.float()).all(), w.name
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), w.name


def test_noalloc_refuses_a_plan_beyond_the_static_array():
    lib = _lib.load()
    dev = torch.device("cuda:0")
    # 60 sequences of 131072 tokens each, known to be uniform, 32/8 heads at d = 256: 64 fixed splits of 2048 tokens
    # with fp32 partials, 127 MB.  The call must fail before anything is enqueued, so the tensors only need to exist.
    b, hq, hk, d = 60, 32, 8, 256
    q = torch.zeros((b, hq, d), dtype=torch.bfloat16, device=dev)
    k = torch.zeros((16, hk, d), dtype=torch.bfloat16, device=dev)
    o = torch.zeros((b, hq, d), dtype=torch.bfloat16, device=dev)
    cu = torch.zeros((b + 1,), dtype=torch.int32, device=dev)
    max_seq = 131072
    total_k = b * max_seq
    need = lib.da_workspace_bytes(max_seq, b, hq, hk, d, d, total_k)
    assert need > lib.da_noalloc_workspace_limit()
    rc = lib.da_decoding_attn_noalloc(q.data_ptr(), k.data_ptr(), k.data_ptr(), o.data_ptr(), cu.data_ptr(), max_seq, b, hq,
                                      hk, d, d, 0, 1, 0.0, None, total_k, torch.cuda.current_stream().cuda_stream)
    assert rc == _lib.DA_ERR_WORKSPACE
    assert "static array" in _lib.last_error()
    torch.cuda.synchronize()
