"""The op under HIP graph capture: the call only enqueues kernels (no allocation of its own when the caller brings
the workspace, no memset, no host synchronisation), so it can be captured once and replayed.

Each replay is checked against the eager result for the inputs of that moment, with eager work and synchronisation
between the replays.
"""
import pytest
import torch

from decoding_attention_amd import decoding_attn_fwd, decoding_attn_paged_fwd
from decoding_attention_amd import workloads as wl

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _replay_matches_eager(run, tensors_to_perturb, out_of):
    """Capture run() once; then, several times: change the inputs in place, replay, compare with an eager call."""
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        for _ in range(2):  # warm-up outside the capture (lazy initialisation, allocator state)
            run()
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = run()
    torch.cuda.synchronize()
    g = torch.Generator(device="cpu").manual_seed(1)
    for step in range(4):
        for t in tensors_to_perturb:
            t.copy_(torch.randn(t.shape, generator=g).to(t.dtype))
        graph.replay()
        torch.cuda.synchronize()
        got = out_of(captured).clone()
        want = out_of(run())  # eager, same inputs
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), f"replay {step}"


@pytest.mark.parametrize("shape", ["gqa_split", "mha_unsplit", "mla", "mla_distinct_v"])
def test_packed_call_replays_from_a_graph(shape):
    if shape == "gqa_split":
        w = wl.make_workload(8, 32, 8, 128, 128, 2048, torch.bfloat16, seed=4, varlen=True)
    elif shape == "mha_unsplit":
        w = wl.make_workload(64, 8, 8, 128, 128, 128, torch.float16, seed=4)
    elif shape == "mla":
        w = wl.config_mla(4, 700, seed=4)  # the pipelined latent kernel, five tiles per split
    else:
        w = wl.make_workload(4, 128, 1, 576, 512, 700, torch.float16, seed=4, latent=False)  # V in its own buffer
    wd = w.to(DEV)

    def run():
        return decoding_attn_fwd(wd.q, wd.k, wd.v, wd.cu_seq_k, w.max_seq_k, w.dim_v, w.is_alibi)

    _replay_matches_eager(run, [wd.q, wd.k] + ([] if wd.v is None else [wd.v]), lambda o: o)


def test_paged_call_replays_from_a_graph():
    w = wl.make_workload(8, 32, 8, 128, 128, 1500, torch.float16, seed=6, varlen=True)
    pk = wl.to_pages(w, 64, seed=6, poison=False).to(DEV)
    q = w.q.to(DEV)

    def run():
        return decoding_attn_paged_fwd(q, pk.k_pages, pk.v_pages, pk.block_table, pk.seq_lens, w.max_seq_k, 128, False)

    _replay_matches_eager(run, [q, pk.k_pages, pk.v_pages], lambda o: o)


def test_fp8_latent_and_16_token_pages_replay_from_a_graph():
    """The FP8 form of the latent kernel (tiles converted in LDS) and the 16-token-page form of the grouped kernel."""
    w = wl.config_mla(3, 900, seed=8)
    q = w.q.to(DEV)
    k8 = (w.k.float() / 0.02).to(torch.float8_e4m3fn).to(DEV)
    ks = torch.full((1,), 0.02, device=DEV)
    cu = w.cu_seq_k.to(DEV)

    def run_latent():
        return decoding_attn_fwd(q, k8, None, cu, w.max_seq_k, 512, False, k_scale=ks, v_scale=ks)

    _replay_matches_eager(run_latent, [q], lambda o: o)

    w2 = wl.make_workload(6, 32, 1, 128, 128, 1100, torch.bfloat16, seed=9, varlen=True)
    pk = wl.to_pages(w2, 16, seed=9, poison=False).to(DEV)
    q2 = w2.q.to(DEV)

    def run_paged():
        return decoding_attn_paged_fwd(q2, pk.k_pages, pk.v_pages, pk.block_table, pk.seq_lens, w2.max_seq_k, 128, False)

    _replay_matches_eager(run_paged, [q2, pk.k_pages, pk.v_pages], lambda o: o)


def test_noalloc_entry_point_under_capture_and_without_allocation():
    """da_decoding_attn_noalloc, the entry point for callers that cannot allocate: after one warm-up call per shape (the
    first call on a device looks up the static array's address and raises the kernels' LDS limits, neither of which
    belongs inside a capture) it is captured, replayed on changed inputs and compared with da_decoding_attn_ex bit for
    bit; and steady-state calls leave the device's free memory where it was."""
    from decoding_attention_amd import _lib

    lib = _lib.load()
    for w in (wl.make_workload(8, 32, 8, 128, 128, 2048, torch.bfloat16, seed=11), wl.config_mla(4, 700, seed=12)):
        wd = w.to(DEV)
        b, hq, d = w.q.shape
        hk, total_k = w.k.shape[1], w.k.shape[0]
        bf16 = int(w.q.dtype == torch.bfloat16)
        v_ptr = None if wd.v is None else wd.v.data_ptr()
        o = torch.zeros((b, hq, w.dim_v), dtype=w.q.dtype, device=DEV)
        o_ex = torch.zeros_like(o)
        n = lib.da_workspace_bytes(w.max_seq_k, b, hq, hk, d, w.dim_v, total_k)
        ws = torch.empty(max(n, 16), dtype=torch.uint8, device=DEV)

        def noalloc():
            rc = lib.da_decoding_attn_noalloc(wd.q.data_ptr(), wd.k.data_ptr(), v_ptr, o.data_ptr(),
                                              wd.cu_seq_k.data_ptr(), w.max_seq_k, b, hq, hk, d, w.dim_v,
                                              int(w.is_alibi), bf16, 0.0, None, total_k,
                                              torch.cuda.current_stream().cuda_stream)
            assert rc == 0, _lib.last_error()

        def ex():
            rc = lib.da_decoding_attn_ex(wd.q.data_ptr(), wd.k.data_ptr(), v_ptr, o_ex.data_ptr(),
                                         wd.cu_seq_k.data_ptr(), w.max_seq_k, b, hq, hk, d, w.dim_v, int(w.is_alibi),
                                         bf16, 0.0, None, total_k, ws.data_ptr(), n,
                                         torch.cuda.current_stream().cuda_stream)
            assert rc == 0, _lib.last_error()

        s = torch.cuda.Stream()
        s.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(s):
            noalloc()  # the warm-up call, outside the capture
        torch.cuda.current_stream().wait_stream(s)
        torch.cuda.synchronize()
        free0 = torch.cuda.mem_get_info()[0]
        for _ in range(5):
            noalloc()
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free0, "steady-state calls changed the device's free memory"
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            noalloc()
        torch.cuda.synchronize()
        g = torch.Generator(device="cpu").manual_seed(2)
        for step in range(3):
            for t in [wd.q, wd.k] + ([] if wd.v is None else [wd.v]):
                t.copy_(torch.randn(t.shape, generator=g).to(t.dtype))
            o.zero_()
            graph.replay()
            ex()
            torch.cuda.synchronize()
            assert torch.equal(o.view(torch.int16), o_ex.view(torch.int16)), f"{w.name} replay {step}"
