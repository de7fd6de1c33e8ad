"""Helpers shared by the GPU parity tests: run the HIP path through the C-ABI and compare with the oracle."""
import numpy as np
import torch

from decoding_attention_amd import decoding_attn_fwd
from oracle import oracle

# acceptance: max-abs against an fp32-accumulated CPU result on the same seeded inputs
TOL = {torch.float16: 2e-3, torch.bfloat16: 1e-2}
ORACLE_THREADS = 16


def run_hip(w, **kw):
    dev = torch.device("cuda:0")
    wd = w.to(dev)
    o = decoding_attn_fwd(wd.q, wd.k, wd.v, wd.cu_seq_k, wd.max_seq_k, wd.dim_v, wd.is_alibi, **kw)
    torch.cuda.synchronize()
    return o.cpu()


def run_hip_ex(w, total_k_hint, fill=None):
    """The packed call through da_decoding_attn_ex with a caller-owned workspace and the given token-count hint
    (the Python face always passes k.shape[0]; 0 here selects the plan of a caller who does not know it).  `fill`: a
    byte value the workspace holds before the call (default: whatever the allocator hands out)."""
    from decoding_attention_amd import _lib
    lib = _lib.load()
    dev = torch.device("cuda:0")
    wd = w.to(dev)
    b, hq, d = w.q.shape
    hk = w.k.shape[1]
    n = lib.da_workspace_bytes(w.max_seq_k, b, hq, hk, d, w.dim_v, total_k_hint)
    ws = torch.empty(max(n, 16), dtype=torch.uint8, device=dev)
    if fill is not None:
        ws.fill_(fill)
    o = torch.full((b, hq, w.dim_v), float("nan"), dtype=w.q.dtype, device=dev)
    rc = lib.da_decoding_attn_ex(wd.q.data_ptr(), wd.k.data_ptr(), None if wd.v is None else wd.v.data_ptr(),
                                 o.data_ptr(), wd.cu_seq_k.data_ptr(), w.max_seq_k, b, hq, hk, d, w.dim_v,
                                 int(w.is_alibi), int(w.q.dtype == torch.bfloat16), 0.0, None, total_k_hint,
                                 ws.data_ptr(), n, torch.cuda.current_stream().cuda_stream)
    assert rc == 0, _lib.last_error()
    torch.cuda.synchronize()
    return o.cpu()


def run_oracle(w, **kw):
    return oracle.attn_cpu(w.q, w.k, w.v, w.cu_seq_k, w.max_seq_k, w.dim_v, w.is_alibi, nthreads=ORACLE_THREADS,
                           return_f32=True, **kw)


def check_against_oracle(w, o_hip, **kw):
    """max-abs of (HIP - oracle fp32) within tolerance; also the reference's own mean-abs bar vs the rounded oracle."""
    o_ref, o_ref32 = run_oracle(w, **kw)
    err = (o_hip.float() - o_ref32).abs().max().item()
    mean_err = (o_hip.float() - o_ref.float()).abs().mean().item()
    assert err <= TOL[w.q.dtype], f"{w.name}: max-abs {err:.3e} > {TOL[w.q.dtype]:.0e}"
    assert mean_err <= 5e-3, f"{w.name}: mean-abs {mean_err:.3e}"
    return err


def sub_workload(w, rows):
    """The same workload restricted to the given sequences (for spot checks of big shapes on the CPU)."""
    from decoding_attention_amd.workloads import Workload, get_cu_seq
    cu = w.cu_seq_k.tolist()
    ks = [w.k[cu[b]:cu[b + 1]] for b in rows]
    vs = None if w.v is None else [w.v[cu[b]:cu[b + 1]] for b in rows]
    lens = torch.tensor([k.shape[0] for k in ks], dtype=torch.int32)
    return Workload(w.name + "_sub", w.q[rows].contiguous(), torch.cat(ks), None if vs is None else torch.cat(vs),
                    get_cu_seq(lens), int(lens.max()), w.dim_v, w.is_alibi, lens.tolist())
