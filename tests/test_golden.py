"""Golden fixtures (tests/golden/*.npz, written by tests/golden/make_fixtures.py): the oracle must reproduce its
recorded output bits and stay within fp32-accumulation distance of the recorded float64 result; on a GPU the HIP
path must match the same fixtures within the acceptance tolerance."""
import glob
import os

import numpy as np
import pytest
import torch

from oracle import oracle

HERE = os.path.dirname(os.path.abspath(__file__))
FIXTURES = sorted(glob.glob(os.path.join(HERE, "golden", "*.npz")))


def _load(path):
    z = np.load(path, allow_pickle=False)
    dtype = torch.bfloat16 if bool(z["is_bf16"]) else torch.float16
    t = lambda a: torch.from_numpy(a.copy()).view(dtype)  # noqa: E731
    v = t(z["v"]) if "v" in z.files else None
    return (t(z["q"]), t(z["k"]), v, torch.from_numpy(z["cu_seq_k"].copy()), int(z["dim_v"]), bool(z["is_alibi"]),
            z["o"], z["o_f64"], dtype)


def test_fixtures_exist():
    assert len(FIXTURES) >= 6


@pytest.mark.parametrize("path", FIXTURES, ids=lambda p: os.path.basename(p)[:-4])
def test_oracle_reproduces_fixture(path):
    q, k, v, cu, dv, alibi, o_bits, o_f64, _ = _load(path)
    lens = (cu[1:] - cu[:-1]).tolist()
    o, o32 = oracle.attn_cpu(q, k, v, cu, max(lens), dv, alibi, return_f32=True)
    assert np.array_equal(o.view(torch.int16).numpy(), o_bits)
    assert np.abs(o32.numpy() - o_f64).max() < 2e-5


@pytest.mark.gpu
@pytest.mark.parametrize("path", FIXTURES, ids=lambda p: os.path.basename(p)[:-4])
def test_hip_matches_fixture(path):
    from decoding_attention_amd import decoding_attn_fwd

    q, k, v, cu, dv, alibi, o_bits, o_f64, dtype = _load(path)
    lens = (cu[1:] - cu[:-1]).tolist()
    dev = torch.device("cuda:0")
    o = decoding_attn_fwd(q.to(dev), k.to(dev), None if v is None else v.to(dev), cu.to(dev), max(lens), dv, alibi)
    torch.cuda.synchronize()
    tol = 1e-2 if dtype == torch.bfloat16 else 2e-3
    assert np.abs(o.cpu().to(torch.float64).numpy() - o_f64).max() <= tol
