"""CPU-side checks: the shared library loads and exports the declared C-ABI, argument validation returns
the documented codes before anything touches a GPU, the launch planner is self-consistent, and the Python
face rejects what the reference's binding rejects (reference csrc/torch/decoding_torch.cpp:24-74)."""
import ctypes
import os
import re

import pytest
import torch

from decoding_attention_amd import _lib, interface
from decoding_attention_amd import workloads as wl

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LEGAL = [(64, 64), (96, 96), (128, 128), (256, 256), (576, 512)]


def test_header_symbols_are_exported():
    text = open(os.path.join(ROOT, "include", "decoding_attn_hip.h")).read()
    c_part = text.split('#ifdef __cplusplus\n} /* extern "C" */')[0]
    declared = set(re.findall(r"\b(da_[a-z_0-9]+)\s*\(", c_part))
    assert declared == set(_lib.EXPORTED_SYMBOLS)
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared:
        assert getattr(lib, name) is not None


def test_version_and_supported_dims():
    lib = _lib.load()
    assert lib.da_version() == 100
    for d in (32, 64, 96, 128, 192, 256, 512, 576):
        for dv in (64, 96, 128, 256, 512, 576):
            assert bool(lib.da_supported_head_dims(d, dv)) == ((d, dv) in LEGAL)


def _call_ex(lib, q=16, k=16, v=16, o=16, cu=16, max_seq_k=8, batch=1, hq=4, hk=4, d=64, dv=64):
    return lib.da_decoding_attn_ex(q, k, v, o, cu, max_seq_k, batch, hq, hk, d, dv, 0, 0, 0.0, None, 0, None, 0, None)


def test_argument_errors_without_gpu():
    lib = _lib.load()
    assert _call_ex(lib, q=None) == _lib.DA_ERR_INVALID_ARGUMENT and "q is null" in _lib.last_error()
    assert _call_ex(lib, k=None) == _lib.DA_ERR_INVALID_ARGUMENT
    assert _call_ex(lib, o=None) == _lib.DA_ERR_INVALID_ARGUMENT
    assert _call_ex(lib, cu=None) == _lib.DA_ERR_INVALID_ARGUMENT
    assert _call_ex(lib, hq=6, hk=4) == _lib.DA_ERR_INVALID_ARGUMENT and "multiple" in _lib.last_error()
    assert _call_ex(lib, d=640, dv=64) == _lib.DA_ERR_INVALID_ARGUMENT
    assert _call_ex(lib, d=576, dv=576) == _lib.DA_ERR_INVALID_ARGUMENT
    assert _call_ex(lib, d=80, dv=80) == _lib.DA_ERR_UNSUPPORTED and "unsupported" in _lib.last_error()
    assert _call_ex(lib, d=128, dv=64) == _lib.DA_ERR_UNSUPPORTED
    assert _call_ex(lib, q=24) == _lib.DA_ERR_INVALID_ARGUMENT and "aligned" in _lib.last_error()
    assert _call_ex(lib, o=24) == _lib.DA_ERR_INVALID_ARGUMENT and "o must be 16-byte aligned" in _lib.last_error()
    assert _call_ex(lib, batch=0) == _lib.DA_OK  # nothing to do, nothing launched


@pytest.mark.parametrize("d,dv", LEGAL)
@pytest.mark.parametrize("batch", [1, 16, 64, 2048])
@pytest.mark.parametrize("sk", [1, 128, 1536, 4096, 16384])
def test_plan_is_consistent(d, dv, batch, sk):
    hq, hk = (128, 1) if d == 576 else (32, 8)
    p = _lib.plan(sk, batch, hq, hk, d, dv)
    assert p["kind"] in (1, 2, 3)
    ws = _lib.load().da_workspace_bytes(sk, batch, hq, hk, d, dv, 0)
    if p["balanced"]:
        # no token count given: equal shares of the concatenated tokens, the share derived on the device; a partial
        # slot per (share, sequence) pair that can occur
        assert p["kind"] == 3 and p["chunk"] == 0 and batch >= 2 and 1 <= p["nsplit"] <= 512
        assert ws == (p["nsplit"] + batch) * hq * (dv + 2) * 4
        return
    assert 1 <= p["nsplit"] <= 256
    assert p["nsplit"] * p["chunk"] >= sk
    assert (p["nsplit"] - 1) * p["chunk"] < max(sk, 1)
    need = 0 if p["nsplit"] == 1 else batch * hq * p["nsplit"] * (dv + 2) * 4
    # (576, 512) also covers the plan used when V is passed as its own buffer
    assert ws >= need if d == 576 else ws == need


def test_plan_total_k_hint_changes_the_splits_and_never_the_kernel():
    """The token-count hint changes how a batch is cut (a ragged one into equal shares, one known to be uniform
    into splits that may be longer), and never the kernel kind."""
    sk, batch = 8192, 64
    base = _lib.plan(sk, batch, 32, 8, 128, 128)
    full = _lib.plan(sk, batch, 32, 8, 128, 128, total_k=batch * sk)
    ragged = _lib.plan(sk, batch, 32, 8, 128, 128, total_k=batch * sk // 2)
    assert full["kind"] == base["kind"] and full["chunk"] >= base["chunk"] and full["nsplit"] <= base["nsplit"]
    # grouped kernel: equal shares of the concatenated tokens, 256 work-groups over the 2 groups of 4 KV heads
    assert ragged["kind"] == base["kind"] == 3 and ragged["balanced"] and not full["balanced"]
    assert ragged["nsplit"] == 128 and ragged["chunk"] == batch * sk // 2 // 128
    # a partial slot per (share, sequence) pair that can occur: shares + sequences
    ws = _lib.load().da_workspace_bytes(sk, batch, 32, 8, 128, 128, batch * sk // 2)
    assert ws == (ragged["nsplit"] + batch) * 32 * (128 + 2) * 4
    # without a count the same grid, the share left to the device
    assert base["balanced"] and base["nsplit"] == 128 and base["chunk"] == 0
    # VALU sweep (one query head per KV head, short sequences): shorter fixed splits
    sk, batch = 2048, 16
    base = _lib.plan(sk, batch, 32, 32, 256, 256)
    ragged = _lib.plan(sk, batch, 32, 32, 256, 256, total_k=batch * sk // 2)
    assert ragged["kind"] == base["kind"] == 1 and ragged["chunk"] < base["chunk"]
    assert ragged["nsplit"] * ragged["chunk"] >= sk


def test_plan_without_a_token_count_at_d128():
    """The reference-signature entry point passes no token count: a batch large enough for whole shares then takes the
    balanced grid, which cuts a uniform batch exactly as the counted plan's fixed splits do (128 shares of 64 x 4096 /
    128 = 2048 tokens, the share derived on the device); smaller problems keep fixed splits of up to 2048 tokens."""
    blind = _lib.plan(4096, 64, 32, 8, 128, 128)
    counted = _lib.plan(4096, 64, 32, 8, 128, 128, total_k=64 * 4096)
    assert blind["kind"] == counted["kind"] == 3
    assert (counted["nsplit"], counted["chunk"], counted["balanced"]) == (2, 2048, False)
    assert (blind["nsplit"], blind["chunk"], blind["balanced"]) == (128, 0, True)
    # a single long sequence: nothing to balance, the cap sets the cut
    one = _lib.plan(16384, 1, 32, 8, 128, 128)
    assert not one["balanced"] and one["chunk"] <= 2048
    # MQA (four waves share the one KV head's tokens): 256 work-groups
    assert _lib.plan(4096, 64, 32, 1, 128, 128, total_k=64 * 4096)["nsplit"] == 4
    assert _lib.load().da_release_workspaces() == _lib.DA_OK  # nothing cached, nothing to free, no GPU needed


def test_workspace_sizes_of_the_paged_and_fp8_variants():
    lib = _lib.load()
    shape = (4096, 64, 32, 8, 128, 128)
    # (with the token count: without one the packed layout takes the balanced grid, which paged K/V only takes with it)
    shape_total = 64 * 4096
    packed = lib.da_workspace_bytes(*shape, shape_total)
    # pages of 16 tokens and more take the packed layout's kernels and plan; shorter pages keep the shorter splits
    for page in (16, 64, 256):
        assert lib.da_workspace_bytes_paged(*shape, shape_total, page) == packed
    for page in (1, 8):
        assert lib.da_workspace_bytes_paged(*shape, shape_total, page) >= packed
    # 8-bit K/V: the same kernel kind, with the shorter splits its half-length rows were measured on
    assert lib.da_workspace_bytes_fp8kv(*shape, shape_total, 0) >= packed
    # the latent form: the larger of the MFMA kernel's plan (V inside K) and the VALU sweep's (a distinct V buffer)
    mla = (4096, 16, 128, 1, 576, 512)
    assert lib.da_workspace_bytes_fp8kv(*mla, 0, 0) > 0
    assert lib.da_workspace_bytes_fp8kv(128, 4, 6, 4, 64, 64, 0, 0) == 0   # head_q not a multiple of head_k
    assert lib.da_workspace_bytes_int8kv(*shape, 0, 0) == lib.da_workspace_bytes_fp8kv(*shape, 0, 0) and lib.da_workspace_bytes_int8kv(*mla, 0, 0) > 0


def test_int4_entry_points_check_their_arguments_without_a_gpu():
    lib = _lib.load()
    shape = (4096, 64, 32, 8, 128, 128)
    assert lib.da_workspace_bytes_int4kv(*shape, 0, 0) == lib.da_workspace_bytes_int8kv(*shape, 0, 0)
    args = (16, 16, 16, 16, 16, 8, 1, 4, 4, 64, 64, 0, 0, 0.0, None, None, None, 0, None, 0, None)
    assert lib.da_decoding_attn_int4kv(None, *args[1:]) == _lib.DA_ERR_INVALID_ARGUMENT and "q is null" in _lib.last_error()
    bad = list(args)
    bad[1] = 24  # k4 not 16-byte aligned
    assert lib.da_decoding_attn_int4kv(*bad) == _lib.DA_ERR_INVALID_ARGUMENT and "aligned" in _lib.last_error()


def test_plan_rejects_bad_shapes():
    with pytest.raises(RuntimeError):
        _lib.plan(128, 1, 6, 4, 64, 64)
    with pytest.raises(RuntimeError):
        _lib.plan(128, 1, 4, 4, 80, 80)


def test_plan_of_every_call_form():
    """da_plan_call: the plan of packed and paged calls, of a V buffer of its own and of the 8- and 4-bit caches, and
    its agreement with the narrower queries."""
    import ctypes
    lib = _lib.load()
    shape = (4096, 64, 128, 1, 576, 512)
    base = _lib.plan(*shape, total_k=64 * 4096)
    assert base == {"kind": 2, "nsplit": 4, "chunk": 1024, "heads_per_group": 128, "balanced": False}
    kind, ns = ctypes.c_int(), ctypes.c_int()
    assert lib.da_plan(*shape, 0, 64 * 4096, ctypes.byref(kind), ctypes.byref(ns), None, None) == 0
    assert (kind.value, ns.value) == (base["kind"], base["nsplit"])
    assert _lib.plan(*shape, total_k=64 * 4096, kv_bits=8)["kind"] == 2       # FP8 / int8: the latent kernel
    assert _lib.plan(*shape, total_k=64 * 4096, kv_bits=4)["kind"] == 3       # int4: groups of 16 heads
    assert _lib.plan(*shape, total_k=64 * 4096, distinct_v=True)["kind"] == 2
    assert _lib.plan(*shape, total_k=64 * 4096, distinct_v=True, page_size=8)["kind"] == 1  # the remaining cliff
    assert _lib.plan(*shape, total_k=64 * 4096, distinct_v=True, kv_bits=8)["kind"] == 1
    # more work-groups over an 8-bit latent cache than over a 16-bit one at a mid-sized batch
    assert _lib.plan(4096, 16, 128, 1, 576, 512, kv_bits=8)["nsplit"] > _lib.plan(4096, 16, 128, 1, 576, 512)["nsplit"]
    ragged = _lib.plan(8192, 64, 32, 8, 128, 128, total_k=300000, page_size=64)
    assert ragged["balanced"] == bool(lib.da_plan_is_balanced(8192, 64, 32, 8, 128, 128, 300000, 64))
    # per-token pairs and pairs per 64 elements: the grouped kernel whatever the shape
    for bits in (_lib.KV_BITS_INT4_PER_TOKEN, _lib.KV_BITS_INT8_PER_TOKEN, _lib.KV_BITS_INT4_GROUP64,
                 _lib.KV_BITS_INT8_GROUP64):
        assert _lib.plan(128, 512, 32, 32, 128, 128, kv_bits=bits)["kind"] == 3
        with pytest.raises(RuntimeError):
            _lib.plan(128, 512, 32, 32, 96, 96, kv_bits=bits)
    # one query head per KV head: the grouped kernel over long sequences of a small batch at d <= 128, else the VALU sweep
    assert _lib.plan(8192, 1, 32, 32, 128, 128, distinct_v=True)["kind"] == 3
    assert _lib.plan(6144, 1, 32, 32, 128, 128, distinct_v=True)["kind"] == 3
    assert _lib.plan(4096, 1, 32, 32, 128, 128, distinct_v=True)["kind"] == 1
    assert _lib.plan(8192, 1, 16, 16, 256, 256, distinct_v=True)["kind"] == 1
    assert _lib.plan(128, 512, 32, 32, 128, 128, distinct_v=True)["kind"] == 1
    for bad in (dict(kv_bits=12), dict(page_size=48)):
        with pytest.raises(RuntimeError):
            _lib.plan(*shape, **bad)
    assert lib.da_plan_call(*shape, 0, 0, 0, 16, None, None, None, None, None) == 0  # every output may be null


def test_python_face_checks_cpu_inputs():
    w = wl.make_workload(2, 4, 2, 64, 64, 8, torch.float16)
    with pytest.raises(RuntimeError, match="GPU"):
        interface.decoding_attn_fwd(w.q, w.k, w.v, w.cu_seq_k, 8, 64, False)
    with pytest.raises(RuntimeError, match="FP16 and BF16"):
        interface.fwd(w.q.float(), w.k.float(), None, None, w.cu_seq_k, 8, 64, False)
    with pytest.raises(RuntimeError, match="same dtype"):
        interface.fwd(w.q, w.k.to(torch.bfloat16), None, None, w.cu_seq_k, 8, 64, False)
    with pytest.raises(RuntimeError, match="int32"):
        interface.fwd(w.q, w.k, None, None, w.cu_seq_k.long(), 8, 64, False)


def test_value_view_of_the_key_rows_is_recognised():
    """`k[..., :dim_v]` passed as v is the latent form's aliasing: it must not be copied into a buffer of its own."""
    k = torch.randn(10, 1, 576).to(torch.float16)
    assert interface.is_leading_columns_view(k[..., :512], k)
    assert interface.is_leading_columns_view(k, k)
    assert not interface.is_leading_columns_view(k[..., :512].contiguous(), k)
    assert not interface.is_leading_columns_view(k[..., 64:], k)          # not the leading columns
    assert not interface.is_leading_columns_view(k[1:, :, :512], k[1:].clone())
    assert not interface.is_leading_columns_view(None, k)
    assert not interface.is_leading_columns_view(k[::2, :, :512], k)       # other rows


def test_drop_in_package_name():
    import decoding_attn

    assert decoding_attn.decoding_attn_fwd is interface.decoding_attn_fwd
    assert decoding_attn.__version__ == "0.1.0"


def test_work_formulas():
    # figures quoted for the benchmark configurations
    assert wl.algorithmic_bytes(1, 32, 32, 128, 128, 128, True) == 2 * (4096 + 2 * 128 * 4096 + 4096) + 8
    gqa = wl.algorithmic_bytes(64, 32, 8, 128, 128, 64 * 4096, True)
    assert abs(gqa - 1074.8e6) < 0.1e6
    mla = wl.algorithmic_bytes(64, 128, 1, 576, 512, 64 * 4096, False)
    assert abs(mla - 319.8e6) < 0.1e6
    assert wl.algorithmic_flops(128, 576, 512, 64 * 4096) == 2 * 64 * 4096 * 128 * 1088
    assert wl.reference_formula_bytes(1, 32, 32, 128, 128, 128) == 2 * (4096 + 128 * 4096 + 4096)


def test_workloads_are_reproducible():
    a = wl.config_gqa_varlen(seed=3, batch=4, max_len=64)
    b = wl.config_gqa_varlen(seed=3, batch=4, max_len=64)
    assert a.lengths == b.lengths and torch.equal(a.k.view(torch.int16), b.k.view(torch.int16))
    assert a.cu_seq_k.tolist()[-1] == sum(a.lengths) == a.k.shape[0]
    assert 1 <= min(a.lengths) and max(a.lengths) <= 64 and a.max_seq_k == max(a.lengths)
    m = wl.config_mla(2, 16)
    assert m.v is None and m.q.shape == (2, 128, 576) and m.dim_v == 512


def test_torch_extension_module_exports_fwd():
    """The PyTorch-ROCm extension (the counterpart of the reference's `decoding_attn_cuda`) loads and exposes `fwd`
    with the reference's argument names (reference csrc/torch/decoding_torch.cpp:82-85)."""
    ext = interface._extension()
    doc = ext.fwd.__doc__
    for name in ("q", "k", "v_", "o_", "cu_seq_k", "max_seq_k", "dim_v", "is_alibi"):
        assert name + ":" in doc


def test_pipelined_latent_kernel_leaves_the_named_registers_alone():
    """da_mla_pipe.hip names most of the register file in its instruction text; the build checks the compiler's own
    code for strays (check_isa).  The same check on the tree's source with the build's flags, and the checker itself on
    three lines it must flag."""
    import shutil

    from decoding_attention_amd import build as da_build
    from decoding_attention_amd import check_isa

    bad = check_isa.check_text("\tv_mov_b32_e32 v64, v1\n\tv_accvgpr_read_b32 v3, a7\n\tscratch_load_dword v1, off, s0\n"
                               "#ASMSTART\n\tv_mov_b32 v200, v1\n#ASMEND\n\tv_add_u32_e32 v63, v1, v2\n")
    assert [i for i, _ in bad] == [1, 2, 3]
    hipcc = da_build._hipcc()
    if shutil.which(hipcc) is None and not os.path.exists(hipcc):
        pytest.skip("no hipcc here")
    src = os.path.join(da_build.CSRC, "da_mla_pipe.hip")
    assert check_isa.check_source(hipcc, da_build.HIPCC_FLAGS + da_build.EXTRA_FLAGS["da_mla_pipe.hip"], src)
