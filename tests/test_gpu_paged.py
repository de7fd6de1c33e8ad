"""Paged K/V entry point: the same attention with K/V scattered over page pools.

Whatever the page size, the paged call runs the same kernels as the packed call, and with the same split plan when
neither is given the batch's token count (with it, a ragged batch may be cut into equal shares of the concatenated
tokens, differently for the two layouts), so its output must then equal the packed call's bit for bit; the cases are
also checked against the CPU oracle on the gathered (packed) inputs.  Unused pool rows are NaN: reading one poisons
the output.
"""
import pytest
import torch

from decoding_attention_amd import _lib, decoding_attn_fwd, decoding_attn_paged_fwd
from decoding_attention_amd import workloads as wl
from tests.gpu_util import TOL, check_against_oracle, run_hip_ex

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _run_both(w, page_size, combined=False, hint=0):
    """Packed and paged call on the same values, both with the token-count hint `hint` (0 = not given)."""
    pk = wl.to_pages(w, page_size, seed=3, combined=combined).to(DEV)
    wd = w.to(DEV)
    dense = run_hip_ex(w, hint)
    paged = decoding_attn_paged_fwd(wd.q, pk.k_pages, pk.v_pages, pk.block_table, pk.seq_lens, w.max_seq_k, w.dim_v,
                                    w.is_alibi, total_k=hint)
    torch.cuda.synchronize()
    return dense, paged.cpu()


SHAPES = {
    "mha": dict(batch=6, head_q=8, head_k=8, dim=128, dim_v=128, seq_k=700, dtype=torch.float16),
    "mha_d64": dict(batch=3, head_q=4, head_k=4, dim=64, dim_v=64, seq_k=300, dtype=torch.bfloat16),
    "gqa": dict(batch=9, head_q=32, head_k=8, dim=128, dim_v=128, seq_k=1500, dtype=torch.bfloat16),
    "gqa_d256": dict(batch=4, head_q=16, head_k=4, dim=256, dim_v=256, seq_k=600, dtype=torch.float16),
    "mqa": dict(batch=5, head_q=32, head_k=1, dim=128, dim_v=128, seq_k=1100, dtype=torch.float16, is_alibi=True),
    "mla": dict(batch=5, head_q=128, head_k=1, dim=576, dim_v=512, seq_k=900, dtype=torch.float16),
    "mla_h16": dict(batch=3, head_q=16, head_k=1, dim=576, dim_v=512, seq_k=400, dtype=torch.bfloat16),
}


def _workload(name, **over):
    args = dict(SHAPES[name])
    args.update(over)
    return wl.make_workload(args.pop("batch"), args.pop("head_q"), args.pop("head_k"), args.pop("dim"),
                            args.pop("dim_v"), args.pop("seq_k"), args.pop("dtype"), seed=5, varlen=True,
                            name="paged_" + name, **args)


@pytest.mark.parametrize("page_size", [1, 4, 16, 32, 64, 256])
@pytest.mark.parametrize("name", list(SHAPES))
def test_tile_sized_pages_match_the_packed_call_bit_for_bit(name, page_size):
    w = _workload(name)
    dense, paged = _run_both(w, page_size)
    assert torch.isfinite(paged.float()).all()
    assert torch.equal(dense.view(torch.int16), paged.view(torch.int16))


@pytest.mark.parametrize("name", ["gqa", "mqa", "mla"])
def test_with_the_token_count_hint(name):
    """Both calls are given the batch's token count: each may choose another split plan for the ragged batch, so
    the outputs agree within the tolerance (and the paged one with the oracle)."""
    w = _workload(name)
    dense, paged = _run_both(w, 64, hint=int(w.k.shape[0]))
    assert (dense.float() - paged.float()).abs().max().item() <= TOL[w.q.dtype]
    check_against_oracle(w, paged)


@pytest.mark.parametrize("page_size", [1, 2, 4, 8])
@pytest.mark.parametrize("name", ["mla", "mla_h16"])
def test_latent_kernel_takes_small_pages_with_a_lookup_per_row(name, page_size):
    """Pages under 16 tokens (token-level paging included): the latent kernel's per-row lookup form; same arithmetic
    as the packed call, same bits."""
    w = _workload(name)
    dense, paged = _run_both(w, page_size)
    assert torch.isfinite(paged.float()).all()
    assert torch.equal(dense.view(torch.int16), paged.view(torch.int16))


@pytest.mark.parametrize("name", ["mla", "mla_h16"])
def test_latent_kernel_takes_16_token_pages(name):
    """The latent kernel fetches a tile as two runs of 16 tokens, so 16-token pages (a common cache block size) stay
    on it: same kernel and plan as the packed call, same bits."""
    w = _workload(name)
    dense, paged = _run_both(w, 16)
    assert torch.isfinite(paged.float()).all()
    assert torch.equal(dense.view(torch.int16), paged.view(torch.int16))
    lib = _lib.load()
    shape = (w.max_seq_k, w.batch, w.head_q, 1, 576, 512)
    assert lib.da_workspace_bytes_paged(*shape, 0, 16) == lib.da_workspace_bytes_paged(*shape, 0, 64)


@pytest.mark.parametrize("page_size", [1, 4, 8, 16])
@pytest.mark.parametrize("name", ["mha", "gqa", "mqa", "mla_h16"])
def test_small_pages_match_the_oracle(name, page_size):
    w = _workload(name, seq_k=260)
    _, paged = _run_both(w, page_size)
    check_against_oracle(w, paged)


def test_combined_kv_pool_passed_as_views():
    """One [pages, 2, page_size, head_k, dim] pool: K and V halves are strided views with the pool's page stride."""
    w = _workload("gqa")
    dense, paged = _run_both(w, 64, combined=True)
    assert torch.equal(dense.view(torch.int16), paged.view(torch.int16))
    w = _workload("mha", seq_k=200)
    _, paged = _run_both(w, 1, combined=True)  # one token per page, as the reference's comparison benchmark sets up
    check_against_oracle(w, paged)


def test_empty_and_single_token_sequences_and_output_argument():
    w = wl.make_workload(4, 32, 8, 128, 128, 2100, torch.float16, seed=9, varlen=True)
    # force an empty and a one-token sequence
    lens = list(w.lengths)
    lens[1], lens[2] = 0, 1
    cu = w.cu_seq_k.tolist()
    ks = [w.k[cu[b]:cu[b] + lens[b]] for b in range(4)]
    vs = [w.v[cu[b]:cu[b] + lens[b]] for b in range(4)]
    t = torch.tensor(lens, dtype=torch.int32)
    w2 = wl.Workload("paged_ragged", w.q, torch.cat(ks), torch.cat(vs), wl.get_cu_seq(t), max(lens), 128, False, lens)
    pk = wl.to_pages(w2, 64, seed=1).to(DEV)
    out = torch.full((4, 32, 128), float("nan"), dtype=torch.float16, device=DEV)
    res = decoding_attn_paged_fwd(w2.q.to(DEV), pk.k_pages, pk.v_pages, pk.block_table, pk.seq_lens, w2.max_seq_k, 128,
                                  False, out=out)
    torch.cuda.synchronize()
    assert res.data_ptr() == out.data_ptr()
    assert (out[1] == 0).all()
    assert torch.equal(out[2].cpu(), w2.v[lens[0]:lens[0] + 1].repeat_interleave(4, dim=1)[0])
    check_against_oracle(w2, out.cpu())


def test_full_size_gqa_and_mla_paged():
    """The benchmark shapes with 64-token pages: bit-equal to the packed call."""
    for w in (wl.config_gqa_fixed(batch=64, seq_k=4096), wl.config_mla(64, 4096)):
        dense, paged = _run_both(w, 64)
        assert torch.equal(dense.view(torch.int16), paged.view(torch.int16)), w.name


def test_c_abi_argument_errors():
    lib = _lib.load()
    w = _workload("mha")
    pk = wl.to_pages(w, 64).to(DEV)
    q = w.q.to(DEV)
    o = torch.empty(w.batch, 8, 128, dtype=torch.float16, device=DEV)

    def call(page_size=64, max_blocks=None, table=pk.block_table, lens=pk.seq_lens, k_stride=None):
        return lib.da_decoding_attn_paged(
            q.data_ptr(), pk.k_pages.data_ptr(), pk.v_pages.data_ptr(), o.data_ptr(),
            None if table is None else table.data_ptr(), None if lens is None else lens.data_ptr(), w.max_seq_k,
            w.batch, 8, 8, 128, 128, page_size, pk.block_table.shape[1] if max_blocks is None else max_blocks,
            64 * 8 * 128 if k_stride is None else k_stride, 64 * 8 * 128, 0, 0, 0.0, None, 0, None, 0, None)

    assert call() == 0, _lib.last_error()
    for kwargs, word in [(dict(page_size=48), "power of two"), (dict(max_blocks=1), "cannot hold"),
                         (dict(table=None), "block_table is null"), (dict(lens=None), "seq_lens is null"),
                         (dict(k_stride=100), "k_page_stride")]:
        assert call(**kwargs) == _lib.DA_ERR_INVALID_ARGUMENT
        assert word in _lib.last_error()
    torch.cuda.synchronize()
