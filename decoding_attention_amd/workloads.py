"""Seeded synthetic workloads and the work formulas used to report them.

Inputs are drawn on the CPU from ``torch.Generator().manual_seed(seed)`` in the fixed
order q, k, v, lengths as fp32 N(0,1) and then cast (round-to-nearest-even) to
fp16/bf16, so a CPU checker and the GPU kernel see identical bits whatever the device.

The packed layout is the reference's: q [batch, head_q, dim], k [total_k, head_k, dim],
v [total_k, head_k, dim_v] or None for the latent (MLA) form where V is the first
dim_v columns of K, and cu_seq_k = int32 prefix offsets built as in the reference's
``get_cu_seq`` (reference tests/test_decoding_attn.py:23-31).
"""
from dataclasses import dataclass
from typing import List, Optional

import torch


@dataclass
class Workload:
    name: str
    q: torch.Tensor
    k: torch.Tensor
    v: Optional[torch.Tensor]
    cu_seq_k: torch.Tensor
    max_seq_k: int
    dim_v: int
    is_alibi: bool
    lengths: List[int]

    @property
    def batch(self):
        return self.q.shape[0]

    @property
    def head_q(self):
        return self.q.shape[1]

    @property
    def head_k(self):
        return self.k.shape[1]

    @property
    def dim(self):
        return self.q.shape[2]

    def to(self, device):
        return Workload(self.name, self.q.to(device), self.k.to(device),
                        None if self.v is None else self.v.to(device), self.cu_seq_k.to(device),
                        self.max_seq_k, self.dim_v, self.is_alibi, self.lengths)


def get_cu_seq(seqs: torch.Tensor) -> torch.Tensor:
    """[batch] lengths -> [batch+1] int32 prefix offsets with a leading zero."""
    return torch.nn.functional.pad(seqs.cumsum(dim=0, dtype=torch.int32), (1, 0))


def make_workload(batch, head_q, head_k, dim, dim_v, seq_k, dtype, *, seed=0, varlen=False, latent=None,
                  is_alibi=False, name=None, min_len=1, device="cpu") -> Workload:
    """Build one workload.

    ``seq_k`` is the common length, or the inclusive upper bound of uniform random lengths
    when ``varlen`` is set.  ``latent`` (default: dim != dim_v) makes V alias K[..., :dim_v].
    ``device`` other than the CPU draws q/k/v there (a different random stream: for timing, not for the parity
    tests, whose inputs are the CPU stream's).
    """
    if latent is None:
        latent = dim != dim_v
    g = torch.Generator(device=device).manual_seed(seed)
    if varlen:
        # lengths are drawn last in the stream order, but are needed first to size K/V;
        # use a generator forked from the same seed so that the order stays reproducible.
        gl = torch.Generator(device="cpu").manual_seed(seed + 0x5EED)
        lens = torch.randint(min_len, seq_k + 1, (batch,), generator=gl, dtype=torch.int32)
    else:
        lens = torch.full((batch,), seq_k, dtype=torch.int32)
    total_k = int(lens.sum().item())
    on_cpu = str(device) == "cpu"
    draw_dtype = torch.float32 if on_cpu else dtype  # (the CPU stream is fp32 rounded to 16 bits)
    q = torch.randn(batch, head_q, dim, generator=g, dtype=draw_dtype, device=device).to(dtype)
    k = torch.randn(total_k, head_k, dim, generator=g, dtype=draw_dtype, device=device).to(dtype)
    v = None
    if not latent:
        v = torch.randn(total_k, head_k, dim_v, generator=g, dtype=draw_dtype, device=device).to(dtype)
    cu = get_cu_seq(lens).to(device)
    max_seq_k = int(lens.max().item()) if batch > 0 else 0
    if name is None:
        name = f"b{batch}_hq{head_q}_hk{head_k}_d{dim}_dv{dim_v}_sk{seq_k}{'_var' if varlen else ''}_" \
               f"{'bf16' if dtype == torch.bfloat16 else 'fp16'}{'_alibi' if is_alibi else ''}"
    return Workload(name, q, k, v, cu, max_seq_k, dim_v, is_alibi, [int(x) for x in lens.tolist()])


# The five benchmark configurations (fixed shapes; sweeps take the swept value as an argument).
@dataclass
class PagedKV:
    """A packed workload's K/V scattered into page pools (see `to_pages`)."""
    k_pages: torch.Tensor               # [pages, page_size, head_k, dim] (a view of `pool` when combined)
    v_pages: Optional[torch.Tensor]     # [pages, page_size, head_k, dim_v] or None (latent form)
    block_table: torch.Tensor           # int32 [batch, max_blocks]
    seq_lens: torch.Tensor              # int32 [batch]
    page_size: int
    pool: Optional[torch.Tensor] = None  # [pages, 2, page_size, head_k, dim] when combined

    def to(self, device):
        if self.pool is not None:
            pool = self.pool.to(device)
            return PagedKV(pool[:, 0], pool[:, 1], self.block_table.to(device), self.seq_lens.to(device),
                           self.page_size, pool)
        return PagedKV(self.k_pages.to(device), None if self.v_pages is None else self.v_pages.to(device),
                       self.block_table.to(device), self.seq_lens.to(device), self.page_size)


def to_pages(w: Workload, page_size: int, *, seed=0, combined=False, spare_pages=3, poison=True) -> PagedKV:
    """Scatter the packed K/V of `w` into page pools with shuffled page ids.

    Unused pages, the unused tail of each sequence's last page and unused block-table entries are poisoned (NaN
    rows, page id -1 replaced by an out-of-sequence valid id) so that a kernel that reads past a sequence's end
    shows up in the output (poison=False fills with zeros instead, for integer-typed byte views).  combined=True builds one [pages, 2, page_size, head_k, dim] pool (K and V interleaved
    per page, dim == dim_v) and returns its two halves as views.
    """
    g = torch.Generator(device="cpu").manual_seed(seed)
    lens = w.lengths
    blocks = [(n + page_size - 1) // page_size for n in lens]
    max_blocks = max(1, max(blocks))
    n_pages = sum(blocks) + spare_pages
    order = torch.randperm(n_pages, generator=g).tolist()
    nan = float("nan") if poison else 0
    if combined:
        assert w.v is not None and w.dim == w.dim_v
        pool = torch.full((n_pages, 2, page_size, w.head_k, w.k.shape[-1]), nan, dtype=w.k.dtype)
        k_pages, v_pages = pool[:, 0], pool[:, 1]
    else:
        pool = None
        # (row widths from the tensors themselves: an int4 cache holds two elements to a byte)
        k_pages = torch.full((n_pages, page_size, w.head_k, w.k.shape[-1]), nan, dtype=w.k.dtype)
        v_pages = None if w.v is None else torch.full((n_pages, page_size, w.head_k, w.v.shape[-1]), nan, dtype=w.k.dtype)
    # unused table entries point at a spare (all-NaN) page
    table = torch.full((w.batch, max_blocks), order[-1], dtype=torch.int32)
    cu = w.cu_seq_k.tolist()
    nxt = 0
    for b, n in enumerate(lens):
        for i in range(blocks[b]):
            page = order[nxt]
            nxt += 1
            table[b, i] = page
            lo, hi = cu[b] + i * page_size, min(cu[b] + (i + 1) * page_size, cu[b] + n)
            k_pages[page, :hi - lo] = w.k[lo:hi]
            if v_pages is not None:
                v_pages[page, :hi - lo] = w.v[lo:hi]
    return PagedKV(k_pages, v_pages, table, torch.tensor(lens, dtype=torch.int32), page_size, pool)


def config_mha_cpu_case(seed=0):
    return make_workload(1, 32, 32, 128, 128, 128, torch.float16, seed=seed, name="C0_mha_fp16_b1_sk128")


def config_mha_sweep(batch, seq_k, seed=0):
    return make_workload(batch, 32, 32, 128, 128, seq_k, torch.float16, seed=seed,
                         name=f"C1_mha_fp16_b{batch}_sk{seq_k}")


def config_gqa_varlen(seed=0, batch=64, max_len=8192):
    return make_workload(batch, 32, 8, 128, 128, max_len, torch.bfloat16, seed=seed, varlen=True,
                         name=f"C2_gqa_bf16_b{batch}_varlen{max_len}")


def config_gqa_fixed(seed=0, batch=64, seq_k=4096):
    return make_workload(batch, 32, 8, 128, 128, seq_k, torch.bfloat16, seed=seed,
                         name=f"C2_gqa_bf16_b{batch}_sk{seq_k}")


def config_mqa_alibi(seed=0, batch=32, seq_k=4096):
    return make_workload(batch, 32, 1, 128, 128, seq_k, torch.float16, seed=seed, is_alibi=True,
                         name=f"C3_mqa_fp16_alibi_b{batch}_sk{seq_k}")


def config_mla(batch, seq_k, seed=0, dtype=torch.float16, head_q=128):
    return make_workload(batch, head_q, 1, 576, 512, seq_k, dtype, seed=seed, latent=True,
                         name=f"C4_mla_{'bf16' if dtype == torch.bfloat16 else 'fp16'}_b{batch}_sk{seq_k}")


def algorithmic_bytes(batch, head_q, head_k, dim, dim_v, total_k, v_distinct, elem_bytes=2) -> int:
    """HBM bytes the operation must move: Q, K, (V if it is its own buffer), O once each, plus cu_seq_k."""
    elems = batch * head_q * dim + total_k * head_k * dim + batch * head_q * dim_v
    if v_distinct:
        elems += total_k * head_k * dim_v
    return elem_bytes * elems + 4 * (batch + 1)


def algorithmic_flops(head_q, dim, dim_v, total_k) -> int:
    """2 * sum(len) * head_q * (dim + dim_v), the reference's count (csrc/common/tester.h:270)."""
    return 2 * total_k * head_q * (dim + dim_v)


def reference_formula_bytes(batch, head_q, head_k, dim, dim_v, seq_k, elem_bytes=2) -> int:
    """The reference's bandwidth numerator (csrc/common/tester.h:273-276); it leaves V out."""
    return elem_bytes * (batch * head_q * dim + batch * seq_k * head_k * dim + batch * head_q * dim_v)


def workload_bytes(w: Workload) -> int:
    return algorithmic_bytes(w.batch, w.head_q, w.head_k, w.dim, w.dim_v, int(w.k.shape[0]), w.v is not None)


def workload_flops(w: Workload) -> int:
    return algorithmic_flops(w.head_q, w.dim, w.dim_v, int(w.k.shape[0]))
