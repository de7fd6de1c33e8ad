#!/usr/bin/env python3
"""Benchmark of the decoding-attention hot path on one MI355X.

Default run (one JSON line on stdout):
  * primary workload — GQA decode, bf16, batch 64, 32 query / 8 KV heads, head_dim 128, seq_k 4096
    (K/V packed [batch*seq_k, 8, 128], distinct V): one "step" = one call of the op;
  * alongside — MLA decode, fp16, batch 64, 128 query heads over one 576-wide latent head, seq_k 4096,
    V = K[..., :512];
  * the CPU oracle timed on the host cores for the same primary workload (bounded sample).

`value` is the achieved HBM rate of the primary workload: algorithmic bytes (Q, K, V, O once each +
cu_seq_k) divided by the mean time of one call, inputs resident in HBM.  Calls are timed with events on the
stream the kernels are launched on.  Working sets below 512 MB are rotated over several input copies so the
256 MB Infinity Cache cannot serve them.

`--sweep mha|mla` prints the reference's two sweeps for that head shape (its `Benchmark Seq` section at batch 1,
then its `Benchmark Batch` section, with the reference's full lists) in the reference's log format, which the
reference's plot script reads (reference benchmarks/python/benchmark_decoding_attn.py:248-249 and :303-330,
formulas :52-57); `--sweep baseline` the remaining benchmark shapes; `--sweep all` all three.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0      # MI355X HBM3E, published
MFMA_PEAK_TFLOPS = 2500.0   # MI355X dense fp16/bf16 MFMA, published
# HBM bytes per call from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of `bench.py --only gqa|mla`, each counter
# scaled by what it reads for a 1 GiB device copy: profiles/hbm_traffic.json, written from the counter runs by
# `python -m decoding_attention_amd.profile_traffic` (profiles/*_hbm_traffic.md describe the runs).  A figure belongs
# to the launch plan it was measured under; when the library plans the workload differently, or the file is not there,
# the bench line carries null instead.
TRAFFIC_JSON = os.path.join(ROOT, "profiles", "hbm_traffic.json")


def measured_traffic(key, plan):
    try:
        with open(TRAFFIC_JSON) as f:
            rec = json.load(f)[key]
    except (OSError, KeyError, ValueError):
        return None
    same = all(plan.get(k) == v for k, v in rec["plan"].items())
    return rec["bytes"] if same else None


def _time_calls(torch, fn_list, steps, warmup):
    """Mean milliseconds per call over `steps` back-to-back calls, rotating over fn_list, and the fastest of a few
    calls timed one by one with a host synchronisation after each (that one includes the launch gap between the
    sweep and the merge kernel, so it can exceed the back-to-back mean)."""
    n = len(fn_list)
    for i in range(warmup):
        fn_list[i % n]()
    torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    start.record()
    for i in range(steps):
        fn_list[i % n]()
    end.record()
    torch.cuda.synchronize()
    mean_ms = start.elapsed_time(end) / steps
    # per-call minimum from a short individually-timed tail
    mins = []
    for i in range(min(steps, 10)):
        s = torch.cuda.Event(enable_timing=True)
        e = torch.cuda.Event(enable_timing=True)
        s.record()
        fn_list[i % n]()
        e.record()
        torch.cuda.synchronize()
        mins.append(s.elapsed_time(e))
    return mean_ms, min(mins)


def _device_copies(torch, w, dev, min_total_bytes=768 << 20):
    """Enough independent device copies of the inputs that consecutive calls cannot hit in the Infinity Cache."""
    from decoding_attention_amd import workloads as wl

    nbytes = wl.workload_bytes(w)
    ncopies = 1 if nbytes >= (512 << 20) else max(2, -(-min_total_bytes // nbytes))
    ncopies = min(ncopies, 64)
    copies = []
    for _ in range(ncopies):
        wd = w.to(dev)
        copies.append(wd if len(copies) == 0 else type(wd)(
            wd.name, wd.q.clone(), wd.k.clone(), None if wd.v is None else wd.v.clone(), wd.cu_seq_k.clone(),
            wd.max_seq_k, wd.dim_v, wd.is_alibi, wd.lengths))
    return copies


def measure(torch, w, steps, warmup, page_size=0, kv_fp8=False, kv_int8=False, kv_int4=False, kv_int4_tok=False,
            kv_int8_tok=False, kv_int4_g64=False, kv_int8_g64=False):
    from decoding_attention_amd import _lib, decoding_attn_fwd
    from decoding_attention_amd import workloads as wl

    dev = torch.device("cuda:0")
    copies = _device_copies(torch, w, dev)
    outs = []

    def make(c):
        if kv_int4_tok or kv_int8_tok or kv_int4_g64 or kv_int8_g64:  # a (scale, zero) pair per row, or per 64 elements
            from decoding_attention_amd import (quantize_int4_per_group, quantize_int4_per_token,
                                                quantize_int8_per_group, quantize_int8_per_token)
            quant = (quantize_int4_per_group if kv_int4_g64 else quantize_int8_per_group if kv_int8_g64 else
                     quantize_int4_per_token if kv_int4_tok else quantize_int8_per_token)
            k4, kp = quant(c.k)
            v4, vp = quant(c.v)

            def call_tok():
                outs[:] = [decoding_attn_fwd(c.q, k4, v4, c.cu_seq_k, c.max_seq_k, c.dim_v, c.is_alibi, k_scale=kp,
                                             v_scale=vp)]
            return call_tok
        if kv_fp8 or kv_int8 or kv_int4:  # K/V as FP8 (e4m3), int8 or int4 with per-head scales; q and o stay 16-bit
            def quantise(x, step):
                if kv_int4:
                    from decoding_attention_amd import pack_int4
                    return pack_int4(torch.round(x.float() / step).clamp(-8, 7).to(torch.int8))
                if kv_int8:
                    return torch.round(x.float() / step).clamp(-128, 127).to(torch.int8)
                return (x.float() / step).to(torch.float8_e4m3fn)

            step = 3.0 / 7 if kv_int4 else (4.0 / 127 if kv_int8 else 0.02)
            ks = torch.full((w.head_k,), step, device=dev)
            k8 = quantise(c.k, step)
            v8 = None if c.v is None else quantise(c.v, step)  # (latent form: V is in K)

            def call_fp8():
                outs[:] = [decoding_attn_fwd(c.q, k8, v8, c.cu_seq_k, c.max_seq_k, c.dim_v, c.is_alibi, k_scale=ks,
                                             v_scale=ks)]
            return call_fp8
        if page_size:
            from decoding_attention_amd import decoding_attn_paged_fwd

            pk = wl.to_pages(w, page_size, seed=len(outs)).to(dev)
            total = int(w.k.shape[0])

            def call_paged():
                outs[:] = [decoding_attn_paged_fwd(c.q, pk.k_pages, pk.v_pages, pk.block_table, pk.seq_lens,
                                                   c.max_seq_k, c.dim_v, c.is_alibi, total_k=total)]
            return call_paged

        def call():
            outs[:] = [decoding_attn_fwd(c.q, c.k, c.v, c.cu_seq_k, c.max_seq_k, c.dim_v, c.is_alibi)]
        return call

    fns = [make(c) for c in copies]
    mean_ms, min_ms = _time_calls(torch, fns, steps, warmup)
    assert torch.isfinite(outs[0].float()).all()
    nbytes = wl.workload_bytes(w)
    per64 = kv_int4_g64 or kv_int8_g64
    if kv_fp8 or kv_int8 or kv_int4 or kv_int4_tok or kv_int8_tok or per64:  # one byte (half a byte) per K/V element
        kv_elems = int(w.k.numel() + (w.v.numel() if w.v is not None else 0))
        nbytes = wl.algorithmic_bytes(w.batch, w.head_q, w.head_k, w.dim, w.dim_v, int(w.k.shape[0]), w.v is not None,
                                      elem_bytes=2) - (kv_elems * 3 // 2 if (kv_int4 or kv_int4_tok or kv_int4_g64) else kv_elems)
        if kv_int4_tok or kv_int8_tok or per64:  # two float pairs per (token, KV head), or per 64 elements of it
            nbytes += int(w.k.shape[0]) * w.head_k * 16 * (w.dim // 64 if per64 else 1)
    flops = wl.workload_flops(w)
    # the plan of the call that was timed
    plan = _lib.plan(w.max_seq_k, w.batch, w.head_q, w.head_k, w.dim, w.dim_v,
                     total_k=int(w.k.shape[0]),
                     distinct_v=w.v is not None and w.dim != w.dim_v, page_size=page_size,
                     kv_bits=_lib.KV_BITS_INT4_GROUP64 if kv_int4_g64 else _lib.KV_BITS_INT8_GROUP64 if kv_int8_g64 else
                     _lib.KV_BITS_INT4_PER_TOKEN if kv_int4_tok else _lib.KV_BITS_INT8_PER_TOKEN if kv_int8_tok else
                     4 if kv_int4 else 8 if (kv_fp8 or kv_int8) else 16)
    return {
        "workload": w.name,
        "us_per_call": mean_ms * 1e3,
        "us_isolated_call_min": min_ms * 1e3,
        "algorithmic_bytes": nbytes,
        "algorithmic_flops": flops,
        "hbm_GBps": nbytes / (mean_ms * 1e-3) / 1e9,
        "hbm_frac_of_peak": nbytes / (mean_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
        "tflops": flops / (mean_ms * 1e-3) / 1e12,
        "mfma_frac_of_peak": flops / (mean_ms * 1e-3) / 1e12 / MFMA_PEAK_TFLOPS,
        "input_copies_rotated": len(copies),
        "plan": plan,
    }


def cpu_baseline(torch, w, budget_s=20.0):
    """The CPU oracle on the host cores: one thread (what the reference's CPU path does) on as many whole
    sequences of the workload as fit the time budget, scaled to the full batch when it is a subset."""
    from decoding_attention_amd import workloads as wl
    from oracle import oracle

    def sub(nseq):
        cu = w.cu_seq_k.tolist()
        end = cu[nseq]
        return (w.q[:nseq].contiguous(), w.k[:end].contiguous(), None if w.v is None else w.v[:end].contiguous(),
                w.cu_seq_k[:nseq + 1].contiguous())

    def run(nseq, threads):
        q, k, v, cu = sub(nseq)
        t0 = time.perf_counter()
        oracle.attn_cpu(q, k, v, cu, w.max_seq_k, w.dim_v, w.is_alibi, nthreads=threads)
        return time.perf_counter() - t0

    t1 = run(1, 1)
    nseq = int(max(1, min(w.batch, budget_s / max(t1, 1e-6))))
    t = run(nseq, 1) if nseq > 1 else t1
    full_s = t * w.batch / nseq
    ncores = oracle.max_threads()
    tm = run(min(w.batch, max(nseq, ncores)), ncores) * w.batch / min(w.batch, max(nseq, ncores))
    nbytes = wl.workload_bytes(w)
    return {
        "value": nbytes / full_s / 1e12,
        "unit": "TB/s",
        "cores": 1,
        "kind": "port",
        "sample": f"{nseq} of {w.batch} sequences of {w.name}, single thread, {t:.2f} s measured"
                  + ("" if nseq == w.batch else ", scaled linearly to the full batch (extrapolated)"),
        "us_per_call": full_s * 1e6,
        "all_cores": {"cores": ncores, "us_per_call": tm * 1e6, "value": nbytes / tm / 1e12},
    }


def call_and_kernel_us(torch, w, reps=50, warmup=5, group=4):
    """Mean duration of the whole call and of its sweep kernel alone, from one loop that alternates groups of
    `group` calls and `group` kernel-alone launches on the launch stream with an event between the groups (so both
    see the same clocks and kernel <= call; an event costs a few microseconds of stream time, which the group
    spreads).  The call is the C-ABI entry with a caller-owned workspace; the kernel alone is the probe library's
    sweep-only entry (the same code without the merge launch).  Inputs rotate over several device copies as in
    measure()."""
    from decoding_attention_amd import _lib

    lib, probe = _lib.load(), _lib.load_probe()
    dev = torch.device("cuda:0")
    copies = _device_copies(torch, w, dev)
    total = int(w.k.shape[0])
    o = torch.empty(w.batch, w.head_q, w.dim_v, dtype=w.q.dtype, device=dev)
    n = lib.da_workspace_bytes(w.max_seq_k, w.batch, w.head_q, w.head_k, w.dim, w.dim_v, total)
    ws = torch.empty(max(n, 16), dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    bf16 = int(w.q.dtype == torch.bfloat16)

    def full(c):
        rc = lib.da_decoding_attn_ex(c.q.data_ptr(), c.k.data_ptr(), None if c.v is None else c.v.data_ptr(),
                                     o.data_ptr(), c.cu_seq_k.data_ptr(), w.max_seq_k, w.batch, w.head_q, w.head_k,
                                     w.dim, w.dim_v, int(w.is_alibi), bf16, 0.0, None, total, ws.data_ptr(), n, stream)
        assert rc == 0, _lib.last_error()

    def sweep(c):
        rc = probe.da_probe_sweep_only(c.q.data_ptr(), c.k.data_ptr(), None if c.v is None else c.v.data_ptr(),
                                       o.data_ptr(), c.cu_seq_k.data_ptr(), w.max_seq_k, w.batch, w.head_q, w.head_k,
                                       w.dim, w.dim_v, int(w.is_alibi), bf16, total, ws.data_ptr(), n, stream)
        assert rc == 0, probe.da_last_error().decode("utf-8", "replace")

    for i in range(warmup):
        full(copies[i % len(copies)])
        sweep(copies[i % len(copies)])
    torch.cuda.synchronize()
    rounds = max(1, -(-reps // group))
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(2 * rounds + 1)]
    ev[0].record()
    j = 0
    for i in range(rounds):
        for _ in range(group):
            full(copies[j % len(copies)])
            j += 1
        ev[2 * i + 1].record()
        for _ in range(group):
            sweep(copies[j % len(copies)])
            j += 1
        ev[2 * i + 2].record()
    torch.cuda.synchronize()
    call_ms = sum(ev[2 * i].elapsed_time(ev[2 * i + 1]) for i in range(rounds)) / (rounds * group)
    kern_ms = sum(ev[2 * i + 1].elapsed_time(ev[2 * i + 2]) for i in range(rounds)) / (rounds * group)
    return call_ms * 1e3, kern_ms * 1e3


def stream_read_GBps(torch, nbytes=1 << 30, reps=20):
    """Bandwidth of the library's plain streaming-read kernel over a fresh buffer: what HBM gives a kernel that
    only reads (the practical ceiling for the bandwidth-bound attention kernels on this GPU)."""
    from decoding_attention_amd import _lib

    lib = _lib.load_probe()
    buf = torch.empty(nbytes, dtype=torch.uint8, device="cuda:0").fill_(1)
    stream = torch.cuda.current_stream().cuda_stream
    for _ in range(3):
        assert lib.da_probe_stream_read(buf.data_ptr(), nbytes, None, stream) == 0
    torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(reps):
        lib.da_probe_stream_read(buf.data_ptr(), nbytes, None, stream)
    end.record()
    torch.cuda.synchronize()
    ms = start.elapsed_time(end) / reps
    return lib.da_probe_stream_read_bytes(nbytes) / (ms * 1e-3) / 1e9


def mfma_sustained_TFLOPs(torch, operand_std=1.0, iters=2000, reps=10):
    """Matrix rate the chip sustains under its power limit: a kernel of nothing but fp16 matrix instructions on every
    SIMD (each fed by one LDS read), operands N(0, operand_std) -- the practical ceiling for the latent kernel's
    matrix work.  With operand_std = 0 (all zeros) the same kernel runs near the nominal clock."""
    from decoding_attention_amd import _lib

    probe = _lib.load_probe()
    g = torch.Generator(device="cpu").manual_seed(0)
    ops = (torch.randn(16384, generator=g) * operand_std).to(torch.float16).to("cuda:0")
    sink = torch.empty(65536, dtype=torch.float32, device="cuda:0")
    stream = torch.cuda.current_stream().cuda_stream
    for _ in range(3):
        assert probe.da_probe_mfma_rate(ops.data_ptr(), iters, sink.data_ptr(), stream) == 0
    torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(reps):
        probe.da_probe_mfma_rate(ops.data_ptr(), iters, sink.data_ptr(), stream)
    end.record()
    torch.cuda.synchronize()
    ms = start.elapsed_time(end) / reps
    return probe.da_probe_mfma_rate_flops(iters) / (ms * 1e-3) / 1e12


def run_default(args):
    import torch

    from decoding_attention_amd import workloads as wl

    if not torch.cuda.is_available():
        print("bench.py needs a GPU (no CPU fallback exists for the op)", file=sys.stderr)
        return 2
    if args.calibrate_copy:
        # a device-to-device copy of known size, so that a profiler's FETCH_SIZE / WRITE_SIZE counters can be scaled
        src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda:0").fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    gqa_w = wl.config_gqa_fixed(seed=0)
    if args.only == "mla":
        mla = measure(torch, wl.config_mla(64, 4096), max(50, args.steps), max(5, args.warmup))
        print(json.dumps({"only": "mla", **mla}))
        return 0
    gqa = measure(torch, gqa_w, args.steps, args.warmup)
    if args.only == "gqa":
        print(json.dumps({"only": "gqa", **gqa}))
        return 0
    mla = None
    if not args.no_mla:
        # (under this kernel the chip's clock moves in slow waves, 82-119 us per launch over some hundred launches in
        # a kernel trace: a long warm-up and a long run, so that the mean is the sustained one)
        mla_w = wl.config_mla(64, 4096)
        mla = measure(torch, mla_w, max(300, args.steps), max(100, args.warmup))
        mla["interleaved_call_us"], mla["kernel_us"] = call_and_kernel_us(torch, mla_w, reps=max(150, args.steps),
                                                                           warmup=max(10, args.warmup))
        mfma_rand = mfma_sustained_TFLOPs(torch, 1.0)
        mfma_zero = mfma_sustained_TFLOPs(torch, 0.0)
    stream_gbps = stream_read_GBps(torch)
    gqa_call_us, sweep_us = call_and_kernel_us(torch, gqa_w, reps=max(30, args.steps), warmup=max(5, args.warmup))
    sweep_gbps = gqa["algorithmic_bytes"] / (sweep_us * 1e-6) / 1e9
    cpu = None if args.no_cpu else cpu_baseline(torch, gqa_w, args.cpu_budget)

    line = {
        "metric": "decode attn achieved HBM TB/s, GQA bf16 b64 seq_k 4096 (us/call and MLA fp16 b64 alongside)",
        "value": gqa["hbm_GBps"] / 1e3,
        "unit": "TB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": gqa["us_per_call"] / 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "GQA decode bf16, batch 64, 32 q heads / 8 kv heads, head_dim 128, seq_k 4096, "
                               "packed K/V [262144, 8, 128], scale 1/sqrt(128), seed 0",
                   "name": gqa["workload"], "plan": gqa["plan"]},
        "us_per_call": gqa["us_per_call"],
        "us_isolated_call_min": gqa["us_isolated_call_min"],
        "pct_hbm_peak": 100.0 * gqa["hbm_frac_of_peak"],
        # the dominant kernel (the grouped-head sweep) on its own: algorithmic bytes of the call over its average
        # launch duration, timed in this run with events on the launch stream
        "roofline": {"bound": "hbm", "achieved": sweep_gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": sweep_gbps / HBM_PEAK_GBPS, "traffic": measured_traffic("gqa", gqa["plan"]),
                     "kernel": "gqa_mfma_kernel", "kernel_us": sweep_us, "interleaved_call_us": gqa_call_us,
                     "whole_call": {"achieved": gqa["hbm_GBps"], "frac": gqa["hbm_frac_of_peak"],
                                    "kernels": "gqa_mfma_kernel + reduce_kernel"},
                     # measured in this run: a kernel that only streams 1 GiB from HBM, and the sweep against it
                     "stream_read_GBps": stream_gbps, "frac_of_stream_read": sweep_gbps / stream_gbps},
        "cpu_baseline": cpu,
    }
    if mla is not None:
        line["mla"] = {
            "workload": "MLA decode fp16, batch 64, 128 q heads / 1 latent kv head, dims 576/512, seq_k 4096, "
                        "V = K[..., :512]",
            "us_per_call": mla["us_per_call"], "us_isolated_call_min": mla["us_isolated_call_min"],
            "hbm_TBps": mla["hbm_GBps"] / 1e3, "pct_hbm_peak": 100.0 * mla["hbm_frac_of_peak"],
            "tflops": mla["tflops"], "pct_mfma_peak": 100.0 * mla["mfma_frac_of_peak"],
            "algorithmic_bytes": mla["algorithmic_bytes"], "algorithmic_flops": mla["algorithmic_flops"],
            "input_copies_rotated": mla["input_copies_rotated"], "plan": mla["plan"],
            # both for the latent MFMA kernel alone: kernel_us from a loop that alternates the whole call and the kernel
            # alone, an event between every launch (interleaved_call_us is the whole call in that same loop)
            "roofline": {"bound": "hbm", "achieved": mla["algorithmic_bytes"] / (mla["kernel_us"] * 1e-6) / 1e9,
                         "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                         "frac": mla["algorithmic_bytes"] / (mla["kernel_us"] * 1e-6) / 1e9 / HBM_PEAK_GBPS,
                         "traffic": measured_traffic("mla", mla["plan"]), "kernel": "latent_pipe_kernel",
                         "kernel_us": mla["kernel_us"], "interleaved_call_us": mla["interleaved_call_us"]},
            "roofline_mfma": {"bound": "mfma", "achieved": mla["algorithmic_flops"] / (mla["kernel_us"] * 1e-6) / 1e12,
                              "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                              "frac": mla["algorithmic_flops"] / (mla["kernel_us"] * 1e-6) / 1e12 / MFMA_PEAK_TFLOPS,
                              # measured in this run: nothing but matrix instructions on every SIMD, with N(0,1)
                              # operands (what the power limit leaves) and with zeros (near the nominal clock)
                              "sustained_TFLOPs_random_operands": mfma_rand,
                              "sustained_TFLOPs_zero_operands": mfma_zero,
                              "frac_of_sustained": mla["algorithmic_flops"] / (mla["kernel_us"] * 1e-6) / 1e12 / mfma_rand},
        }
    print(json.dumps(line))
    return 0


# The reference's sweep lists (benchmarks/python/benchmark_decoding_attn.py:303-330): sequence lengths at batch 1,
# then batches at one length, for the head shape given on its command line (run_python.sh:25-31: MHA 32/32 x 128,
# MLA 128/1 x 576/512).
REF_SWEEPS = {
    "mha": {"heads": (32, 32, 128, 128),
            "seq_ks": [1, 8, 16, 32, 64, 128, 256, 512, 1024, 2048, 3072, 4096, 5120, 6144, 7168, 8192],
            "batch_seq_k": 128},
    "mla": {"heads": (128, 1, 576, 512),
            "seq_ks": [256, 512, 1024, 2048, 3072, 4096, 5120, 6144, 7168, 8192],
            "batch_seq_k": 4096},
}
REF_BATCHES = [1, 2, 4, 8, 16, 32, 64, 128, 256, 512, 768, 1024, 1536, 2048]
SEQ_MARKER = "------------------------------- Benchmark Seq -------------------------------"
BATCH_MARKER = "------------------------------- Benchmark Batch -------------------------------"


def reference_log_line(batch, seq_k, ms, tflops, gbps):
    """One result in the reference's log format (benchmarks/python/benchmark_decoding_attn.py:248-249): its plot
    script (tools/performance/python/performance.py:82-104) splits the line at spaces and reads token 0 as the
    method, token 1 as batch-seq_k, token 7 as TFLOPS and token 10 as GB/s."""
    return (f"Decoding-Attention {batch}-{seq_k} profiling time: {ms:.4f} ms, throughput: {tflops:.4f} TFLOPS, "
            f"bandwidth: {gbps:.3f} GB/s")


def sweep_sections(kind):
    """The shapes `--sweep kind` measures, as (section marker or None, tag, workload arguments) in print order.
    `mha` and `mla` are the reference's two sections with its full lists; `baseline` holds the benchmark shapes
    those lists leave out (the ragged and fixed GQA batches, MQA with ALiBi, sequence length 1536, the latent
    form's length sweep at batch 16, and the latent shape with V passed as its own buffer)."""
    out = []
    for fam in ("mha", "mla"):
        if kind in (fam, "all"):
            r = REF_SWEEPS[fam]
            out += [(SEQ_MARKER if i == 0 else None, f"{fam}-seq", (fam, 1, sk)) for i, sk in enumerate(r["seq_ks"])]
            out += [(BATCH_MARKER if i == 0 else None, f"{fam}-batch", (fam, b, r["batch_seq_k"]))
                    for i, b in enumerate(REF_BATCHES)]
    if kind in ("baseline", "gqa", "all"):
        title = "------------------------------- Other shapes -------------------------------"
        out += [(title, "gqa-varlen", ("gqa-varlen",)), (None, "gqa-fixed", ("gqa-fixed",)),
                (None, "mqa-alibi", ("mqa-alibi",)), (None, "mha-seq", ("mha", 1, 1536))]
        out += [(None, "mla-seq-b16", ("mla", 16, sk)) for sk in (512, 1024, 2048, 4096, 8192, 16384)]
        # (576, 512) with V in a buffer of its own, as the reference's binding accepts it: K and V are both read
        out += [(None, "mla-distinct-v", ("mla-distinct-v", b, 4096)) for b in (16, 64)]
    return out


def _sweep_workload(torch, wl, spec, device):
    if spec[0] == "mha":
        hq, hk, d, dv = REF_SWEEPS["mha"]["heads"]
        return wl.make_workload(spec[1], hq, hk, d, dv, spec[2], torch.float16, device=device)
    if spec[0] == "mla":
        hq, hk, d, dv = REF_SWEEPS["mla"]["heads"]
        return wl.make_workload(spec[1], hq, hk, d, dv, spec[2], torch.float16, device=device)
    if spec[0] == "mla-distinct-v":
        hq, hk, d, dv = REF_SWEEPS["mla"]["heads"]
        return wl.make_workload(spec[1], hq, hk, d, dv, spec[2], torch.float16, device=device, latent=False)
    return {"gqa-varlen": wl.config_gqa_varlen, "gqa-fixed": wl.config_gqa_fixed, "mqa-alibi": wl.config_mqa_alibi}[spec[0]]()


def run_sweep(args, measure_fn=None, workload_fn=None, out=None):
    """The reference's sweeps, printed in its log format: per head shape a header line, the `Benchmark Seq` marker
    and one line per sequence length, the `Benchmark Batch` marker and one line per batch (the reference's plot script
    cuts the log at the second marker; give it the log of one family, `--sweep mha` or `--sweep mla`).  Lines that
    start with four spaces carry this build's own figures and are skipped by that script (no `TFLOPS` in them)."""
    import torch

    from decoding_attention_amd import workloads as wl

    out = out or sys.stdout
    measure_fn = measure_fn or measure  # (tests of the log format pass their own, and shapes without data)
    workload_fn = workload_fn or (lambda spec: _sweep_workload(torch, wl, spec, "cuda:0"))
    shapes = [(m, tag, spec, {}) for m, tag, spec in sweep_sections(args.sweep)]
    if args.sweep == "paged":  # the benchmark shapes over shuffled pages of 64, 16 and 1 tokens, beside the packed layout
        for w in (wl.config_gqa_fixed(), wl.config_gqa_varlen(), wl.config_mqa_alibi(), wl.config_mla(64, 4096)):
            shapes += [(None, "packed", w, {})] + [(None, f"paged-{n}", w, {"page_size": n}) for n in (64, 16, 1)]
    if args.sweep == "fp8":  # 16-bit against FP8, int8 and int4 K/V on the bandwidth-bound shapes and the latent form
        for w in (wl.config_gqa_fixed(), wl.config_mha_sweep(512, 128), wl.config_mha_sweep(1, 8192),
                  wl.config_mqa_alibi(), wl.config_mla(64, 4096), wl.config_mla(16, 4096)):
            shapes += [(None, "kv16", w, {}), (None, "kv-fp8", w, {"kv_fp8": True}), (None, "kv-int8", w, {"kv_int8": True})]
            if w.dim != 576:  # (the latent kernel has no int4 form)
                shapes += [(None, "kv-int4", w, {"kv_int4": True})]
                shapes += [(None, "kv-int4-tok", w, {"kv_int4_tok": True})]
                shapes += [(None, "kv-int8-tok", w, {"kv_int8_tok": True})]
                shapes += [(None, "kv-int4-g64", w, {"kv_int4_g64": True})]
                shapes += [(None, "kv-int8-g64", w, {"kv_int8_g64": True})]
    results = []
    for marker, tag, spec, kw in shapes:
        if marker == SEQ_MARKER:
            hq, hk, d, dv = REF_SWEEPS[spec[0]]["heads"]
            print(f"Benchmark Decoding Attention: head q: {hq}, head k: {hk}, dim: {d}, dim v: {dv}, is alibi: False, "
                  f"is bf16: False, warmup iterations: {args.warmup}, profiling iterations: {args.steps}", file=out)
        if marker:
            print(marker, file=out, flush=True)
        w = workload_fn(spec) if isinstance(spec, tuple) else spec
        r = measure_fn(torch, w, args.steps, args.warmup, **kw)
        ms = r["us_per_call"] / 1e3
        sk = w.max_seq_k
        ref_bytes = wl.reference_formula_bytes(w.batch, w.head_q, w.head_k, w.dim, w.dim_v, sk)
        print(reference_log_line(w.batch, sk, ms, r["tflops"], ref_bytes / (ms * 1e-3) / 1e9), file=out, flush=True)
        print(f"    [{tag}] {w.name}: {r['us_per_call']:.1f} us/call (min {r['us_isolated_call_min']:.1f}), "
              f"{r['hbm_GBps'] / 1e3:.3f} TB/s of real traffic = {100 * r['hbm_frac_of_peak']:.1f}% of "
              f"{HBM_PEAK_GBPS / 1e3:.0f} TB/s, plan {r['plan']}", file=out, flush=True)
        r["tag"] = tag
        results.append(r)
        del w
    if args.json_out:
        with open(args.json_out, "w") as f:
            json.dump(results, f, indent=1)
    return 0


# Shapes of the latent form whose launch plan `--sweep latent-plan` derives: the benchmark's two sweeps (batch at 4096
# tokens, length at batch 16) and the reference's lists around them.
LATENT_PLAN_SHAPES = ([(b, 4096) for b in (1, 2, 4, 8, 16, 32, 64, 128, 256)] +
                      [(16, sk) for sk in (512, 1024, 2048, 8192, 16384)] + [(1, sk) for sk in (512, 2048, 8192)] +
                      [(4, 16384), (8, 8192), (32, 1024), (64, 1024), (100, 4096)] +
                      # short sequences of small batches, where a work-group's fixed cost decides the split count
                      [(8, 512), (8, 1024), (24, 1024), (16, 768), (16, 1536), (4, 2048), (8, 2048), (24, 2048), (8, 3072)] +
                      # batches of 20 to 128 sequences between one and two work-groups a CU
                      [(20, 4096), (40, 2048), (48, 1024), (48, 2048), (48, 4096), (64, 512), (64, 2048), (96, 1024),
                       (128, 512), (128, 1024)] +
                      # the smallest problems, where the grouped kernel's latent form competes
                      [(1, 128), (1, 256), (1, 1024), (2, 256), (2, 512), (2, 1024), (4, 256), (4, 512), (4, 1024)])


def run_latent_plan_sweep(args):
    """Every shape of LATENT_PLAN_SHAPES (128 heads over one latent head, fp16) timed under the library's own plan
    and under forced alternatives: the grouped kernel's latent form, and the latent kernel with 64 or 128 heads per
    work-group at each split count.  The planner's thresholds for the latent path are read off this log.  Runs on the
    probe library (the same code with a setter for the planner's tunables)."""
    import ctypes

    import torch

    from decoding_attention_amd import _lib
    from decoding_attention_amd import workloads as wl

    probe = _lib.load_probe()
    dev = torch.device("cuda:0")
    stream = torch.cuda.current_stream().cuda_stream
    defaults = {"DA_NSPLIT": 0, "DA_MLA_HEADS": 0, "DA_MLA_GROUP_SMALL": 65536}

    def set_tunables(**kw):
        for name, value in {**defaults, **kw}.items():
            assert probe.da_probe_set_tunable(name.encode(), int(value)) == 0

    kv_bits = 8 if args.kv == "fp8" else 16

    def plan_of(w):
        kind, ns, ch, rt = (ctypes.c_int() for _ in range(4))
        assert probe.da_plan_call(w.max_seq_k, w.batch, 128, 1, 576, 512, int(w.k.shape[0]), 0, 0, kv_bits,
                                  ctypes.byref(kind), ctypes.byref(ns), ctypes.byref(ch), ctypes.byref(rt), None) == 0
        return kind.value, rt.value, ns.value, ch.value

    def time_us(copies, w):
        total = int(w.k.shape[0])
        if kv_bits == 8:
            n = probe.da_workspace_bytes_fp8kv(w.max_seq_k, w.batch, 128, 1, 576, 512, total, 0)
        else:
            n = probe.da_workspace_bytes(w.max_seq_k, w.batch, 128, 1, 576, 512, total)
        ws = torch.empty(max(n, 16), dtype=torch.uint8, device=dev)
        o = torch.empty(w.batch, 128, 512, dtype=torch.float16, device=dev)
        scale = torch.full((1,), 0.02, device=dev)
        k8 = [(c.k.float() / 0.02).to(torch.float8_e4m3fn) for c in copies] if kv_bits == 8 else None

        def call(i):
            c = copies[i]
            if kv_bits == 8:
                rc = probe.da_decoding_attn_fp8kv(c.q.data_ptr(), k8[i].data_ptr(), None, o.data_ptr(),
                                                  c.cu_seq_k.data_ptr(), w.max_seq_k, w.batch, 128, 1, 576, 512, 0, 0,
                                                  0.0, None, scale.data_ptr(), scale.data_ptr(), total, ws.data_ptr(),
                                                  n, stream)
            else:
                rc = probe.da_decoding_attn_ex(c.q.data_ptr(), c.k.data_ptr(), None, o.data_ptr(),
                                               c.cu_seq_k.data_ptr(), w.max_seq_k, w.batch, 128, 1, 576, 512, 0, 0,
                                               0.0, None, total, ws.data_ptr(), n, stream)
            assert rc == 0, probe.da_last_error().decode("utf-8", "replace")

        mean_ms, _ = _time_calls(torch, [lambda i=i: call(i) for i in range(len(copies))], args.steps, args.warmup)
        return mean_ms * 1e3

    print("shape: candidates as kernel/heads-per-work-group/splits = us per call; kernel g = grouped (16 heads per "
          "group), l = latent", flush=True)
    for batch, sk in LATENT_PLAN_SHAPES:
        w = wl.make_workload(batch, 128, 1, 576, 512, sk, torch.float16, device="cuda:0")
        copies = _device_copies(torch, w, dev)
        set_tunables()
        kind, rt, ns, ch = plan_of(w)
        chosen = f"{'g' if kind == 3 else 'l'}/{rt}/{ns}"
        results = {}
        # the grouped kernel's latent form, its own split count
        set_tunables(DA_MLA_GROUP_SMALL=1 << 30)
        k2, rt2, ns2, _ = plan_of(w)
        if k2 == 3:
            results[f"g/{rt2}/{ns2}"] = time_us(copies, w)
        for heads in (64, 128):
            for nsplit in (1, 2, 3, 4, 5, 6, 8, 10, 12, 16, 24, 32):
                if sk // nsplit < 128 or batch * nsplit * (128 // heads) > 1024:
                    continue
                set_tunables(DA_MLA_GROUP_SMALL=0, DA_MLA_HEADS=heads, DA_NSPLIT=nsplit)
                k3, rt3, ns3, _ = plan_of(w)
                key = f"l/{rt3}/{ns3}"
                if k3 == 2 and key not in results:
                    results[key] = time_us(copies, w)
        set_tunables()
        if chosen not in results:
            results[chosen] = time_us(copies, w)
        best = min(results, key=results.get)
        ranked = ", ".join(f"{k} = {v:.1f}" for k, v in sorted(results.items(), key=lambda kv: kv[1])[:6])
        print(f"b{batch} x {sk}: planner {chosen} = {results[chosen]:.1f} us; best {best} = {results[best]:.1f} us "
              f"(planner / best = {results[chosen] / results[best]:.3f}); fastest six: {ranked}", flush=True)
        del w, copies
    return 0


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--kv", choices=["16", "fp8"], default="16", help="--sweep latent-plan: the K cache's format")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU oracle timing")
    ap.add_argument("--no-mla", action="store_true", help="skip the MLA measurement")
    ap.add_argument("--only", choices=["gqa", "mla"], help="measure one workload only and print its record "
                    "(for profiler runs)")
    ap.add_argument("--calibrate-copy", action="store_true", help="first run three 1 GiB device copies (a known "
                    "traffic figure for scaling profiler byte counters)")
    ap.add_argument("--cpu-budget", type=float, default=15.0, help="seconds of single-thread CPU work to sample")
    ap.add_argument("--sweep", choices=["mha", "mla", "baseline", "gqa", "all", "paged", "fp8", "latent-plan"], help="print the reference's sweeps instead "
                    "(paged / fp8: benchmark shapes over a paged or an 8-bit, FP8 and int8, K/V cache)")
    ap.add_argument("--json-out", help="with --sweep: also write the results as JSON")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: the op has no multi-GPU path (sequences and KV heads shard without "
              "communication); run with --gpus 1", file=sys.stderr)
        return 2
    if args.sweep == "latent-plan":
        return run_latent_plan_sweep(args)
    if args.sweep:
        return run_sweep(args)
    return run_default(args)


if __name__ == "__main__":
    sys.exit(main())
