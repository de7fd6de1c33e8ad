"""The log `bench.py --sweep` prints is the reference's: its plot script must be able to read it.  The reader below
restates what that script does with a log (reference tools/performance/python/performance.py:22-38: lines with
`TFLOPS` before the line holding `Benchmark Batch` are the sequence sweep, those after it the batch sweep; :82-104:
a line is split at single spaces, token 0 the method, token 1 `batch-seq_k`, token 7 TFLOPS, token 10 GB/s)."""
import io
import os
import sys
import types

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
import bench  # noqa: E402


def read_log_like_the_plot_script(text):
    seq, batch, in_batch = [], [], False
    for line in text.splitlines():
        in_batch = in_batch or "Benchmark Batch" in line
        if "TFLOPS" in line:
            (batch if in_batch else seq).append(line)

    def table(lines, which):
        rows = {}
        for line in lines:
            items = line.split(" ")
            assert items[0] == "Decoding-Attention"
            rows[int(items[1].split("-")[which])] = (float(items[7]), float(items[10]))
        return rows

    return table(seq, 1), table(batch, 0)


def _fake_run(kind):
    def workload(spec):
        fam, batch, seq_k = spec
        hq, hk, d, dv = bench.REF_SWEEPS[fam]["heads"]
        return types.SimpleNamespace(batch=batch, head_q=hq, head_k=hk, dim=d, dim_v=dv, max_seq_k=seq_k,
                                     name=f"{fam}-{batch}-{seq_k}")

    def measure(torch, w, steps, warmup):
        # 1 us per 1000 batch x tokens: throughput and bandwidth then follow from the formulas
        us = w.batch * w.max_seq_k / 1000.0 + 1.0
        flops = 4 * w.batch * w.head_q * w.max_seq_k * (w.dim + w.dim_v) // 2
        return {"us_per_call": us, "us_isolated_call_min": us, "tflops": flops / (us * 1e-6) / 1e12, "hbm_GBps": 1.0,
                "hbm_frac_of_peak": 0.0, "plan": {}}

    out = io.StringIO()
    args = types.SimpleNamespace(sweep=kind, steps=10, warmup=1, json_out=None)
    assert bench.run_sweep(args, measure_fn=measure, workload_fn=workload, out=out) == 0
    return out.getvalue()


def test_mha_sweep_log_has_the_reference_sections_and_lists():
    text = _fake_run("mha")
    lines = text.splitlines()
    assert lines[0].startswith("Benchmark Decoding Attention: head q: 32, head k: 32, dim: 128, dim v: 128,")
    assert lines[1] == bench.SEQ_MARKER and lines.count(bench.SEQ_MARKER) == lines.count(bench.BATCH_MARKER) == 1
    seq, batch = read_log_like_the_plot_script(text)
    # reference benchmarks/python/benchmark_decoding_attn.py:307-309 and :320-324
    assert sorted(seq) == [1, 8, 16, 32, 64, 128, 256, 512, 1024, 2048, 3072, 4096, 5120, 6144, 7168, 8192]
    assert sorted(batch) == [1, 2, 4, 8, 16, 32, 64, 128, 256, 512, 768, 1024, 1536, 2048]
    # the numbers survive the round trip: batch 2048 x 128 tokens took 263.144 us in the fake measurement
    from decoding_attention_amd import workloads as wl
    us = 2048 * 128 / 1000.0 + 1.0
    tflops, gbps = batch[2048]
    assert abs(tflops - wl.algorithmic_flops(32, 128, 128, 2048 * 128) / (us * 1e-6) / 1e12) < 1e-3
    assert abs(gbps - wl.reference_formula_bytes(2048, 32, 32, 128, 128, 128) / (us * 1e-6) / 1e9) < 1e-2


def test_mla_sweep_log_has_the_reference_sections_and_lists():
    seq, batch = read_log_like_the_plot_script(_fake_run("mla"))
    assert sorted(seq) == [256, 512, 1024, 2048, 3072, 4096, 5120, 6144, 7168, 8192]  # (:310-311)
    assert sorted(batch) == [1, 2, 4, 8, 16, 32, 64, 128, 256, 512, 768, 1024, 1536, 2048]


def test_own_figures_stay_out_of_the_plot_scripts_way():
    for line in _fake_run("mha").splitlines():
        if line.startswith("    ["):
            assert "TFLOPS" not in line and "Benchmark" not in line


def test_log_line_tokens():
    items = bench.reference_log_line(16, 4096, 0.1234, 56.789, 4321.5).split(" ")
    assert (items[0], items[1], items[4], items[7], items[10]) == ("Decoding-Attention", "16-4096", "0.1234", "56.7890",
                                                                 "4321.500")
