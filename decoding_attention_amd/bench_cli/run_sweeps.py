"""Run the benchmark executable over the reference's two sweeps and write one log per point.

The sweeps are those of the reference's run_cpp.sh:33-75 (key length at batch 1; batch at key length 128) for
MHA 32/32 d128 and MLA 128/1 576/512; logs go to <out>/<decoding_seq|decoding_batch>/da_<b>_<sq>_<sk>_<hq>_<hk>_<d>_<dv>.log,
the names the reference's tools/performance/cpp/performance.py takes its x axis from.

Usage: python -m decoding_attention_amd.bench_cli.run_sweeps [--out log] [--which mha|mla|all] [--bf16]
"""
import argparse
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
EXE = os.path.join(HERE, "benchmark_decoding_attn")

SEQ_K = [1, 8, 16, 32, 64, 128, 256, 512, 1024, 2048, 3072, 4096, 5120, 6144, 7168, 8192]
BATCH = [1, 2, 4, 8, 16, 32, 64, 128, 256, 512, 768, 1024, 1536, 2048]
HEADS = {"mha": (32, 32, 128, 128), "mla": (128, 1, 576, 512)}


def run_point(out_dir, kind, b, sk, hq, hk, d, dv, bf16):
    os.makedirs(os.path.join(out_dir, kind), exist_ok=True)
    log = os.path.join(out_dir, kind, f"da_{b}_1_{sk}_{hq}_{hk}_{d}_{dv}.log")
    cmd = [EXE, f"-b={b}", "-sq=1", f"-sk={sk}", f"-hq={hq}", f"-hk={hk}", f"-d={d}", f"-dv={dv}", "-is_causal=false",
           "-is_alibi=false", f"-is_bf16={'true' if bf16 else 'false'}", "-warmup_iterations=1",
           "-profiling_iterations=10", "-sleep_duration=100", "-enable_check=false"]
    with open(log, "w") as fp:
        rc = subprocess.run(cmd, stdout=fp, stderr=subprocess.STDOUT, timeout=300).returncode
    if rc != 0:
        raise RuntimeError(f"{' '.join(cmd)} exited with {rc}; see {log}")
    with open(log) as fp:
        for line in fp:
            if " exit, profiling time" in line:
                print(f"{kind} b={b} sk={sk}: " + line.split("] ", 1)[1].strip(), flush=True)


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--out", default="log")
    ap.add_argument("--which", default="all", choices=["mha", "mla", "all"])
    ap.add_argument("--bf16", action="store_true")
    args = ap.parse_args(argv)
    if not os.path.exists(EXE):
        sys.exit(f"{EXE} is not built: run python -m decoding_attention_amd.build")
    for name in (["mha", "mla"] if args.which == "all" else [args.which]):
        hq, hk, d, dv = HEADS[name]
        out = os.path.join(args.out, name)
        for sk in SEQ_K:
            run_point(out, "decoding_seq", 1, sk, hq, hk, d, dv, args.bf16)
        for b in BATCH:
            run_point(out, "decoding_batch", b, 128, hq, hk, d, dv, args.bf16)


if __name__ == "__main__":
    main()
