"""HBM bytes per call of the two benchmark workloads from rocprofv3 counter runs, written as the JSON that bench.py
reads for its `roofline.traffic` figures.

The counter runs (on the GPU box, one counter per run, each with three 1 GiB device copies in front as a known figure):

    rocprofv3 --pmc FETCH_SIZE --output-format csv -d <dir>/pmc_<w>_FETCH_SIZE -o x -- python3 bench.py --steps 5 --warmup 2 --only <w> --calibrate-copy
    rocprofv3 --pmc WRITE_SIZE --output-format csv -d <dir>/pmc_<w>_WRITE_SIZE -o x -- python3 bench.py --steps 5 --warmup 2 --only <w> --calibrate-copy

for <w> in gqa, mla.  Then, anywhere:  python -m decoding_attention_amd.profile_traffic <dir> profiles/hbm_traffic.json

A counter's reading is scaled by what the same counter read for the 1 GiB copy (1 048 576 KiB moved each way).  The
figures belong to the launch plan they were measured under, which is stored beside them; bench.py reports no traffic
when the library plans the workload differently.
"""
import collections
import csv
import json
import os
import sys

COPY_KIB = 1048576.0
WORKLOADS = {
    # name: (max_seq_k, batch, head_q, head_k, dim, dim_v)
    "gqa": (4096, 64, 32, 8, 128, 128),
    "mla": (4096, 64, 128, 1, 576, 512),
}


def _readings(path):
    """{kernel name: counter values, one per dispatch} of one counter_collection.csv."""
    acc = collections.defaultdict(list)
    with open(path, newline="") as f:
        for row in csv.DictReader(f):
            acc[row["Kernel_Name"]].append(float(row["Counter_Value"]))
    return acc


def summarise(run_dir):
    from . import _lib

    out = {}
    for name, shape in WORKLOADS.items():
        kernels = {}
        total_kib = 0.0
        for counter in ("FETCH_SIZE", "WRITE_SIZE"):
            path = os.path.join(run_dir, f"pmc_{name}_{counter}", "x_counter_collection.csv")
            readings = _readings(path)
            # (the 1 GiB copies are the largest device copies of the run; the inputs' own copies are smaller)
            copy = [max(v) for k, v in readings.items() if "copyBuffer" in k]
            if not copy or max(copy) < 0.4 * COPY_KIB:
                raise RuntimeError(f"{path}: no 1 GiB device copy to scale the counter by (run with --calibrate-copy)")
            factor = COPY_KIB / max(copy)
            for k, vals in readings.items():
                if "da::" not in k:
                    continue
                v = sum(vals) / len(vals)
                short = k[:k.rfind("(")].replace("void ", "")  # (without the argument list)
                kernels.setdefault(short, {})[counter] = {"reading": v, "factor": factor, "KiB": v * factor}
                total_kib += v * factor
        max_seq_k, batch, hq, hk, d, dv = shape
        plan = _lib.plan(max_seq_k, batch, hq, hk, d, dv, total_k=batch * max_seq_k)
        out[name] = {"bytes": int(round(total_kib * 1024)), "plan": plan, "kernels": kernels}
    return out


if __name__ == "__main__":
    if len(sys.argv) != 3:
        sys.exit(__doc__)
    result = summarise(sys.argv[1])
    with open(sys.argv[2], "w") as f:
        json.dump(result, f, indent=1)
    for name, rec in result.items():
        print(name, rec["bytes"], "bytes per call under plan", rec["plan"])
