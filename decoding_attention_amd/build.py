"""Build libdecoding_attn_hip.so for gfx950 with hipcc (cross-compiles without a GPU).

Usage: python -m decoding_attention_amd.build [--force]
"""
import concurrent.futures
import os
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_PATH = os.path.join(PKG_DIR, "libdecoding_attn_hip.so")
OBJ_DIR = os.path.join(PKG_DIR, "build")

SOURCES = [
    "da_api.hip",
    "da_sweep_d64.hip",
    "da_sweep_d96.hip",
    "da_sweep_d128.hip",
    "da_sweep_d256.hip",
    "da_sweep_d576.hip",
    "da_mla.hip",
    "da_mla_pipe.hip",
    "da_gqa_mfma.hip",
    "da_sweep_kv8.hip",
    "da_gqa_mfma_kv8.hip",
    "da_gqa_mfma_i8.hip",
    "da_gqa_mfma_i4.hip",
    "da_gqa_mfma_i4t.hip",
    "da_gqa_mfma_i4g.hip",
    "da_gqa_mfma_i8g.hip",
    "da_gqa_mfma_i8t.hip",
]

# libdecoding_attn_probe.so (measurement aids of bench.py, csrc/decoding_attn_probe.h): the same objects, with
# da_api.hip compiled once more with the sweep-only entry point, plus the streaming-read kernel.
PROBE_LIB_PATH = os.path.join(PKG_DIR, "libdecoding_attn_probe.so")

# packed-fp32 VALU forms are switched off on purpose: only scalar fp32 arithmetic is emitted.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wextra",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _hipcc():
    return os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")


# Per-file flags.  da_mla_pipe.hip names most of the register file in its instruction text and confines the compiler
# to the rest; the compiler must then never park its own values in accumulation registers.
EXTRA_FLAGS = {
    "da_mla_pipe.hip": ["-mllvm", "-amdgpu-spill-vgpr-to-agpr=0"],
}


# Sources whose generated code is verified after compiling (check_isa.py).
ISA_CHECKED = {"da_mla_pipe.hip"}


def _compile(src, obj_name=None, defines=()):
    obj = os.path.join(OBJ_DIR, (obj_name or os.path.splitext(src)[0]) + ".o")
    cmd = ([_hipcc()] + HIPCC_FLAGS + EXTRA_FLAGS.get(src, []) + [f"-D{d}" for d in defines] +
           ["-c", os.path.join(CSRC, src), "-o", obj])
    if os.environ.get("DA_SAVE_TEMPS"):
        cmd += ["-save-temps=obj"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{res.stdout}\n{res.stderr}")
    if src in ISA_CHECKED:
        from . import check_isa
        check_isa.check_source(_hipcc(), HIPCC_FLAGS + EXTRA_FLAGS.get(src, []), os.path.join(CSRC, src))
    warn = "\n".join(ln for ln in res.stderr.splitlines() if "packed-fp32-ops" not in ln and ln.strip())
    return obj, warn


def build(force=True, verbose=False):
    """Compile every translation unit and link the shared library.  Always compiles when force is set."""
    if not force and os.path.exists(LIB_PATH):
        return LIB_PATH
    os.makedirs(OBJ_DIR, exist_ok=True)
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        results = list(ex.map(_compile, SOURCES))
    objs = [r[0] for r in results]
    if verbose:
        for _, w in results:
            if w:
                print(w, file=sys.stderr)
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH] + objs
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stdout}\n{res.stderr}")
    # the probe library: every object but da_api.o, da_api.hip with the probe entry point, the streaming-read kernel
    api_probe, _ = _compile("da_api.hip", obj_name="da_api_probe", defines=("DA_BUILD_PROBES",))
    stream_probe, _ = _compile("da_probe.hip")
    api_obj = os.path.join(OBJ_DIR, "da_api.o")
    cmd = ([_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", PROBE_LIB_PATH] +
           [o for o in objs if o != api_obj] + [api_probe, stream_probe])
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link of the probe library failed:\n{res.stdout}\n{res.stderr}")
    return LIB_PATH


CLI_SRC = os.path.join(PKG_DIR, "bench_cli", "benchmark_decoding_attn.cpp")
CLI_PATH = os.path.join(PKG_DIR, "bench_cli", "benchmark_decoding_attn")


def build_cli(force=True):
    """Compile the benchmark executable (host code only) against the in-tree library."""
    if not force and os.path.exists(CLI_PATH):
        return CLI_PATH
    if not os.path.exists(LIB_PATH):
        build(force=True)
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    include = os.path.join(os.path.dirname(PKG_DIR), "include")
    cmd = [os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-Wall", "-Wextra", "-fopenmp", "-D__HIP_PLATFORM_AMD__=1",
           f"-I{include}", f"-I{rocm}/include", CLI_SRC, "-o", CLI_PATH, f"-L{PKG_DIR}", "-ldecoding_attn_hip",
           f"-L{rocm}/lib", "-lamdhip64", "-Wl,-rpath,$ORIGIN/..", f"-Wl,-rpath,{rocm}/lib"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"building the benchmark executable failed:\n{res.stdout}\n{res.stderr}")
    return CLI_PATH


if __name__ == "__main__":
    path = build(force=True, verbose=True)
    print(path)
    print(build_cli(force=True))
