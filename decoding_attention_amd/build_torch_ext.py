"""Build the PyTorch-ROCm extension module `decoding_attn_hip` (host C++ over the C-ABI library).

Usage: python -m decoding_attention_amd.build_torch_ext
"""
import os
import subprocess
import sysconfig

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(PKG_DIR, "csrc", "torch_binding.cpp")
EXT_NAME = "decoding_attn_hip"
EXT_PATH = os.path.join(PKG_DIR, EXT_NAME + (sysconfig.get_config_var("EXT_SUFFIX") or ".so"))


def build(force=True):
    """Compile the binding with the host compiler and link it against the in-tree libdecoding_attn_hip.so."""
    if not force and os.path.exists(EXT_PATH):
        return EXT_PATH
    import torch
    from torch.utils import cpp_extension as ce

    from . import build as da_build

    if not os.path.exists(da_build.LIB_PATH):
        da_build.build(force=True)
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    includes = ce.include_paths() + [sysconfig.get_paths()["include"], os.path.join(rocm, "include")]
    try:
        import pybind11
        includes.append(pybind11.get_include())
    except ImportError:
        pass
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = [os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_API_INCLUDE_EXTENSION_H",
           f"-DTORCH_EXTENSION_NAME={EXT_NAME}", f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}"]
    cmd += [f"-I{p}" for p in includes]
    cmd += [SRC, "-o", EXT_PATH, f"-L{PKG_DIR}", "-ldecoding_attn_hip", f"-L{torch_lib}", "-lc10", "-lc10_hip",
            "-ltorch_cpu", "-ltorch_hip", "-ltorch", "-ltorch_python", f"-L{rocm}/lib", "-lamdhip64",
            "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{torch_lib}", f"-Wl,-rpath,{rocm}/lib"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("building the torch extension failed:\n" + res.stdout + "\n" + res.stderr)
    return EXT_PATH


if __name__ == "__main__":
    print(build(force=True))
