"""ctypes binding of libdecoding_attn_hip.so (the C-ABI declared in include/decoding_attn_hip.h).

The library is loaded from this package directory.  There is no fallback of any kind: if the
shared object is missing the import of the op fails loudly with the build command to run.
"""
import ctypes
import os

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(PKG_DIR, "libdecoding_attn_hip.so")

# Every symbol include/decoding_attn_hip.h declares.
EXPORTED_SYMBOLS = (
    "da_decoding_attn",
    "da_decoding_attn_ex",
    "da_workspace_bytes",
    "da_release_workspaces",
    "da_decoding_attn_noalloc",
    "da_noalloc_workspace_limit",
    "da_decoding_attn_paged",
    "da_workspace_bytes_paged",
    "da_decoding_attn_fp8kv",
    "da_decoding_attn_paged_fp8kv",
    "da_workspace_bytes_fp8kv",
    "da_decoding_attn_int8kv",
    "da_decoding_attn_paged_int8kv",
    "da_workspace_bytes_int8kv",
    "da_decoding_attn_int4kv",
    "da_decoding_attn_paged_int4kv",
    "da_workspace_bytes_int4kv",
    "da_plan",
    "da_plan_distinct_v",
    "da_plan_is_balanced",
    "da_plan_call",
    "da_decoding_attn_int4kv_tok",
    "da_decoding_attn_paged_int4kv_tok",
    "da_workspace_bytes_int4kv_tok",
    "da_decoding_attn_int4kv_grp64",
    "da_decoding_attn_paged_int4kv_grp64",
    "da_workspace_bytes_int4kv_grp64",
    "da_decoding_attn_int8kv_grp64",
    "da_decoding_attn_paged_int8kv_grp64",
    "da_workspace_bytes_int8kv_grp64",
    "da_decoding_attn_int8kv_tok",
    "da_decoding_attn_paged_int8kv_tok",
    "da_workspace_bytes_int8kv_tok",
    "da_supported_head_dims",
    "da_last_error",
    "da_version",
)

DA_OK = 0
DA_ERR_INVALID_ARGUMENT = 1
DA_ERR_UNSUPPORTED = 2
DA_ERR_WORKSPACE = 3
DA_ERR_HIP = 4

_lib = None


class LibraryNotBuilt(ImportError):
    pass


def load():
    """Load the shared library once and declare the prototypes."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise LibraryNotBuilt(
            f"{LIB_PATH} is missing: build it with `python -m decoding_attention_amd.build` "
            "(hipcc, --offload-arch=gfx950). There is no CPU or PyTorch fallback.")
    lib = ctypes.CDLL(LIB_PATH)
    _declare(lib)
    _lib = lib
    return lib


def _declare(lib):
    """Prototypes of the drop-in ABI (include/decoding_attn_hip.h)."""
    vp, sz, ci, cf = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int, ctypes.c_float
    lib.da_decoding_attn.restype = ci
    lib.da_decoding_attn.argtypes = [vp, vp, vp, vp, vp, sz, sz, sz, sz, sz, sz, ci, ci, vp]
    lib.da_decoding_attn_ex.restype = ci
    lib.da_decoding_attn_ex.argtypes = [vp, vp, vp, vp, vp, sz, sz, sz, sz, sz, sz, ci, ci, cf, vp, sz, vp, sz, vp]
    lib.da_workspace_bytes.restype = sz
    lib.da_workspace_bytes.argtypes = [sz, sz, sz, sz, sz, sz, sz]
    lib.da_release_workspaces.restype = ci
    lib.da_release_workspaces.argtypes = []
    lib.da_decoding_attn_noalloc.restype = ci
    lib.da_decoding_attn_noalloc.argtypes = [vp, vp, vp, vp, vp, sz, sz, sz, sz, sz, sz, ci, ci, cf, vp, sz, vp]
    lib.da_noalloc_workspace_limit.restype = sz
    lib.da_noalloc_workspace_limit.argtypes = []
    lib.da_decoding_attn_paged.restype = ci
    lib.da_decoding_attn_paged.argtypes = [vp, vp, vp, vp, vp, vp, sz, sz, sz, sz, sz, sz, sz, sz, sz, sz, ci, ci, cf,
                                           vp, sz, vp, sz, vp]
    lib.da_workspace_bytes_paged.restype = sz
    lib.da_workspace_bytes_paged.argtypes = [sz, sz, sz, sz, sz, sz, sz, sz]
    lib.da_decoding_attn_fp8kv.restype = ci
    lib.da_decoding_attn_fp8kv.argtypes = [vp, vp, vp, vp, vp, sz, sz, sz, sz, sz, sz, ci, ci, cf, vp, vp, vp, sz, vp, sz,
                                           vp]
    lib.da_decoding_attn_paged_fp8kv.restype = ci
    lib.da_decoding_attn_paged_fp8kv.argtypes = [vp, vp, vp, vp, vp, vp, sz, sz, sz, sz, sz, sz, sz, sz, sz, sz, ci, ci,
                                                 cf, vp, vp, vp, sz, vp, sz, vp]
    lib.da_workspace_bytes_fp8kv.restype = sz
    lib.da_workspace_bytes_fp8kv.argtypes = [sz, sz, sz, sz, sz, sz, sz, sz]
    # the int8 entry points take the FP8 ones' arguments
    lib.da_decoding_attn_int8kv.restype = ci
    lib.da_decoding_attn_int8kv.argtypes = lib.da_decoding_attn_fp8kv.argtypes
    lib.da_decoding_attn_paged_int8kv.restype = ci
    lib.da_decoding_attn_paged_int8kv.argtypes = lib.da_decoding_attn_paged_fp8kv.argtypes
    lib.da_workspace_bytes_int8kv.restype = sz
    lib.da_workspace_bytes_int8kv.argtypes = lib.da_workspace_bytes_fp8kv.argtypes
    lib.da_decoding_attn_int4kv.restype = ci
    lib.da_decoding_attn_int4kv.argtypes = lib.da_decoding_attn_fp8kv.argtypes
    lib.da_decoding_attn_paged_int4kv.restype = ci
    lib.da_decoding_attn_paged_int4kv.argtypes = lib.da_decoding_attn_paged_fp8kv.argtypes
    lib.da_workspace_bytes_int4kv.restype = sz
    lib.da_workspace_bytes_int4kv.argtypes = lib.da_workspace_bytes_fp8kv.argtypes
    # ... and so do the int4 entry points with per-token (scale, zero) pairs (k_params, v_params in the scales' places)
    lib.da_decoding_attn_int4kv_tok.restype = ci
    lib.da_decoding_attn_int4kv_tok.argtypes = lib.da_decoding_attn_fp8kv.argtypes
    lib.da_decoding_attn_paged_int4kv_tok.restype = ci
    lib.da_decoding_attn_paged_int4kv_tok.argtypes = lib.da_decoding_attn_paged_fp8kv.argtypes
    lib.da_decoding_attn_int4kv_grp64.restype = ci
    lib.da_decoding_attn_int4kv_grp64.argtypes = lib.da_decoding_attn_fp8kv.argtypes
    lib.da_decoding_attn_paged_int4kv_grp64.restype = ci
    lib.da_decoding_attn_paged_int4kv_grp64.argtypes = lib.da_decoding_attn_paged_fp8kv.argtypes
    lib.da_decoding_attn_int8kv_grp64.restype = ci
    lib.da_decoding_attn_int8kv_grp64.argtypes = lib.da_decoding_attn_fp8kv.argtypes
    lib.da_decoding_attn_paged_int8kv_grp64.restype = ci
    lib.da_decoding_attn_paged_int8kv_grp64.argtypes = lib.da_decoding_attn_paged_fp8kv.argtypes
    lib.da_workspace_bytes_int8kv_grp64.restype = sz
    lib.da_workspace_bytes_int8kv_grp64.argtypes = lib.da_workspace_bytes_fp8kv.argtypes
    lib.da_workspace_bytes_int4kv_grp64.restype = sz
    lib.da_workspace_bytes_int4kv_grp64.argtypes = lib.da_workspace_bytes_fp8kv.argtypes
    lib.da_workspace_bytes_int4kv_tok.restype = sz
    lib.da_workspace_bytes_int4kv_tok.argtypes = lib.da_workspace_bytes_fp8kv.argtypes
    lib.da_decoding_attn_int8kv_tok.restype = ci
    lib.da_decoding_attn_int8kv_tok.argtypes = lib.da_decoding_attn_fp8kv.argtypes
    lib.da_decoding_attn_paged_int8kv_tok.restype = ci
    lib.da_decoding_attn_paged_int8kv_tok.argtypes = lib.da_decoding_attn_paged_fp8kv.argtypes
    lib.da_workspace_bytes_int8kv_tok.restype = sz
    lib.da_workspace_bytes_int8kv_tok.argtypes = lib.da_workspace_bytes_fp8kv.argtypes
    ip = ctypes.POINTER(ci)
    lib.da_plan.restype = ci
    lib.da_plan.argtypes = [sz, sz, sz, sz, sz, sz, ci, sz, ip, ip, ip, ip]
    lib.da_plan_distinct_v.restype = ci
    lib.da_plan_distinct_v.argtypes = [sz, sz, sz, sz, sz, sz, sz, sz, ip, ip, ip, ip]
    lib.da_plan_is_balanced.restype = ci
    lib.da_plan_is_balanced.argtypes = [sz, sz, sz, sz, sz, sz, sz, sz]
    ip = ctypes.POINTER(ci)
    lib.da_plan_call.restype = ci
    lib.da_plan_call.argtypes = [sz, sz, sz, sz, sz, sz, sz, sz, ci, ci, ip, ip, ip, ip, ip]
    lib.da_supported_head_dims.restype = ci
    lib.da_supported_head_dims.argtypes = [sz, sz]
    lib.da_last_error.restype = ctypes.c_char_p
    lib.da_last_error.argtypes = []
    lib.da_version.restype = ci
    lib.da_version.argtypes = []


PROBE_LIB_PATH = os.path.join(PKG_DIR, "libdecoding_attn_probe.so")
_probe = None


def load_probe():
    """The benchmark's measurement aids (csrc/decoding_attn_probe.h): a second build of the library with the
    sweep-only entry point and the streaming-read kernel.  Not part of the drop-in ABI; only bench.py loads it."""
    global _probe
    if _probe is not None:
        return _probe
    if not os.path.exists(PROBE_LIB_PATH):
        raise LibraryNotBuilt(f"{PROBE_LIB_PATH} is missing: build it with `python -m decoding_attention_amd.build`")
    lib = ctypes.CDLL(PROBE_LIB_PATH)
    _declare(lib)  # (the probe library is the same code: it exports the drop-in entry points too)
    vp, sz, ci = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int
    lib.da_probe_set_tunable.restype = ci
    lib.da_probe_set_tunable.argtypes = [ctypes.c_char_p, ci]
    lib.da_probe_stream_read.restype = ci
    lib.da_probe_stream_read.argtypes = [vp, sz, vp, vp]
    lib.da_probe_sweep_only.restype = ci
    lib.da_probe_sweep_only.argtypes = [vp, vp, vp, vp, vp, sz, sz, sz, sz, sz, sz, ci, ci, sz, vp, sz, vp]
    lib.da_probe_stream_read_bytes.restype = sz
    lib.da_probe_stream_read_bytes.argtypes = [sz]
    lib.da_probe_mfma_rate.restype = ci
    lib.da_probe_mfma_rate.argtypes = [vp, ci, vp, vp]
    lib.da_probe_mfma_rate_flops.restype = ctypes.c_double
    lib.da_probe_mfma_rate_flops.argtypes = [ci]
    _probe = lib
    return lib


def last_error() -> str:
    return load().da_last_error().decode("utf-8", "replace")


KV_BITS_INT4_PER_TOKEN = 5  # DA_KV_BITS_INT4_PER_TOKEN of include/decoding_attn_hip.h
KV_BITS_INT8_PER_TOKEN = 9  # DA_KV_BITS_INT8_PER_TOKEN
KV_BITS_INT4_GROUP64 = 6  # DA_KV_BITS_INT4_GROUP64
KV_BITS_INT8_GROUP64 = 10  # DA_KV_BITS_INT8_GROUP64


def plan(max_seq_k, batch, head_q, head_k, dim, dim_v, is_bf16=False, total_k=0, distinct_v=False, page_size=0,
         kv_bits=16):
    """Launch plan of a call: dict(kind, nsplit, chunk, heads_per_group, balanced).  `distinct_v`: V passed as its own
    buffer; `page_size`: pages of that many tokens (0 = packed); `kv_bits`: 16, 8 (FP8, int8), 4 (int4) or
    KV_BITS_INT4_PER_TOKEN / KV_BITS_INT8_PER_TOKEN (int4 / int8 with per-token pairs) or KV_BITS_INT4_GROUP64 /
    KV_BITS_INT8_GROUP64 (a pair per 64 elements); distinct_v is implied for these."""
    if kv_bits in (KV_BITS_INT4_PER_TOKEN, KV_BITS_INT8_PER_TOKEN, KV_BITS_INT4_GROUP64, KV_BITS_INT8_GROUP64):
        distinct_v = True
    del is_bf16  # (the plan does not depend on it)
    lib = load()
    kind, ns, ch, rt, bal = (ctypes.c_int() for _ in range(5))
    rc = lib.da_plan_call(max_seq_k, batch, head_q, head_k, dim, dim_v, int(total_k), int(page_size), int(distinct_v),
                          int(kv_bits), ctypes.byref(kind), ctypes.byref(ns), ctypes.byref(ch), ctypes.byref(rt),
                          ctypes.byref(bal))
    if rc != DA_OK:
        raise RuntimeError(f"da_plan_call failed ({rc}): {last_error()}")
    return {"kind": kind.value, "nsplit": ns.value, "chunk": ch.value, "heads_per_group": rt.value,
            "balanced": bool(bal.value)}
