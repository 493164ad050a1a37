"""ctypes binding of libhyperattn.so (the C ABI declared in include/hyperattn.h) and its build.

The library is built in-tree with hipcc for gfx950 only.  There is no fallback: if the shared
object is missing or fails to load, every operator raises.
"""
from __future__ import annotations

import ctypes
import os
import shutil
import subprocess
from concurrent.futures import ThreadPoolExecutor

_PKG = os.path.dirname(os.path.abspath(__file__))
_CSRC = os.path.join(_PKG, "csrc")
_BUILD = os.path.join(_PKG, "build")
LIB_PATH = os.path.join(_PKG, "libhyperattn.so")

SOURCES = ["api.hip", "lsh_hash.hip", "bucket_sort.hip", "gather_rows.hip", "lse_merge.hip", "attn_fwd.hip",
           "attn_bwd.hip", "power_probe.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # packed-fp32 instructions are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]

# exported symbols, in the order of include/hyperattn.h
SYMBOLS = [
    "ha_abi_version", "ha_last_error", "ha_lsh_hash", "ha_bucket_argsort_workspace_bytes",
    "ha_bucket_argsort", "ha_bucket_argsort_static", "ha_gather_rows", "ha_block_attn_fwd", "ha_flash_attn_fwd",
    "ha_attn_bwd_workspace_bytes", "ha_block_attn_bwd", "ha_flash_attn_bwd", "ha_lse_merge",
    "ha_lse_merge_segments",
    "ha_forward_workspace_bytes", "ha_forward", "ha_forward_sort", "ha_lse_merge_levels", "ha_power_probe",
]

HA_F16, HA_BF16 = 0, 1
ABI_VERSION = 6
HA_IDX_I32, HA_IDX_I64 = 0, 1


def build(verbose: bool = False) -> str:
    """Compile every HIP source for gfx950 and link libhyperattn.so next to this file."""
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    os.makedirs(_BUILD, exist_ok=True)

    def compile_one(src: str) -> str:
        obj = os.path.join(_BUILD, src.replace(".hip", ".o"))
        cmd = [hipcc, *HIPCC_FLAGS, "-c", os.path.join(_CSRC, src), "-o", obj]
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{res.stdout}\n{res.stderr}")
        if verbose and res.stderr.strip():
            print(res.stderr)
        return obj

    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as pool:
        objs = list(pool.map(compile_one, SOURCES))
    tmp = LIB_PATH + ".tmp"
    res = subprocess.run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp, *objs],
                         capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stdout}\n{res.stderr}")
    os.replace(tmp, LIB_PATH)
    global _lib
    _lib = None
    return LIB_PATH


class AttnOperands(ctypes.Structure):
    _fields_ = [
        ("q", ctypes.c_void_p), ("k", ctypes.c_void_p), ("v", ctypes.c_void_p),
        ("out", ctypes.c_void_p), ("lse", ctypes.c_void_p),
        ("batch", ctypes.c_int64), ("heads", ctypes.c_int64), ("n_q", ctypes.c_int64),
        ("n_k", ctypes.c_int64), ("d", ctypes.c_int64), ("dv", ctypes.c_int64),
        ("q_stride_b", ctypes.c_int64), ("q_stride_h", ctypes.c_int64), ("q_stride_n", ctypes.c_int64),
        ("k_stride_b", ctypes.c_int64), ("k_stride_h", ctypes.c_int64), ("k_stride_n", ctypes.c_int64),
        ("v_stride_b", ctypes.c_int64), ("v_stride_h", ctypes.c_int64), ("v_stride_n", ctypes.c_int64),
        ("o_stride_b", ctypes.c_int64), ("o_stride_h", ctypes.c_int64), ("o_stride_n", ctypes.c_int64),
        ("lse_stride_b", ctypes.c_int64), ("lse_stride_h", ctypes.c_int64),
        ("segs", ctypes.c_int64), ("seg_stride_rows", ctypes.c_int64),
        ("q_seg_offset", ctypes.c_int64), ("k_seg_offset", ctypes.c_int64),
        ("o_seg_stride_rows", ctypes.c_int64), ("o_seg_offset", ctypes.c_int64),
        ("kv_group", ctypes.c_int64),
        ("scale", ctypes.c_float), ("dtype", ctypes.c_int),
    ]


class BlockAttnArgs(ctypes.Structure):
    _fields_ = [
        ("t", AttnOperands),
        ("q_idx", ctypes.c_void_p), ("k_idx", ctypes.c_void_p), ("sampled_idx", ctypes.c_void_p),
        ("idx_type", ctypes.c_int),
        ("q_idx_stride_b", ctypes.c_int64), ("q_idx_stride_h", ctypes.c_int64), ("q_idx_stride_n", ctypes.c_int64),
        ("k_idx_stride_b", ctypes.c_int64), ("k_idx_stride_h", ctypes.c_int64), ("k_idx_stride_n", ctypes.c_int64),
        ("sampled_stride_b", ctypes.c_int64), ("sampled_stride_h", ctypes.c_int64),
        ("block_size", ctypes.c_int64), ("sample_size", ctypes.c_int64),
        ("smooth_block", ctypes.c_int), ("accumulate", ctypes.c_int),
        ("sampled_pos", ctypes.c_void_p), ("sample_bias", ctypes.c_float), ("mask_sampled_in_block", ctypes.c_int),
    ]


class AttnGrads(ctypes.Structure):
    _fields_ = [
        ("dout", ctypes.c_void_p), ("dq", ctypes.c_void_p), ("dk", ctypes.c_void_p), ("dv", ctypes.c_void_p),
        ("do_stride_b", ctypes.c_int64), ("do_stride_h", ctypes.c_int64), ("do_stride_n", ctypes.c_int64),
        ("dq_stride_b", ctypes.c_int64), ("dq_stride_h", ctypes.c_int64), ("dq_stride_n", ctypes.c_int64),
        ("dk_stride_b", ctypes.c_int64), ("dk_stride_h", ctypes.c_int64), ("dk_stride_n", ctypes.c_int64),
        ("dv_stride_b", ctypes.c_int64), ("dv_stride_h", ctypes.c_int64), ("dv_stride_n", ctypes.c_int64),
        ("workspace", ctypes.c_void_p), ("workspace_bytes", ctypes.c_int64),
        ("accumulate", ctypes.c_int),
    ]


class ForwardArgs(ctypes.Structure):
    _fields_ = [
        ("q", ctypes.c_void_p), ("k", ctypes.c_void_p), ("v", ctypes.c_void_p),
        ("proj", ctypes.c_void_p), ("sampled_idx", ctypes.c_void_p),
        ("out", ctypes.c_void_p), ("lse", ctypes.c_void_p),
        ("batch", ctypes.c_int64), ("heads", ctypes.c_int64), ("kv_heads", ctypes.c_int64),
        ("n", ctypes.c_int64), ("d", ctypes.c_int64), ("dv", ctypes.c_int64),
        ("lsh_num_projs", ctypes.c_int64), ("block_size", ctypes.c_int64),
        ("sample_size", ctypes.c_int64), ("min_seq_len", ctypes.c_int64),
        ("smooth_block", ctypes.c_int), ("causal", ctypes.c_int),
        ("scale", ctypes.c_float), ("dtype", ctypes.c_int),
        ("workspace", ctypes.c_void_p), ("workspace_bytes", ctypes.c_int64),
        ("q_stride_b", ctypes.c_int64), ("q_stride_h", ctypes.c_int64), ("q_stride_n", ctypes.c_int64),
        ("k_stride_b", ctypes.c_int64), ("k_stride_h", ctypes.c_int64), ("k_stride_n", ctypes.c_int64),
        ("v_stride_b", ctypes.c_int64), ("v_stride_h", ctypes.c_int64), ("v_stride_n", ctypes.c_int64),
    ]


_lib = None


def _declare(lib):
    i64, vp, ci = ctypes.c_int64, ctypes.c_void_p, ctypes.c_int
    lib.ha_abi_version.restype = ci
    lib.ha_abi_version.argtypes = []
    lib.ha_last_error.restype = ctypes.c_char_p
    lib.ha_last_error.argtypes = []
    lib.ha_lsh_hash.restype = ci
    lib.ha_lsh_hash.argtypes = [vp, vp, vp] + [i64] * 10 + [ci, vp]
    lib.ha_bucket_argsort_workspace_bytes.restype = i64
    lib.ha_bucket_argsort_workspace_bytes.argtypes = [i64, i64, i64]
    lib.ha_bucket_argsort.restype = ci
    lib.ha_bucket_argsort.argtypes = [vp, vp, ci, i64, i64, i64, i64, i64, vp, i64, vp]
    lib.ha_bucket_argsort_static.restype = ci
    lib.ha_bucket_argsort_static.argtypes = [vp, vp, ci, i64, i64, i64, i64, i64, vp]
    lib.ha_gather_rows.restype = ci
    lib.ha_gather_rows.argtypes = [vp, vp, ci, vp] + [i64] * 9 + [ci, vp]
    lib.ha_block_attn_fwd.restype = ci
    lib.ha_block_attn_fwd.argtypes = [ctypes.POINTER(BlockAttnArgs), vp]
    lib.ha_flash_attn_fwd.restype = ci
    lib.ha_flash_attn_fwd.argtypes = [ctypes.POINTER(AttnOperands), ci, vp]
    lib.ha_attn_bwd_workspace_bytes.restype = i64
    lib.ha_attn_bwd_workspace_bytes.argtypes = [ctypes.POINTER(AttnOperands), i64]
    lib.ha_block_attn_bwd.restype = ci
    lib.ha_block_attn_bwd.argtypes = [ctypes.POINTER(BlockAttnArgs), ctypes.POINTER(AttnGrads), vp]
    lib.ha_flash_attn_bwd.restype = ci
    lib.ha_flash_attn_bwd.argtypes = [ctypes.POINTER(AttnOperands), ci, ctypes.POINTER(AttnGrads), vp]
    lib.ha_lse_merge.restype = ci
    lib.ha_lse_merge.argtypes = [vp] * 6 + [i64] * 8 + [ci, vp]
    lib.ha_lse_merge_segments.restype = ci
    lib.ha_lse_merge_segments.argtypes = [vp] * 7 + [i64] * 13 + [ci, vp]
    lib.ha_forward_workspace_bytes.restype = i64
    lib.ha_forward_workspace_bytes.argtypes = [ctypes.POINTER(ForwardArgs)]
    lib.ha_forward.restype = ci
    lib.ha_forward.argtypes = [ctypes.POINTER(ForwardArgs), vp]
    lib.ha_lse_merge_levels.restype = ci
    lib.ha_lse_merge_levels.argtypes = [vp, vp, ctypes.POINTER(vp), ctypes.POINTER(vp), ctypes.POINTER(vp), vp, vp, vp,
                                        ci, i64, i64, i64, ci, ci, vp]
    lib.ha_power_probe.restype = ci
    lib.ha_power_probe.argtypes = [ci, i64, ci, vp, vp]
    lib.ha_forward_sort.restype = ci
    lib.ha_forward_sort.argtypes = [ctypes.POINTER(ForwardArgs), ctypes.POINTER(i64), ctypes.POINTER(i64),
                                    ctypes.POINTER(ci), vp]


def lib():
    """The loaded shared library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
                "(hipcc, gfx950). There is no fallback path.")
        loaded = ctypes.CDLL(LIB_PATH)
        _declare(loaded)
        if loaded.ha_abi_version() != ABI_VERSION:
            raise RuntimeError("libhyperattn.so: ABI version mismatch")
        _lib = loaded
    return _lib


_ARG_ERRORS = {-1: ValueError, -2: AssertionError, -3: AssertionError, -4: AssertionError,
               -5: NotImplementedError, -6: ValueError}


def check(status: int):
    """Map a C status to the exception type the reference raises for the same mistake."""
    if status == 0:
        return
    msg = lib().ha_last_error().decode("utf-8", "replace")
    if status < 0:
        raise _ARG_ERRORS.get(status, RuntimeError)(msg)
    raise RuntimeError(f"HIP error {status}: {msg}")
