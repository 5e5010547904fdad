"""ctypes binding of libparrot_hip.so (the C ABI declared in include/parrot_hip.h).

The library is mandatory: there is no CPU or PyTorch fallback behind these
bindings.  ``load()`` raises ``RuntimeError`` when the shared object has not
been built (``python -m parrotserve_amd.build``).
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int64, c_size_t, c_void_p
from typing import Dict, List, Tuple

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(PKG_DIR, "libparrot_hip.so")

PH_F16, PH_BF16, PH_F32 = 0, 1, 2
PH_IDX_I32, PH_IDX_I64 = 0, 1
PH_OK, PH_ERR_DTYPE, PH_ERR_HEAD_DIM, PH_ERR_ALIGN, PH_ERR_ARG, PH_ERR_WORKSPACE, PH_ERR_LAUNCH, PH_ERR_SCRATCH = range(8)

P, I, L, F, Z = c_void_p, c_int, c_int64, c_float, c_size_t

# name -> (restype, argtypes); must list every symbol of include/parrot_hip.h
SIGNATURES: Dict[str, Tuple[object, List[object]]] = {
    "ph_status_string": (c_char_p, [I]),
    "ph_abi_version": (I, []),
    "ph_move_tokens": (I, [P, P, P, P, I, L, L, L, I, L, L, L, L, L, L, P]),
    "ph_kv_append": (I, [P, P, P, P, P, I, L, L, L, I, L, L, L, P]),
    "ph_gather_blocked_k": (I, [P, P, P, P, I, L, L, L, L, L, I, L, L, L, L, L, L, L, L, P]),
    "ph_gather_blocked_v": (I, [P, P, P, P, I, L, L, L, L, I, L, L, L, L, L, L, L, P]),
    "ph_rms_norm": (I, [P, P, P, F, L, L, L, L, I, I, P]),
    "ph_rope_neox": (I, [P, P, P, P, L, L, L, L, L, L, L, I, P]),
    "ph_rotary_embedding": (I, [P, P, P, L, L, L, L, L, L, I, P]),
    "ph_decode_workspace_bytes": (Z, [L, L, L, L, L, L, L, L]),
    "ph_decode_suffix_lanes": (L, [L, L, L, I, L, L, L, L]),
    "ph_decode_attention": (I, [P, P, P, P, L, L, L, I, L, L, L, F, L, P, P, P, P, L, P, P, L, L, P, L, L, P, P, Z, P]),
    "ph_decode_attention_gqa": (I, [P, P, P, P, L, L, L, P, L, L, I, L, L, L, F, L, P, P, P, P, L, P, P, L, L, P, L, L, P, P, Z,
                                    P]),
    "ph_prefix_attention": (I, [P, P, P, P, P, P, L, L, L, I, L, L, L, F, P, L, P, Z, P]),
    "ph_suffix_post_attention": (I, [P, P, P, P, P, P, L, L, L, I, L, L, L, F, P, P, L, L, P, L, L, P, Z, P]),
    "ph_suffix_prev_attention": (I, [P, P, P, P, P, P, L, L, L, I, L, L, L, F, P, P, L, L, P, L, L, P, Z, P]),
    "ph_prefix_post_attention": (I, [P, P, P, P, P, P, L, L, L, I, L, L, L, F, P, L, P, Z, P]),
    "ph_add_rms_norm": (I, [P, P, P, P, F, L, L, L, L, L, I, I, P]),
    "ph_silu_mul": (I, [P, P, P, L, L, L, L, L, I, P]),
    "ph_rope_append": (I, [P, P, P, P, P, P, P, P, I, L, L, L, L, L, L, L, L, L, I, I, P]),
    "ph_suffix_tables_append": (I, [P, L, P, P, P, L, P]),
    "ph_decode_static_scratch_bytes": (Z, []),
    "ph_decode_attention_static": (I, [P, P, P, P, L, L, L, I, L, L, L, F, L, P, P, P, P, L, P, P, L, L, P, L, L, P, P]),
    "ph_decode_attention_timed": (I, [P, P, P, P, L, L, L, I, L, L, L, F, L, P, P, P, P, L, P, P, L, L, P, L, L, P, P, Z, P, P]),
    "ph_suffix_plan_build": (I, [P, L, L, L, P, P, P, P]),
    "ph_sample_top_p": (I, [P, L, P, P, P, P, L, L, I, P]),
    "ph_top_p_probs": (I, [P, L, P, P, P, L, L, L, I, P]),
    "ph_prefill_workspace_bytes": (Z, [L, L, L, I, L]),
    "ph_prefill_attention": (I, [P, P, P, P, L, L, L, L, I, L, L, L, F, P, P, P, L, L, P, Z, P]),
}



class SuffixPlan(ctypes.Structure):
    """ph_suffix_plan: host struct of device pointers."""

    _fields_ = [("items", c_void_p), ("num_items", c_int64), ("lane_rec", c_void_p), ("num_lanes", c_int64),
                ("req_item_cu", c_void_p)]


_lib = None


def load() -> ctypes.CDLL:
    """Load the shared library once and attach the prototypes."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: the HIP extension is mandatory (no fallback). "
            "Build it with `python -m parrotserve_amd.build`."
        )
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is not exported
        fn.restype = res
        fn.argtypes = args
    if hasattr(lib, "ph_timeline_read"):  # profiling variant of the library (build.TIMELINE_LIB_PATH)
        lib.ph_timeline_read.restype = c_int
        lib.ph_timeline_read.argtypes = [c_void_p, c_size_t]
        lib.ph_timeline_read_clocks.restype = c_int
        lib.ph_timeline_read_clocks.argtypes = [c_void_p, c_size_t]
        lib.ph_timeline_clear.restype = c_int
        lib.ph_timeline_clear.argtypes = []
    _lib = lib
    return lib


def status_string(code: int) -> str:
    return load().ph_status_string(code).decode()


def check(code: int, what: str) -> None:
    """Translate a non-zero status the way the reference's extension surfaces
    errors: unsupported dtype / head size / launch failures are RuntimeError
    (TORCH_CHECK, csrc/attention/attention_kernels.cu:482,535,568); malformed
    arguments are ValueError."""
    if code == PH_OK:
        return
    msg = f"{what}: {status_string(code)} (status {code})"
    if code in (PH_ERR_ARG, PH_ERR_ALIGN):
        raise ValueError(msg)
    raise RuntimeError(msg)
