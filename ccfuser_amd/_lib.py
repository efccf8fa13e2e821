"""ctypes binding of libccfuser_moe.so (the C ABI declared in include/ccfuser_moe.h).

The library is loaded on first use.  There is no CPU fallback: if it has not
been built, or a call fails, the caller gets an exception.
"""
from __future__ import annotations

import ctypes as C
import os
from pathlib import Path
from typing import Optional

# CCFUSER_MOE_LIB overrides the path (to compare two builds in one process launch each)
LIB_PATH = Path(os.environ.get("CCFUSER_MOE_LIB") or Path(__file__).resolve().parent / "libccfuser_moe.so")

_lib: Optional[C.CDLL] = None

_p = C.c_void_p
_i = C.c_int
_sz = C.c_size_t

# name -> (restype, argtypes); mirrors include/ccfuser_moe.h declaration by declaration
SIGNATURES = {
    "ccf_version": (_i, []),
    "ccf_last_error": (C.c_char_p, []),
    "ccf_set_option": (_i, [C.c_char_p, _i]),
    "ccf_gate_topk_softmax": (_i, [_p, _p, _p, _i, _i, _i, _i, _i, _p, _p, _p, _p]),
    "ccf_gate_backward_workspace_bytes": (_sz, [_i, _i]),
    "ccf_gate_backward": (_i, [_p, _p, _p, _i, _i, _i, _p, _p, _p, _sz, _p]),
    "ccf_route_workspace_bytes": (_sz, [_i, _i]),
    "ccf_expert_count": (_i, [_p, _i, _p, _i, _p]),
    "ccf_assign_pos": (_i, [_p, _p, _i, _i, _p, _p, _sz, _p]),
    "ccf_route": (_i, [_p, _i, _i, _i, _i, _p, _p, _p, _p, _p, _p, _p, _p, _sz, _p]),
    "ccf_route_static": (_i, [_p, _i, _i, _i, _i, _p, _p, _p, _p, _p, _p, _p, _p]),
    "ccf_route_static_max_entries": (_i, []),
    "ccf_plan_blocks": (_i, [_p, _i, _i, _i, _i, _p, _p, _p, _p, _p, _p, _p, _p]),
    "ccf_segments_to_rows": (_i, [_p, _p, _p, _i, _i, _i, _p, _p, _p, _p]),
    "ccf_local_scatter": (_i, [_p, _p, _p, _i, _i, _p]),
    "ccf_local_gather": (_i, [_p, _p, _p, _i, _i, _p]),
    "ccf_combine": (_i, [_p, _p, _p, _p, _i, _i, _i, _p]),
    "ccf_ffn_workspace_bytes": (_sz, [_i, _i, _i, _i]),
    "ccf_ffn_plan_info": (_i, [_p, _i, _i, _i, _i, _i, C.POINTER(C.c_int32), _p]),
    "ccf_ffn1_forward": (_i, [_p, _p, _p, _p, _i, _i, _i, _i, _p, _p, _i, _p, _p, _sz, _p]),
    "ccf_ffn2_forward": (_i, [_p, _p, _p, _p, _i, _i, _i, _i, _p, _p, _p, _p, _p, _sz, _p]),
    "ccf_combine_backward": (_i, [_p, _p, _p, _p, _i, _i, _i, _p, _p, _p]),
    "ccf_ffn_backward_workspace_bytes": (_sz, [_i, _i, _i, _i]),
    "ccf_ffn1_forward_keep": (_i, [_p, _p, _p, _i, _i, _i, _i, _p, _p, _p, _p, _p, _sz, _p]),
    "ccf_ffn2_backward": (_i, [_p, _p, _p, _p, _p, _i, _i, _i, _i, _p, _p, _p, _p, _p, _sz, _p]),
    "ccf_ffn1_backward": (_i, [_p, _p, _p, _p, _p, _i, _i, _i, _i, _p, _p, _p, _p, _p, _sz, _p]),
    "ccf_ffn1_backward_gelu": (_i, [_p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _p, _p, _p, _p, _p, _sz, _p]),
    "ccf_moe_workspace_bytes": (_sz, [_i, _i, _i, _i, _i]),
    "ccf_moe_forward": (_i, [_p] * 7 + [_i] * 6 + [_p] * 6 + [_p, _sz, _p]),
    "ccf_moe_forward_set_events": (_i, [C.POINTER(_p), _i]),
    "ccf_segments_workspace_bytes": (_sz, [_i, _i, _i, _i, _i]),
    "ccf_moe_ffn_segments": (_i, [_p, _p, _p, _p, _i, _i, _i, _i, _i, _p, _p, _p, _p, _p, _p, _sz, _p]),
}


# libccfuser_probe.so (include/ccfuser_probe.h): measurement probes, not part of the product ABI
PROBE_LIB_PATH = Path(__file__).resolve().parent / "libccfuser_probe.so"
PROBE_SIGNATURES = {
    "ccf_probe_mfma": (_i, [_i, _i, _i, _p, C.POINTER(C.c_double), _p]),
    "ccf_probe_mfma_chain": (_i, [_p, _p, _i, _i, _p, _p]),
}
_probe: Optional[C.CDLL] = None


class CcfError(RuntimeError):
    """A C-ABI call returned a non-zero code."""

    def __init__(self, fn: str, code: int, text: str):
        super().__init__(f"{fn} failed with code {code}: {text}")
        self.code = code


def lib() -> C.CDLL:
    """The loaded library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            raise RuntimeError(
                f"{LIB_PATH} is missing: the HIP library has not been built. "
                "Run `python -m ccfuser_amd.build` (needs hipcc); there is no CPU fallback.")
        handle = C.CDLL(str(LIB_PATH))
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)       # AttributeError if the symbol is not exported
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def probe_lib() -> C.CDLL:
    """The loaded probe library (bench.py and one GPU test use it); raises if it has not been built."""
    global _probe
    if _probe is None:
        if not PROBE_LIB_PATH.exists():
            raise RuntimeError(f"{PROBE_LIB_PATH} is missing: run `python -m ccfuser_amd.build`")
        handle = C.CDLL(str(PROBE_LIB_PATH))
        for name, (res, args) in PROBE_SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _probe = handle
    return _probe


def call(name: str, *args) -> None:
    """Call an int-returning entry point and raise CcfError on failure."""
    handle = lib()
    rc = getattr(handle, name)(*args)
    if rc != 0:
        raise CcfError(name, rc, handle.ccf_last_error().decode("utf-8", "replace"))
