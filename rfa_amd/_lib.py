"""ctypes loader for librfa_hip.so, the C-ABI kernel library (include/rfa_hip.h).

There is no fallback: if the library has not been built, importing any
kernel-backed function raises, and calling one with tensors that are not on a
HIP device raises as well.
"""
from __future__ import annotations

import ctypes
import os
import re
from ctypes import POINTER, c_char_p, c_double, c_float, c_int, c_int64, c_size_t, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "librfa_hip.so")
HEADER_PATH = os.path.join(os.path.dirname(_HERE), "include", "rfa_hip.h")

RFA_OK = 0
ERROR_NAMES = {
    -1: "RFA_ERR_NULL_POINTER", -2: "RFA_ERR_BAD_SHAPE", -3: "RFA_ERR_UNSUPPORTED",
    -4: "RFA_ERR_ALIGNMENT", -5: "RFA_ERR_WORKSPACE", -6: "RFA_ERR_HIP",
}


class RfaHipError(RuntimeError):
    def __init__(self, code: int, message: str):
        self.code = code
        super().__init__(f"{ERROR_NAMES.get(code, code)}: {message}")


# name -> (restype, argtypes); kept in step with include/rfa_hip.h (tests check it)
SIGNATURES = {
    "rfa_version": (c_int, []),
    "rfa_last_error": (c_char_p, []),
    "rfa_shape_supported": (c_int, [c_int, c_int]),
    "rfa_selftest_layout": (c_int, [c_void_p]),
    "rfa_selftest_mfma_rate": (c_int, [c_int, c_int, c_void_p, ctypes.POINTER(ctypes.c_double), c_void_p]),
    "rfa_causal_num_segments": (c_int, [c_int64, c_int64, c_int, c_int]),
    "rfa_tuning_set": (c_int, [c_char_p, c_int]),
    "rfa_tuning_get": (c_int, [c_char_p, POINTER(c_int)]),
    "rfa_causal_backward_saved_workspace_bytes": (c_size_t, [c_void_p, c_int64, c_int64, c_int, c_int]),
    "rfa_causal_saved_describe": (c_int, [c_void_p, POINTER(ctypes.c_int32), c_void_p]),
    "rfa_causal_forward_workspace_bytes": (c_size_t, [c_int64, c_int64, c_int, c_int]),
    "rfa_causal_forward": (c_int, [c_void_p] * 4 + [c_int64, c_int64, c_int, c_int, c_void_p, c_size_t, c_void_p]),
    "rfa_static_scratch_bytes": (c_size_t, []),
    "rfa_causal_forward_noalloc": (c_int, [c_void_p] * 4 + [c_int64, c_int64, c_int, c_int, c_void_p]),
    "rfa_causal_prefill": (c_int, [c_void_p] * 6 + [c_int64, c_int64, c_int, c_int, c_void_p, c_size_t, c_void_p]),
    "rfa_causal_backward_workspace_bytes": (c_size_t, [c_int64, c_int64, c_int, c_int]),
    "rfa_causal_backward": (c_int, [c_void_p] * 7 + [c_int64, c_int64, c_int, c_int, c_void_p, c_size_t, c_void_p]),
    "rfa_causal_saved_state_bytes": (c_size_t, [c_int64, c_int64, c_int, c_int]),
    "rfa_causal_forward_save": (c_int, [c_void_p] * 5 + [c_size_t, c_int64, c_int64, c_int, c_int, c_void_p, c_size_t, c_void_p]),
    "rfa_causal_backward_saved": (c_int, [c_void_p] * 6 + [c_size_t] + [c_void_p] * 3 + [c_int64, c_int64, c_int, c_int, c_void_p, c_size_t, c_void_p]),
    "rfa_feature_map_supported": (c_int, [c_int, c_int]),
    "rfa_build_random_matrices": (c_int, [c_void_p, c_void_p, c_float, c_void_p, c_int, c_int, c_int, c_void_p]),
    "rfa_build_random_matrices_backward": (c_int, [c_void_p] * 3 + [c_float, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]),
    "rfa_feature_map_forward": (c_int, [c_void_p] * 3 + [c_int64, c_int, c_int, c_int, c_float, c_void_p]),
    "rfa_feature_map_forward_pair": (c_int, [c_void_p] * 5 + [c_int64, c_int, c_int, c_int, c_float, c_void_p]),
    "rfa_feature_map_backward_workspace_bytes": (c_size_t, [c_int64, c_int, c_int, c_int]),
    "rfa_feature_map_backward": (c_int, [c_void_p] * 5 + [c_int64, c_int, c_int, c_int, c_float, c_void_p, c_size_t, c_void_p]),
    "rfa_feature_map_backward_pair_workspace_bytes": (c_size_t, [c_int64, c_int, c_int, c_int]),
    "rfa_feature_map_backward_pair": (c_int, [c_void_p] * 8 + [c_int64, c_int, c_int, c_int, c_float, c_void_p, c_size_t, c_void_p]),
    "rfa_feature_map_backward_pair_packed": (c_int, [c_void_p] * 8 + [c_int64, c_int, c_int, c_int, c_float, c_void_p, c_size_t, c_void_p]),
    "rfa_project_feature_map": (c_int, [c_void_p] * 5 + [c_int, c_void_p, c_int64, c_int, c_int, c_int, c_int, c_float, c_void_p]),
    "rfa_linear_weight_grad_workspace_bytes": (c_size_t, [c_int64, c_int, c_int, c_int]),
    "rfa_linear_weight_grad": (c_int, [c_void_p] * 4 + [c_int, c_int64, c_int, c_int, c_void_p, c_size_t, c_void_p]),
    "rfa_cross_state": (c_int, [c_void_p] * 5 + [c_int64, c_int64, c_int, c_int, c_int, c_void_p]),
    "rfa_cross_readout": (c_int, [c_void_p] * 4 + [c_int64, c_int64, c_int, c_int, c_void_p]),
    "rfa_cross_readout_backward": (c_int, [c_void_p] * 7 + [c_int64, c_int64, c_int, c_int, c_void_p]),
    "rfa_cross_state_backward": (c_int, [c_void_p] * 7 + [c_int64, c_int64, c_int, c_int, c_int, c_void_p]),
    "rfa_masked_forward": (c_int, [c_void_p] * 7 + [c_int64, c_int64, c_int64, c_int, c_int, c_int, c_void_p]),
    "rfa_masked_backward_workspace_bytes": (c_size_t, [c_int64, c_int64, c_int]),
    "rfa_masked_backward": (c_int, [c_void_p] * 12 + [c_int64, c_int64, c_int64, c_int, c_int, c_int, c_void_p, c_size_t, c_void_p]),
    "rfa_incremental": (c_int, [c_void_p] * 6 + [c_int64, c_int64, c_int, c_int, c_void_p]),
    "rfa_profile_enable": (c_int, [c_int]),
    "rfa_profile_collect": (c_int, []),
    "rfa_profile_reset": (c_int, []),
    "rfa_profile_kernel_count": (c_int, []),
    "rfa_profile_get": (c_int, [c_int, POINTER(c_char_p), POINTER(c_double), POINTER(c_int64)]),
    "rfa_incremental_fused": (c_int, [c_void_p] * 4 + [c_float] + [c_void_p] * 3 + [c_int64, c_int64, c_int, c_int, c_int, c_void_p]),
    "rfa_incremental_out": (c_int, [c_void_p] * 8 + [c_int64, c_int64, c_int, c_int, c_void_p]),
    "rfa_incremental_fused_out": (c_int, [c_void_p] * 4 + [c_float] + [c_void_p] * 5 + [c_int64, c_int64, c_int, c_int, c_int, c_void_p]),
    "rfa_incremental_qkv": (c_int, [c_void_p] * 2 + [c_float] + [c_void_p] * 5 + [c_int64, c_int64, c_int, c_int, c_int, c_void_p]),
}

_lib = None


def load() -> ctypes.CDLL:
    """Load the library once; raise ImportError with build instructions if absent."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `python -m rfa_amd.build` "
                "(hipcc, --offload-arch=gfx950). There is no CPU fallback.")
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def check(code: int) -> None:
    if code != RFA_OK:
        raise RfaHipError(code, load().rfa_last_error().decode())


def declared_symbols() -> list:
    """Function names declared in include/rfa_hip.h."""
    with open(HEADER_PATH) as f:
        text = re.sub(r"/\*.*?\*/", "", f.read(), flags=re.S)
    return sorted(set(re.findall(r"\b(rfa_[a-z0-9_]+)\s*\(", text)))


def tuning_set(name: str, value: int) -> None:
    """Override a launch heuristic of the library (-1 restores it); see rfa_tuning_set in the header."""
    check(load().rfa_tuning_set(name.encode(), int(value)))


def tuning_get(name: str) -> int:
    v = c_int(0)
    check(load().rfa_tuning_get(name.encode(), ctypes.byref(v)))
    return v.value


class tuning:
    """``with tuning(nseg=2, prefix=1): ...`` sets knobs for the block and puts the old values back."""

    def __init__(self, **knobs):
        self.knobs = knobs
        self.old = {}

    def __enter__(self):
        for name, value in self.knobs.items():
            self.old[name] = tuning_get(name)
            tuning_set(name, value)
        return self

    def __exit__(self, *exc):
        for name, value in self.old.items():
            tuning_set(name, value)
        return False


def profile_totals() -> dict:
    """{kernel name: (total_ms, calls)} accumulated since the last rfa_profile_reset."""
    lib = load()
    check(lib.rfa_profile_collect())
    out = {}
    for i in range(lib.rfa_profile_kernel_count()):
        name, ms, calls = c_char_p(), c_double(), c_int64()
        check(lib.rfa_profile_get(i, name, ms, calls))
        if calls.value:
            out[name.value.decode()] = (ms.value, calls.value)
    return out
