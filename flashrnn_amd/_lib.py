"""ctypes binding of libflashrnn_hip.so (declarations: include/flashrnn_hip.h)."""
from __future__ import annotations

import ctypes
import os
import subprocess
from ctypes import c_char_p, c_int, c_size_t, c_void_p, POINTER

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

FUNCTION_IDS = {"lstm": 0, "slstm": 1, "gru": 2, "elman": 3}
DTYPE_IDS = {"bfloat16": 0, "float32": 1, "float16": 2}

# error codes of include/flashrnn_hip.h
E_ARG, E_UNSUPPORTED, E_NULL, E_ALIGN, E_WORKSPACE, E_DEVICE, E_TOO_LARGE = -1, -2, -3, -4, -5, -6, -7



class Options(ctypes.Structure):
    """frnn_options of include/flashrnn_hip.h (0 / False = option off)."""

    _fields_ = [("struct_size", ctypes.c_uint), ("forward_clipval", ctypes.c_float),
                ("gradient_recurrent_clipval", ctypes.c_float), ("gradient_recurrent_cut", c_int), ("recompute", c_int),
                ("batch_stride", c_int)]

    def __init__(self, forward_clipval=0.0, gradient_recurrent_clipval=0.0, gradient_recurrent_cut=0, recompute=0,
                 batch_stride=0):
        super().__init__(ctypes.sizeof(Options), forward_clipval, gradient_recurrent_clipval, gradient_recurrent_cut,
                         recompute, batch_stride)


_P6 = [c_int] * 6
_FWD = [c_int] * 7 + [c_void_p] * 7 + [c_size_t, c_void_p]
_BWD = _P6 + [c_void_p] * 11 + [c_size_t, c_void_p]
_SIGNATURES = {
    "frnn_last_error": (c_char_p, []),
    "frnn_version": (c_char_p, []),
    "frnn_profile_enable": (None, [c_int]),
    "frnn_profile_reset": (None, []),
    "frnn_profile_count": (c_int, []),
    "frnn_profile_name": (c_char_p, [c_int]),
    "frnn_profile_ms": (ctypes.c_float, [c_int]),
    "frnn_function_dims": (c_int, [c_int] + [POINTER(c_int)] * 5),
    "frnn_fused_supported": (c_int, [c_int] * 5),
    "frnn_fused_plan": (c_int, [c_int] * 6 + [POINTER(c_int)] * 4),
    "frnn_fused_cache_bytes": (c_size_t, _P6),
    "frnn_fused_workspace_bytes": (c_size_t, _P6 + [c_int]),
    "frnn_fused_forward": (c_int, [c_int] * 7 + [c_void_p] * 7 + [c_size_t, c_void_p]),
    "frnn_fused_backward": (c_int, _P6 + [c_void_p] * 11 + [c_size_t, c_void_p]),
    "frnn_alt_supported": (c_int, [c_int] * 5),
    "frnn_alt_cache_bytes": (c_size_t, _P6),
    "frnn_alt_workspace_bytes": (c_size_t, _P6 + [c_int]),
    "frnn_alt_forward": (c_int, [c_int] * 7 + [c_void_p] * 7 + [c_size_t, c_void_p]),
    "frnn_alt_backward": (c_int, _P6 + [c_void_p] * 11 + [c_size_t, c_void_p]),
    "frnn_fused_forward_opt": (c_int, _FWD + [POINTER(Options)]),
    "frnn_fused_backward_opt": (c_int, _BWD + [POINTER(Options)]),
    "frnn_alt_forward_opt": (c_int, _FWD + [POINTER(Options)]),
    "frnn_alt_backward_opt": (c_int, _BWD + [POINTER(Options)]),
    "frnn_fused_cache_bytes_opt": (c_size_t, _P6 + [POINTER(Options)]),
    "frnn_alt_cache_bytes_opt": (c_size_t, _P6 + [POINTER(Options)]),
    "frnn_fused_recompute_supported": (c_int, [c_int] * 5),
    "frnn_fused_max_batch": (c_int, [c_int] * 7 + [POINTER(Options)]),
    "frnn_fused_workspace_bytes_opt": (c_size_t, _P6 + [c_int, POINTER(Options)]),
    "frnn_fused_backward_recompute": (c_int, _P6 + [c_void_p] * 11 + [c_size_t, c_void_p, POINTER(Options)]),
    "frnn_fused_step": (c_int, [c_int] * 5 + [c_void_p] * 7 + [POINTER(Options)]),
    "frnn_alt_step": (c_int, [c_int] * 5 + [c_void_p] * 7 + [POINTER(Options)]),
    "frnn_streams_overlap": (c_int, [c_void_p, c_void_p]),
    "frnn_fused_decode_mailbox_bytes": (c_size_t, _P6),
    "frnn_fused_decode_mailbox_layout": (c_int, _P6 + [POINTER(c_size_t)] * 4),
    "frnn_fused_decode_open": (c_int, [c_int] * 5 + [c_void_p] * 5 + [c_size_t, c_int, c_int, c_int, c_void_p, c_void_p, POINTER(Options)]),
    "frnn_fused_decode_step": (c_int, [c_int] * 6 + [c_void_p] * 3 + [c_size_t, c_int, c_void_p]),
    "frnn_fused_decode_close": (c_int, [c_void_p] * 3),
    "frnn_fused_forward_static_max_bytes": (c_size_t, []),
    "frnn_fused_forward_static": (c_int, [c_int] * 7 + [c_void_p] * 7 + [POINTER(Options)]),
}
EXPORTED_SYMBOLS = tuple(_SIGNATURES)


def library_path() -> str:
    """The in-tree library; FLASHRNN_HIP_LIBRARY overrides it (e.g. an instrumented build)."""
    return os.environ.get("FLASHRNN_HIP_LIBRARY") or os.path.join(_HERE, "libflashrnn_hip.so")


def build_library(jobs: int = 8, force: bool = False) -> str:
    """Compile the HIP sources for gfx950 with hipcc (cross-compiles without a GPU)."""
    src = os.path.join(_HERE, "csrc")
    if force:
        subprocess.run(["make", "-C", src, "clean"], check=True, stdout=subprocess.DEVNULL)
    subprocess.run(["make", "-C", src, f"-j{jobs}"], check=True)
    return library_path()


def load_library():
    """Load the prebuilt library; raises if it is missing (there is no fallback path)."""
    global _LIB
    if _LIB is None:
        path = library_path()
        if not os.path.exists(path):
            raise RuntimeError(
                f"{path} is missing: build it with `make -C {os.path.join(_HERE, 'csrc')}` "
                "(flashrnn_amd has no CPU or PyTorch fallback)")
        lib = ctypes.CDLL(path)
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        _LIB = lib
    return _LIB


def last_error() -> str:
    return load_library().frnn_last_error().decode()
