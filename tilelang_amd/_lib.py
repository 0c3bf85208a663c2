"""ctypes loader for ``libdqgemm.so`` (the C-ABI declared in ``include/dqgemm.h``).

The reference loads each JIT-built kernel library with ``ctypes.CDLL`` and calls ``init()``
once (tilelang/jit/adapter/libgen.py:52-57, tilelang/jit/adapter/cython/adapter.py:131-140).
Here there is one ahead-of-time library.  There is no fallback: if it is missing or fails
to load, every kernel call raises.
"""

from __future__ import annotations

import ctypes
import os
import subprocess
import threading

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG_DIR, "libdqgemm.so")
CSRC_DIR = os.path.join(_PKG_DIR, "csrc")

_lock = threading.Lock()
_lib = None
_initialised_devices: set = set()

_vp, _i = ctypes.c_void_p, ctypes.c_int

#: name -> argtypes; every entry point returns int (0 ok / -1 error) except get_last_error and SIZE_QUERIES
SIGNATURES = {
    "init": [],
    "call_dequantize_gemv_w4a16": [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp],
    "call_dequantize_gemv_w4a16_ws": [_vp, _vp, _vp, _vp, _vp, _vp, ctypes.c_size_t, _i, _i, _i, _i, _i, _i, _i, _vp],
    "call_dequantize_gemv_lowbit": [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _vp],
    "call_unpack_qzeros": [_vp, _vp, _i, _i, _i, _vp],
    "call_dequantize_w4": [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp],
    "call_dequant_gemm_bf16_mxfp4": [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp],
    "call_dequant_gemm_bf16_fp4": [_vp, _vp, _vp, _i, _i, _i, _i, _vp],
    "call_dequant_gemm_fp16_fp4": [_vp, _vp, _vp, _i, _i, _i, _i, _vp],
    "call_dequant_gemm_fp16_fp4_splitk": [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp],
    "call_dequant_gemm_fp16_fp4_splitk_static": [_vp, _vp, _vp, _i, _i, _i, _i, _i, _vp],
    "call_dequant_gemm_w4_fp16": [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp],
    "call_gemm_int8xint2": [_vp, _vp, _vp, _i, _i, _i, _i, _i, _vp, ctypes.c_float, _i, _vp],
    "call_bitnet_activation_quant": [_vp, _vp, _vp, _i, _i, _vp],
    "call_quantize_bf16_mxfp4": [_vp, _vp, _vp, _i, _i, _i, _vp],
    "call_gemm_int8xint4": [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp],
    "call_gemv_int8xint1": [_vp, _vp, _vp, _i, _i, _i, _i, _i, _vp],
    "call_gemm_plain": [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp],
    "call_mfma_rate": [_vp, _vp, _i, _i, _i, _vp],
    "call_gemm_mxfp4_mxfp4": [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp],
}

#: name -> argtypes of the functions that return a byte count (size_t) and launch nothing
SIZE_QUERIES = {
    "dq_w4a16_workspace_bytes": [_i, _i, _i, _i, _i],
}


class LibraryNotBuiltError(RuntimeError):
    pass


def build_library(jobs: int = 8, clean: bool = False) -> str:
    """Compile every HIP source for gfx950 into ``libdqgemm.so`` (hipcc cross-compiles without a GPU)."""
    if clean:
        subprocess.run(["make", "-C", CSRC_DIR, "clean"], check=True, capture_output=True)
    proc = subprocess.run(["make", "-C", CSRC_DIR, f"-j{jobs}"], capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"building libdqgemm.so failed:\n{proc.stdout[-4000:]}\n{proc.stderr[-4000:]}")
    return LIB_PATH


def load_library() -> ctypes.CDLL:
    """Load the library and bind the signatures (no GPU call is made)."""
    global _lib
    with _lock:
        if _lib is None:
            if not os.path.exists(LIB_PATH):
                raise LibraryNotBuiltError(
                    f"{LIB_PATH} is missing: build it with `make -C {CSRC_DIR}` "
                    "(or `python -c 'import __graft_entry__ as g; g.build()'`). There is no fallback path."
                )
            lib = ctypes.CDLL(LIB_PATH)
            lib.get_last_error.restype = ctypes.c_char_p
            lib.get_last_error.argtypes = []
            for name, argtypes in SIGNATURES.items():
                fn = getattr(lib, name)
                fn.restype = ctypes.c_int
                fn.argtypes = argtypes
            for name, argtypes in SIZE_QUERIES.items():
                fn = getattr(lib, name)
                fn.restype = ctypes.c_size_t
                fn.argtypes = argtypes
            _lib = lib
    return _lib


def get_library(device_index: int | None = None) -> ctypes.CDLL:
    """Library ready for kernel calls on the CURRENT device: loaded, and ``init()`` (architecture check, LDS limit,
    the device's copy of the static scratch buffer) run once per device.  ``device_index`` names the current device
    when the caller knows it; ``None`` asks torch (and falls back to one ``init()`` per process when torch sees no
    GPU runtime, in which case ``init()`` itself reports the error).

    Calls through ``call_dequant_gemm_fp16_fp4_splitk_static`` share one scratch buffer per GPU: two of them that
    overlap in time on one GPU (different streams, or two captured graphs replayed concurrently) race on it."""
    lib = load_library()
    if device_index is None:
        try:
            import torch

            device_index = torch.cuda.current_device() if torch.cuda.is_available() else -1
        except ImportError:
            device_index = -1
    if device_index not in _initialised_devices:
        with _lock:
            if device_index not in _initialised_devices:
                if lib.init() != 0:
                    raise RuntimeError(f"libdqgemm init failed: {lib.get_last_error().decode()}")
                _initialised_devices.add(device_index)
    return lib


def last_error() -> str:
    return load_library().get_last_error().decode("utf-8", "replace")
