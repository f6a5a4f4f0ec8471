"""ctypes binding of ``libnf4hip.so`` (C ABI in ``include/nf4hip.h``).

The library is built in-tree (``lightning-thunder_amd/libnf4hip.so``) by
``__graft_entry__.build()`` / ``make -C lightning-thunder_amd/csrc``.  There is no CPU fallback:
if the library is missing or its ABI version differs, every op raises.
"""

from __future__ import annotations

import ctypes
import os
import threading

ABI_VERSION = 6

BF16, F16, F32 = 0, 1, 2

STATIC_SCRATCH_BYTES = 4 << 20  # NF4HIP_STATIC_SCRATCH_BYTES

E_NULL, E_DTYPE, E_BLOCKSIZE, E_SHAPE, E_ALIGN, E_WORKSPACE, E_HIP = -1, -2, -3, -4, -5, -6, -7

_ERROR_NAMES = {
    E_NULL: "NF4HIP_E_NULL",
    E_DTYPE: "NF4HIP_E_DTYPE",
    E_BLOCKSIZE: "NF4HIP_E_BLOCKSIZE",
    E_SHAPE: "NF4HIP_E_SHAPE",
    E_ALIGN: "NF4HIP_E_ALIGN",
    E_WORKSPACE: "NF4HIP_E_WORKSPACE",
    E_HIP: "NF4HIP_E_HIP",
}

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libnf4hip.so")

# every symbol include/nf4hip.h declares: name -> (restype, argtypes)
_vp, _i32, _i64, _f32, _sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_float, ctypes.c_size_t
_MATMUL = [_vp, _i32, _i64, _vp, _vp, _vp, _vp, _i64, _i64, _i32, _vp, _vp, _sz, _vp]
_MATMUL_DQ = [_vp, _i32, _i64, _vp, _vp, _vp, _vp, _f32, _i32, _vp, _vp, _i64, _i64, _i32, _vp, _vp, _sz, _vp]


class Epilogue(ctypes.Structure):
    """``nf4hip_epilogue`` of include/nf4hip.h."""

    _fields_ = [("flags", _i32), ("eps", _f32), ("in_sumsq", _vp), ("in_parts", _i32), ("resid_in", _vp),
                ("norm_weight", _vp), ("resid_out", _vp), ("xnext_out", _vp), ("out_sumsq", _vp)]


EPI_ROWSCALE, EPI_SILU_PAIRS, EPI_RESID_NORM = 1, 2, 4

SYMBOLS = {
    "nf4hip_abi_version": (_i32, []),
    "nf4hip_last_error": (ctypes.c_char_p, []),
    "nf4hip_quantize": (_i32, [_vp, _i32, _i64, _i32, _vp, _vp, _vp]),
    "nf4hip_dequantize": (_i32, [_vp, _vp, _vp, _i64, _i32, _vp, _i32, _vp]),
    "nf4hip_dq_compress": (_i32, [_vp, _i64, _i32, _vp, _f32, _vp, _vp, _vp]),
    "nf4hip_dq_reconstruct": (_i32, [_vp, _vp, _vp, _f32, _i64, _i32, _vp, _vp]),
    "nf4hip_dequantize_dq": (_i32, [_vp, _vp, _vp, _vp, _f32, _i32, _vp, _i64, _i32, _vp, _i32, _vp]),
    "nf4hip_gemv_workspace_bytes": (_sz, [_i64, _i64, _i64]),
    "nf4hip_gemv_prefer_staged": (_i32, [_i32]),
    "nf4hip_gemv": (_i32, _MATMUL),
    "nf4hip_gemv_dq": (_i32, _MATMUL_DQ),
    "nf4hip_gemv_epilogue": (_i32, _MATMUL[:-1] + [ctypes.POINTER(Epilogue), _vp]),
    "nf4hip_gemv_norm_parts": (_i32, [_i64, _i64, _i64]),
    "nf4hip_gemv_epilogue_served": (_i32, [_i64, _i64, _i64, _i32, _i32, _i32]),
    "nf4hip_gemv_static": (_i32, [_vp, _i32, _i64, _vp, _vp, _vp, _vp, _i64, _i64, _i32, _vp, _vp]),
    "nf4hip_gemv_plan": (_i32, [_i64, _i64, _i64, _i32, _i32, ctypes.POINTER(_i32 * 4)]),
    "nf4hip_gemm_workspace_bytes": (_sz, [_i64, _i64, _i64]),
    "nf4hip_gemm_plan": (_i32, [_i64, _i64, _i64, ctypes.POINTER(_i32 * 4)]),
    "nf4hip_gemm": (_i32, _MATMUL),
    "nf4hip_gemm_dq": (_i32, _MATMUL_DQ),
    "nf4hip_linear_workspace_bytes": (_sz, [_i64, _i64, _i64]),
    "nf4hip_linear_plan": (_i32, [_i64, _i64, _i64, ctypes.POINTER(_i32 * 4)]),
    "nf4hip_linear": (_i32, [_vp, _i32, _i64, _vp, _vp, _i64, _i64, _vp, _vp, _sz, _vp]),
}


class NF4HipError(RuntimeError):
    """A call into libnf4hip.so returned a negative status."""

    def __init__(self, code: int, message: str):
        self.code = code
        super().__init__(f"{_ERROR_NAMES.get(code, code)}: {message}")


_lib = None
_lock = threading.Lock()


def load(path: str | None = None) -> ctypes.CDLL:
    """Load (once) and return the shared library; raises if it is absent or of another ABI."""
    global _lib
    if _lib is not None and path is None:
        return _lib
    with _lock:
        if _lib is not None and path is None:
            return _lib
        p = path or LIB_PATH
        if not os.path.exists(p):
            raise RuntimeError(
                f"{p} not found: the HIP extension has not been built "
                "(run `python -c 'import __graft_entry__ as g; g.build()'` or `make -C lightning-thunder_amd/csrc`). "
                "There is no CPU fallback."
            )
        lib = ctypes.CDLL(p)
        for name, (restype, argtypes) in SYMBOLS.items():
            fn = getattr(lib, name)  # AttributeError if the library lacks a declared symbol
            fn.restype = restype
            fn.argtypes = argtypes
        got = lib.nf4hip_abi_version()
        if got != ABI_VERSION:
            raise RuntimeError(f"{p}: ABI version {got}, host code expects {ABI_VERSION}")
        if path is None:
            _lib = lib
        return lib


def check(rc: int) -> None:
    if rc != 0:
        raise NF4HipError(rc, load().nf4hip_last_error().decode("utf-8", "replace"))
