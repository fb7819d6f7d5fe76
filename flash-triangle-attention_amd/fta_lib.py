"""ctypes binding of libfta.so (see include/fta.h).  No torch types cross this boundary."""
from __future__ import annotations

import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libfta.so")
MAX_L2 = 4096  # FTA_MAX_L2 of include/fta.h
STATIC_WORKSPACE_BYTES = 128 * 1024 * 1024  # FTA_STATIC_WORKSPACE_BYTES of include/fta.h


class Tensor5(ctypes.Structure):
    _fields_ = [("ptr", ctypes.c_void_p), ("stride", ctypes.c_int64 * 4)]


class Tensor4(ctypes.Structure):
    _fields_ = [("ptr", ctypes.c_void_p), ("stride", ctypes.c_int64 * 3)]


class Options(ctypes.Structure):
    _fields_ = [("dtype", ctypes.c_int), ("dbias_f32", ctypes.c_int), ("dropout_p", ctypes.c_float), ("seed", ctypes.c_uint64),
                ("precise", ctypes.c_int)]


DTYPE_F16, DTYPE_BF16 = 0, 1


class FtaError(RuntimeError):
    def __init__(self, status: int, message: str):
        super().__init__(f"libfta: {message} (status {status})")
        self.status = status


_lib = None

PO = ctypes.POINTER(Options)
P5 = ctypes.POINTER(Tensor5)
P4 = ctypes.POINTER(Tensor4)
_DIMS = [ctypes.c_int] * 5

SIGNATURES = {
    "fta_version": (ctypes.c_int, []),
    "fta_seq_len_supported": (ctypes.c_int, [ctypes.c_int, ctypes.c_int]),
    "fta_seq_len_supported_ex": (ctypes.c_int, [ctypes.c_int, ctypes.c_int, PO]),
    "fta_strerror": (ctypes.c_char_p, [ctypes.c_int]),
    "fta_debug_select_kernels": (ctypes.c_int, [ctypes.c_int]),
    "fta_describe_plan": (ctypes.c_int, _DIMS + [ctypes.c_char_p, ctypes.c_size_t]),
    "fta_describe_plan_ex": (ctypes.c_int, _DIMS + [ctypes.c_float, PO, ctypes.c_char_p, ctypes.c_size_t]),
    "fta_check_fwd": (ctypes.c_int, [P5, P5, P5, P4, P5, ctypes.c_void_p] + _DIMS + [ctypes.c_float]),
    "fta_fwd": (ctypes.c_int, [P5, P5, P5, P4, P5, ctypes.c_void_p] + _DIMS + [ctypes.c_float, ctypes.c_void_p]),
    "fta_bwd_workspace_bytes": (ctypes.c_size_t, _DIMS),
    "fta_bwd_workspace_bytes_ex": (ctypes.c_size_t, _DIMS + [PO]),
    "fta_fwd_ex": (ctypes.c_int, [P5, P5, P5, P4, P5, ctypes.c_void_p] + _DIMS + [ctypes.c_float, PO, ctypes.c_void_p]),
    "fta_bwd_ex": (ctypes.c_int, [P5, P5, P5, P4, P5, ctypes.c_void_p, P5, P5, P5, P5, P4, ctypes.c_void_p,
                                  ctypes.c_size_t] + _DIMS + [ctypes.c_float, PO, ctypes.c_void_p]),
    "fta_dropout_mask": (ctypes.c_int, [PO, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p,
                                        ctypes.c_void_p]),
    "fta_check_bwd": (ctypes.c_int, [P5, P5, P5, P4, P5, ctypes.c_void_p, P5, P5, P5, P5, P4, ctypes.c_void_p,
                                     ctypes.c_size_t] + _DIMS + [ctypes.c_float]),
    "fta_bwd": (ctypes.c_int, [P5, P5, P5, P4, P5, ctypes.c_void_p, P5, P5, P5, P5, P4, ctypes.c_void_p,
                               ctypes.c_size_t] + _DIMS + [ctypes.c_float, ctypes.c_void_p]),
    "fta_bwd_noalloc": (ctypes.c_int, [P5, P5, P5, P4, P5, ctypes.c_void_p, P5, P5, P5, P5, P4] + _DIMS
                        + [ctypes.c_float, ctypes.c_void_p]),
    "fta_bwd_profile": (ctypes.c_int, [P5, P5, P5, P4, P5, ctypes.c_void_p, P5, P5, P5, P5, P4, ctypes.c_void_p,
                                       ctypes.c_size_t] + _DIMS + [ctypes.c_float, ctypes.c_void_p,
                                                                   ctypes.POINTER(ctypes.c_float)]),
}


def load() -> ctypes.CDLL:
    """Loads the in-tree library; fails loudly when it has not been built (there is no fallback)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `python flash-triangle-attention_amd/build.py` "
                "(hipcc, gfx950). The HIP library is the only implementation of attention().")
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def strerror(status: int) -> str:
    return load().fta_strerror(int(status)).decode()


def describe_plan(B: int, H: int, L1: int, L2: int, D: int, sm_scale: float = 1.0, options: "Options | None" = None) -> dict:
    """Kernel instance, launch count, grid, block and LDS bytes per stage, and the workspace parts, for a
    call with these sizes, softmax scale and options (None: fp16, no dropout)."""
    buf = ctypes.create_string_buffer(1024)
    check(load().fta_describe_plan_ex(B, H, L1, L2, D, float(sm_scale), ctypes.byref(options) if options is not None else None,
                                      buf, len(buf)))
    out = {}
    for line in buf.value.decode().strip().split("\n"):
        stage, rest = line.split(": ", 1)
        fields = rest.split(" ")
        d = {"kernel": fields[0]} if "=" not in fields[0] else {}
        d.update({k: (int(v) if v.lstrip("-").isdigit() else v) for k, v in (f.split("=") for f in fields if "=" in f)})
        out[stage] = d
    return out


def check(status: int) -> None:
    if status != 0:
        raise FtaError(status, strerror(status))


def t5(ptr: int, strides) -> Tensor5:
    return Tensor5(ptr, (ctypes.c_int64 * 4)(*[int(s) for s in strides[:4]]))


def t4(ptr: int, strides) -> Tensor4:
    return Tensor4(ptr, (ctypes.c_int64 * 3)(*[int(s) for s in strides[:3]]))
