"""ctypes binding of the timing diagnostics library (include/msnh_hip_diag.h, msnhnet_amd/lib/libmsnh_diag.so).

Measurement only: bench.py's --conv-shape mode uses it for the table of timing switches; nothing in the product path loads it."""
import ctypes
import os

from . import hipabi

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libmsnh_diag.so")
SYMBOLS = ["msnh_hip_diag_patch8", "msnh_hip_diag_patch8_switches", "msnh_hip_diag_empty_launch"]
SWITCH_NAMES = {1: "main-loop loads", 2: "LDS fragment reads", 4: "main-loop barrier", 8: "MFMAs", 16: "epilogue", 32: "prologue loads"}
_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is not built: run python -m msnhnet_amd.build")
        hipabi.lib()                      # the kernel library first: the diagnostics link against it
        L = ctypes.CDLL(LIB_PATH)
        vp, ci = ctypes.c_void_p, ctypes.c_int
        L.msnh_hip_diag_patch8.argtypes = [ci, ci, ci, ci, ci, ci, ci, vp, vp, vp, vp, vp, vp, vp]
        L.msnh_hip_diag_patch8_switches.argtypes = [ctypes.POINTER(ci), ci]
        L.msnh_hip_diag_empty_launch.argtypes = [ci, ci, vp]
        for n in SYMBOLS:
            getattr(L, n).restype = ci
        _lib = L
    return _lib


def switches():
    buf = (ctypes.c_int * 64)()
    n = lib().msnh_hip_diag_patch8_switches(buf, 64)
    return [buf[i] for i in range(n)]


def describe(sw):
    """what a switch combination leaves out, in words"""
    off = [name for bit, name in SWITCH_NAMES.items() if sw & bit]
    text = "complete" if not off else "without " + ", ".join(off)
    return text + (" (clocks read)" if sw & 64 else "")
