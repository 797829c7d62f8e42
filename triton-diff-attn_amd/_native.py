"""ctypes binding of libdiffattn.so (C ABI in include/diffattn.h).

torch is imported first on purpose: the library resolves the HIP runtime by soname, so it shares
the runtime (and therefore streams and device pointers) that torch has already loaded.
"""
import ctypes
import os

import torch  # noqa: F401  (must precede loading the library)

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libdiffattn.so")

ABI_VERSION = 7   # the version of include/diffattn.h this binding is written against

_lib = None

_vp = ctypes.c_void_p
_fp = ctypes.c_void_p  # float* passed as raw addresses


class Layout(ctypes.Structure):
    """diffattn_layout: element strides (batch, head, row) of q/k, v, y, dy and of the gradients of q/k and v
    (gradient strides left at zero mean dense)."""
    _fields_ = [(n, ctypes.c_longlong) for n in (
        "qk_b", "qk_h", "qk_n", "v_b", "v_h", "v_n", "y_b", "y_h", "y_n", "dy_b", "dy_h", "dy_n",
        "dqk_b", "dqk_h", "dqk_n", "dv_b", "dv_h", "dv_n")]


class Dropout(ctypes.Structure):
    """diffattn_dropout: drop probability and seed."""
    _fields_ = [("p", ctypes.c_float), ("seed", ctypes.c_ulonglong)]


_lp = ctypes.POINTER(Layout)
_dp = ctypes.POINTER(Dropout)

SYMBOLS = {
    "diffattn_abi_version": (ctypes.c_int, []),
    "diffattn_strerror": (ctypes.c_char_p, [ctypes.c_int]),
    "diffattn_forward": (ctypes.c_int, [_vp] * 5 + [_vp, _vp, _vp, _fp, _fp, _fp] + [ctypes.c_int] * 4
                         + [ctypes.c_float, ctypes.c_float, ctypes.c_int, _vp]),
    "diffattn_forward_padded": (ctypes.c_int, [_vp] * 5 + [_vp, _vp, _vp, _fp, _fp, _fp] + [ctypes.c_int] * 5
                                + [ctypes.c_float, ctypes.c_float, ctypes.c_int, _lp, _dp, _vp]),
    "diffattn_backward_workspace_bytes": (ctypes.c_size_t, [ctypes.c_int] * 5),
    "diffattn_backward": (ctypes.c_int, [_vp] * 5 + [_vp, _vp, _vp, _fp, _fp, _fp, _vp] + [_vp] * 6
                          + [_vp, ctypes.c_size_t] + [ctypes.c_int] * 4
                          + [ctypes.c_float, ctypes.c_float, ctypes.c_int, _vp]),
    "diffattn_backward_stages": (ctypes.c_int, [_vp] * 5 + [_vp, _vp, _vp, _fp, _fp, _fp, _vp] + [_vp] * 6
                                 + [_vp, ctypes.c_size_t] + [ctypes.c_int] * 5
                                 + [ctypes.c_float, ctypes.c_float, ctypes.c_int, ctypes.c_uint, _lp, _dp, _vp]),
    "diffattn_dropout_mask": (ctypes.c_int, [_vp] + [ctypes.c_int] * 4 + [_dp, _vp]),
    "diffattn_backward_static": (ctypes.c_int, [_vp] * 5 + [_vp, _vp, _vp, _fp, _fp, _fp, _vp] + [_vp] * 6
                                 + [ctypes.c_int] * 4 + [ctypes.c_float, ctypes.c_float, ctypes.c_int, _vp]),
}


class NativeLibraryMissing(RuntimeError):
    pass


def lib():
    """Returns the loaded library; raises if it has not been built (there is no fallback)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise NativeLibraryMissing(
                "libdiffattn.so is not built: run `python %s`" % os.path.join(_HERE, "build.py"))
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SYMBOLS.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        if handle.diffattn_abi_version() != ABI_VERSION:
            raise NativeLibraryMissing(
                "libdiffattn.so has ABI version %d, this binding needs %d: rebuild it with `python %s`"
                % (handle.diffattn_abi_version(), ABI_VERSION, os.path.join(_HERE, "build.py")))
        _lib = handle
    return _lib


def check(code):
    if code != 0:
        raise RuntimeError("libdiffattn: %s (code %d)" % (lib().diffattn_strerror(code).decode(), code))
