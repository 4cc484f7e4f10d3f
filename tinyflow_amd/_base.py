"""Loader of libc_runtime_api.so and small ctypes helpers.

Counterpart of the reference ``pycode/tinyflow/_base.py:10-57``: the library is
opened once with ``RTLD_GLOBAL`` at import and no argtypes are declared, so
calls marshal exactly as they do from the reference binding.
"""
import ctypes
import os

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("TINYFLOW_LIB", os.path.join(_PKG_DIR, "lib", "libc_runtime_api.so"))


def _load_lib():
    if not os.path.exists(LIB_PATH):
        raise OSError(
            "%s is missing: build it with `python -m tinyflow_amd.build` "
            "(there is no CPU fallback for the kernels)" % LIB_PATH)
    return ctypes.CDLL(LIB_PATH, ctypes.RTLD_GLOBAL)


_LIB = _load_lib()


def check_call(ret):
    """Every C entry point returns 0 on success."""
    if ret != 0:
        raise RuntimeError("libc_runtime_api call failed with status %d" % ret)


def c_array(ctype, values):
    """ctypes array holding ``values``."""
    return (ctype * len(values))(*values)
