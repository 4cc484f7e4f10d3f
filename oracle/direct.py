"""ctypes access to the brute-force C convolutions (oracle/conv_direct.c) --
TEST INFRASTRUCTURE, NOT PRODUCT CODE."""
import ctypes
import os

import numpy as np

from . import ops as O
from .build_oracle import LIB, build

_lib = None


def _load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB):
            build()
        _lib = ctypes.CDLL(LIB)
    return _lib


def _ptr(a):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_double))


def _geometry(x_shape, w_shape, padding, u, v):
    N, C, H, W = x_shape
    K, _, R, S = w_shape
    ph, pw = O.conv_pad(R, padding), O.conv_pad(S, padding)
    P, Q = O.conv_out_extent(H, R, ph, u), O.conv_out_extent(W, S, pw, v)
    return (N, C, H, W, K, R, S, P, Q, ph, pw, u, v)


def forward(x, w, padding, u, v):
    g = _geometry(x.shape, w.shape, padding, u, v)
    x = np.ascontiguousarray(x, np.float64)
    w = np.ascontiguousarray(w, np.float64)
    y = np.empty((g[0], g[4], g[7], g[8]), np.float64)
    _load().conv_direct_forward(_ptr(x), _ptr(w), _ptr(y), *[ctypes.c_int(i) for i in g])
    return y


def backward_data(dy, w, x_shape, padding, u, v):
    g = _geometry(x_shape, w.shape, padding, u, v)
    dy = np.ascontiguousarray(dy, np.float64)
    w = np.ascontiguousarray(w, np.float64)
    dx = np.empty(x_shape, np.float64)
    _load().conv_direct_backward_data(_ptr(dy), _ptr(w), _ptr(dx), *[ctypes.c_int(i) for i in g])
    return dx


def backward_filter(x, dy, w_shape, padding, u, v):
    g = _geometry(x.shape, w_shape, padding, u, v)
    x = np.ascontiguousarray(x, np.float64)
    dy = np.ascontiguousarray(dy, np.float64)
    dw = np.empty(w_shape, np.float64)
    _load().conv_direct_backward_filter(_ptr(x), _ptr(dy), _ptr(dw), *[ctypes.c_int(i) for i in g])
    return dw
