"""ctypes loader for the plain-C restatement ``conv_ref.c`` (TEST INFRASTRUCTURE ONLY)."""
import ctypes
import os
import subprocess

import numpy as np

_here = os.path.dirname(os.path.abspath(__file__))
_path = os.path.join(_here, '_build', 'libios_oracle.so')
_lib = None
_ACT = {'identity': 0, 'relu': 1, 'tanh': 2, 'sigmoid': 3}


def build():
    subprocess.run(['make', '-C', _here, '-s'], check=True)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_path):
            build()
        _lib = ctypes.cdll.LoadLibrary(_path)
    return _lib


def _ptr(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def conv2d(x, w, b, stride, padding, groups, act='identity'):
    x = np.ascontiguousarray(x, dtype=np.float32)
    w = np.ascontiguousarray(w, dtype=np.float32)
    b = np.ascontiguousarray(b, dtype=np.float32)
    n, ic, h, wd = x.shape
    oc, _, kh, kw = w.shape
    oh = 1 + (h - kh + 2 * padding[0]) // stride[0]
    ow = 1 + (wd - kw + 2 * padding[1]) // stride[1]
    y = np.empty((n, oc, oh, ow), dtype=np.float32)
    lib().oracle_conv2d(_ptr(x), _ptr(w), _ptr(b), _ptr(y), n, ic, h, wd, oc, kh, kw, stride[0], stride[1],
                        padding[0], padding[1], groups, _ACT[act])
    return y


def pool2d(x, pool_type, kernel, stride, padding):
    x = np.ascontiguousarray(x, dtype=np.float32)
    n, c, h, wd = x.shape
    if 'global' in pool_type:
        kernel, stride, padding = (h, wd), (1, 1), (0, 0)
    oh = 1 + (h - kernel[0] + 2 * padding[0]) // stride[0]
    ow = 1 + (wd - kernel[1] + 2 * padding[1]) // stride[1]
    y = np.empty((n, c, oh, ow), dtype=np.float32)
    lib().oracle_pool2d(_ptr(x), _ptr(y), n, c, h, wd, kernel[0], kernel[1], stride[0], stride[1],
                        padding[0], padding[1], 1 if 'max' in pool_type else 0)
    return y
