"""ctypes loader of oracle/libqtip_oracle.so (TEST INFRASTRUCTURE ONLY)."""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libqtip_oracle.so")
_lib = None


def build():
    subprocess.run(["make", "-C", _HERE, "-s"], check=True)
    return _SO


def _load():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
        _lib.qtip_oracle_decode.restype = ctypes.c_int
        _lib.qtip_oracle_matvec.restype = ctypes.c_int
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def decode(packed, tlut, m, k, K):
    pk = np.ascontiguousarray(packed).reshape(-1).view(np.uint8)
    tl = np.ascontiguousarray(tlut, dtype=np.float16).reshape(-1).view(np.uint16)
    assert pk.size * 8 == m * k * K and tl.size == 1024
    out = np.empty((m, k), dtype=np.uint16)
    rc = _load().qtip_oracle_decode(_p(pk), _p(tl), m, k, K, _p(out))
    assert rc == 0
    return out.view(np.float16)


def matvec(packed, x, tlut, m, k, K):
    pk = np.ascontiguousarray(packed).reshape(-1).view(np.uint8)
    tl = np.ascontiguousarray(tlut, dtype=np.float16).reshape(-1).view(np.uint16)
    xv = np.ascontiguousarray(x, dtype=np.float16).reshape(-1).view(np.uint16)
    assert pk.size * 8 == m * k * K and tl.size == 1024 and xv.size == k
    out = np.empty(m, dtype=np.float64)
    rc = _load().qtip_oracle_matvec(_p(pk), _p(tl), _p(xv), m, k, K, _p(out))
    assert rc == 0
    return out
