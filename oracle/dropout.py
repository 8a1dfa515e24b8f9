"""Seeded dropout keep-mask oracle (test infrastructure): ctypes front end of dropout_oracle.c.

The mask stream is the build's own definition (Philox4x32-10, sixteen bits per element, integer
compare), not the reference's Triton stream (dropout.py:49-50): the reference's stream could only
be reproduced by running Triton on a GPU, and nothing downstream depends on which Bernoulli
stream is drawn.  What is pinned here is that the device kernel implements exactly this
definition, and that the definition is the published Philox4x32-10.
"""

from __future__ import annotations

import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_lib = None


def _load():
    global _lib
    if _lib is None:
        path = os.path.join(_HERE, "libdropout_oracle.so")
        if not os.path.exists(path):
            raise RuntimeError(f"{path} missing: run `make -C oracle`")
        l = ctypes.CDLL(path)
        l.philox4x32_10_ref.argtypes = [ctypes.c_void_p] * 3
        l.keep_threshold_ref.argtypes = [ctypes.c_float]
        l.keep_threshold_ref.restype = ctypes.c_uint32
        l.keep_mask_ref.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p, ctypes.c_uint64]
        _lib = l
    return _lib


def philox4x32_10(counter, key) -> np.ndarray:
    """counter: 4 uint32, key: 2 uint32 -> 4 uint32 (dropout_oracle.c:philox4x32_10_ref)."""
    c = np.ascontiguousarray(counter, dtype=np.uint32)
    k = np.ascontiguousarray(key, dtype=np.uint32)
    out = np.empty(4, dtype=np.uint32)
    _load().philox4x32_10_ref(c.ctypes.data, k.ctypes.data, out.ctypes.data)
    return out


def keep_threshold(p: float) -> int:
    return int(_load().keep_threshold_ref(ctypes.c_float(p)))


def keep_mask(M: int, K: int, p, seed: int) -> np.ndarray:
    """uint8 [M, K]; ``p`` is a float or one value per row."""
    row_p = np.ascontiguousarray(np.broadcast_to(np.asarray(p, dtype=np.float32), (M,)))
    out = np.empty((M, K), dtype=np.uint8)
    _load().keep_mask_ref(out.ctypes.data, M, K, row_p.ctypes.data, ctypes.c_uint64(seed & 0xFFFFFFFFFFFFFFFF))
    return out
