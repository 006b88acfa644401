"""ctypes loader for the plain-C oracle (oracle/colsum_ref.c).  Test infrastructure."""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


def build() -> str:
    subprocess.run(["make", "-s", "-C", _HERE], check=True)
    return os.path.join(_HERE, "libcolsum_ref.so")


def _lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "libcolsum_ref.so")
        if not os.path.exists(path):
            build()
        lib = ctypes.CDLL(path)
        lib.colsum_ref.restype = ctypes.c_int
        lib.colsum_ref.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p] + [ctypes.c_int] * 5 + [
            ctypes.c_double, ctypes.c_int, ctypes.c_int]
        lib.colsum_ref_ext.restype = ctypes.c_int
        lib.colsum_ref_ext.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p] + [ctypes.c_int] * 6 + [
            ctypes.c_double, ctypes.c_int, ctypes.c_int, ctypes.c_long]
        _LIB = lib
    return _LIB


def colsum_ref(q, k, scale=None, is_causal=False, cls_len=None) -> np.ndarray:
    """float64 (B, S_k) column means from the C triple loop; q, k are array-likes."""
    q = np.ascontiguousarray(np.asarray(q, dtype=np.float32))
    k = np.ascontiguousarray(np.asarray(k, dtype=np.float32))
    b, h, sq, d = q.shape
    sk = k.shape[2]
    if scale is None:
        scale = 1.0 / (d ** 0.5)
    out = np.empty((b, sk), dtype=np.float64)
    rc = _lib().colsum_ref(q.ctypes.data, k.ctypes.data, out.ctypes.data, b, h, sq, sk, d,
                           float(scale), int(bool(is_causal)), int(cls_len) if cls_len else 0)
    if rc != 0:
        raise RuntimeError(f"colsum_ref failed with code {rc}")
    return out


def colsum_ref_ext(q, k, scale=None, is_causal=False, cls_len=None, k_past=None) -> np.ndarray:
    """float64 (B, S_k) column means for grouped key heads / batched causal / causal cls_len / explicit k_past."""
    q = np.ascontiguousarray(np.asarray(q, dtype=np.float32))
    k = np.ascontiguousarray(np.asarray(k, dtype=np.float32))
    b, hq, sq, d = q.shape
    hk, sk = k.shape[1], k.shape[2]
    if scale is None:
        scale = 1.0 / (d ** 0.5)
    out = np.empty((b, sk), dtype=np.float64)
    rc = _lib().colsum_ref_ext(q.ctypes.data, k.ctypes.data, out.ctypes.data, b, hq, hk, sq, sk, d, float(scale),
                               int(bool(is_causal)), int(cls_len) if cls_len else 0, -1 if k_past is None else int(k_past))
    if rc != 0:
        raise RuntimeError(f"colsum_ref_ext failed with code {rc}")
    return out
