"""ctypes loader for the C oracle (oracle/cherryq_oracle.c).  Test infrastructure only."""
from __future__ import annotations

import ctypes
import subprocess
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
LIB = HERE / "libcherryq_oracle.so"


def build(force: bool = False) -> Path:
    if force or not LIB.exists() or LIB.stat().st_mtime < (HERE / "cherryq_oracle.c").stat().st_mtime:
        subprocess.check_call(["make", "-C", str(HERE), "-B", "libcherryq_oracle.so"],
                              stdout=subprocess.DEVNULL)
    return LIB


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = ctypes.CDLL(str(LIB))
        _lib.cherryq_oracle_h2f.restype = ctypes.c_float
        _lib.cherryq_oracle_h2f.argtypes = [ctypes.c_uint16]
        _lib.cherryq_oracle_f2h.restype = ctypes.c_uint16
        _lib.cherryq_oracle_f2h.argtypes = [ctypes.c_float]
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _c(a, dtype):
    a = np.ascontiguousarray(a)
    assert a.dtype == dtype, (a.dtype, dtype)
    return a


def threads() -> int:
    return int(lib().cherryq_oracle_threads())


def unpack(packed, w_bits, group_size, in_features):
    qw = _c(packed["qweight"], np.uint8)
    n = qw.shape[1]
    idx = _c(packed["cherry_indices"], np.int16)
    g = group_size if group_size != -1 else in_features
    dense = np.zeros((n, in_features), dtype=np.float16)
    rc = lib().cherryq_oracle_unpack(w_bits, _p(qw), _p(_c(packed["scales"], np.float16)),
                                     _p(_c(packed["cherry_weight"], np.float16)), _p(idx),
                                     in_features, n, idx.shape[0], g, _p(dense))
    assert rc == 0, rc
    return dense


def linear(x, dense, want_f64=False):
    x = _c(x, np.float16)
    dense = _c(dense, np.float16)
    b, k = x.shape
    n = dense.shape[0]
    y = np.zeros((b, n), dtype=np.float16)
    y64 = np.zeros((b, n), dtype=np.float64)
    rc = lib().cherryq_oracle_linear(_p(x), _p(dense), b, k, n, _p(y), _p(y64))
    assert rc == 0, rc
    return (y, y64) if want_f64 else y


def fused(x, packed, w_bits, group_size):
    x = _c(x, np.float16)
    b, k = x.shape
    qw = _c(packed["qweight"], np.uint8)
    n = qw.shape[1]
    idx = _c(packed["cherry_indices"], np.int16)
    g = group_size if group_size != -1 else k
    y = np.zeros((b, n), dtype=np.float64)
    rc = lib().cherryq_oracle_fused(w_bits, _p(x), _p(qw), _p(_c(packed["cherry_weight"], np.float16)),
                                    _p(idx), _p(_c(packed["scales"], np.float16)),
                                    b, k, n, idx.shape[0], g, _p(y))
    assert rc == 0, rc
    return y


def dequant_matmul(x, packed, w_bits, group_size, dense_scratch=None):
    """unpack() + linear(): the reference CPU path, as timed by the benchmark."""
    x = _c(x, np.float16)
    b, k = x.shape
    qw = _c(packed["qweight"], np.uint8)
    n = qw.shape[1]
    idx = _c(packed["cherry_indices"], np.int16)
    g = group_size if group_size != -1 else k
    if dense_scratch is None:
        dense_scratch = np.zeros((n, k), dtype=np.float16)
    y = np.zeros((b, n), dtype=np.float16)
    rc = lib().cherryq_oracle_dequant_matmul(
        w_bits, _p(x), _p(qw), _p(_c(packed["cherry_weight"], np.float16)), _p(idx),
        _p(_c(packed["scales"], np.float16)), b, k, n, idx.shape[0], g, _p(dense_scratch), _p(y))
    assert rc == 0, rc
    return y


def dequantize_normal(qweight, scales_f32, w_bits, height, cherry_size, group_size):
    qw = _c(qweight, np.uint8)
    s = _c(scales_f32, np.float32)
    n = qw.shape[1]
    out = np.zeros((height - cherry_size, n), dtype=np.float32)
    rc = lib().cherryq_oracle_dequantize_normal(w_bits, _p(qw), _p(s), _p(out), height, n,
                                                cherry_size, group_size)
    assert rc == 0, rc
    return out
