"""ctypes front end of oracle/c/packed_interp.c.  Test infrastructure (see
oracle/__init__.py)."""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "c", "libdl_oracle.so")
_lib = None


def build():
    subprocess.run(["make", "-s", "-B", "-C", _HERE], check=True)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        i64p = np.ctypeslib.ndpointer(np.int64, flags="C_CONTIGUOUS")
        u8p = np.ctypeslib.ndpointer(np.uint8, flags="C_CONTIGUOUS")
        u64p = np.ctypeslib.ndpointer(np.uint64, flags="C_CONTIGUOUS")
        _lib.dl_oracle_net_eval.restype = ctypes.c_int
        _lib.dl_oracle_net_eval.argtypes = [
            u8p, ctypes.c_int64, ctypes.c_int64, ctypes.c_int, i64p, i64p, i64p, u8p, ctypes.c_int,
            np.ctypeslib.ndpointer(np.int32, flags="C_CONTIGUOUS"), ctypes.c_int]
        _lib.dl_oracle_eval_layer.restype = ctypes.c_int
        _lib.dl_oracle_eval_layer.argtypes = [u64p, u64p, ctypes.c_int64, ctypes.c_int64, i64p, i64p,
                                              u8p, ctypes.c_int]
    return _lib


def _cat(layers):
    widths = np.array([len(l[0]) for l in layers], dtype=np.int64)
    a = np.ascontiguousarray(np.concatenate([np.asarray(l[0], dtype=np.int64) for l in layers]))
    b = np.ascontiguousarray(np.concatenate([np.asarray(l[1], dtype=np.int64) for l in layers]))
    op = np.ascontiguousarray(np.concatenate([np.asarray(l[2]).astype(np.uint8) for l in layers]))
    return widths, a, b, op


def net_eval(x_bool, layers, k: int, threads: int = 1):
    """bool [B,F] -> int32 [B,k]."""
    x = np.ascontiguousarray(np.asarray(x_bool)).view(np.uint8) if np.asarray(x_bool).dtype == np.bool_ \
        else np.ascontiguousarray(np.asarray(x_bool, dtype=np.uint8))
    B, F = x.shape
    widths, a, b, op = _cat(layers)
    d = F
    for (la, lb, _), w in zip(layers, widths):
        assert min(np.min(la), np.min(lb)) >= 0 and max(np.max(la), np.max(lb)) < d
        d = int(w)
    out = np.zeros((B, k), dtype=np.int32)
    rc = lib().dl_oracle_net_eval(x, B, F, len(layers), widths, a, b, op, k, out, threads)
    if rc != 0:
        raise RuntimeError(f"dl_oracle_net_eval failed ({rc})")
    return out


def eval_layer(x_words, idx_a, idx_b, ops, threads: int = 1):
    """int64 [in,W] -> int64 [out,W]."""
    x = np.ascontiguousarray(x_words).view(np.uint64)
    a = np.ascontiguousarray(idx_a, dtype=np.int64)
    b = np.ascontiguousarray(idx_b, dtype=np.int64)
    op = np.ascontiguousarray(np.asarray(ops).astype(np.uint8))
    assert a.min() >= 0 and b.min() >= 0 and a.max() < x.shape[0] and b.max() < x.shape[0]
    y = np.empty((len(a), x.shape[1]), dtype=np.uint64)
    lib().dl_oracle_eval_layer(x, y, len(a), x.shape[1], a, b, op, threads)
    return y.view(np.int64)
