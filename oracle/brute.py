"""ctypes binding of oracle/brute.c (fp64 loops).  TEST INFRASTRUCTURE ONLY."""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


def build():
    subprocess.run(["make", "-C", _HERE, "libbrute.so"], check=True, capture_output=True)


def _lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "libbrute.so")
        if not os.path.exists(path):
            build()
        _LIB = ctypes.CDLL(path)
    return _LIB


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _c(x):
    return np.ascontiguousarray(np.asarray(x, dtype=np.float32))


def attention_fwd(q, k, v, scale, causal=False):
    q, k, v = _c(q), _c(k), _c(v)
    bh = int(np.prod(q.shape[:-2]))
    sq, kd = q.shape[-2:]
    sk, d = v.shape[-2:]
    o = np.empty(q.shape[:-1] + (d,), dtype=np.float32)
    _lib().brute_attention_fwd(_p(q), _p(k), _p(v), _p(o), bh, sq, sk, kd, d, ctypes.c_double(scale), int(causal))
    return o


def retnet_fwd(q, k, v, mask):
    q, k, v, mask = _c(q), _c(k), _c(v), _c(mask)
    bh = int(np.prod(q.shape[:-2]))
    sq, kd = q.shape[-2:]
    sk, d = v.shape[-2:]
    h = mask.shape[0]
    o = np.empty(q.shape[:-1] + (d,), dtype=np.float32)
    r = np.empty(q.shape[:-1], dtype=np.float32)
    _lib().brute_retnet_fwd(_p(q), _p(k), _p(v), _p(mask), _p(o), _p(r), bh, h, sq, sk, kd, d)
    return o, r


def retnet_bwd(q, k, v, mask, do):
    q, k, v, mask, do = _c(q), _c(k), _c(v), _c(mask), _c(do)
    bh = int(np.prod(q.shape[:-2]))
    sq, kd = q.shape[-2:]
    sk, d = v.shape[-2:]
    h = mask.shape[0]
    dq, dk, dv = np.empty_like(q), np.empty_like(k), np.empty_like(v)
    _lib().brute_retnet_bwd(_p(q), _p(k), _p(v), _p(mask), _p(do), _p(dq), _p(dk), _p(dv), bh, h, sq, sk, kd, d)
    return dq, dk, dv


def retnet_recurrent(q, k, v, decay, block_kdim=None):
    """q, k [..., kdim, L], v [..., vdim, L], decay [H, L] -> out [..., vdim, L] (fp64 recurrence, fp32 result)."""
    q, k, v, decay = _c(q), _c(k), _c(v), _c(decay)
    bh = int(np.prod(q.shape[:-2]))
    kdim, l = q.shape[-2:]
    vdim = v.shape[-2]
    out = np.empty(v.shape, dtype=np.float32)
    _lib().brute_retnet_recurrent(_p(q), _p(k), _p(v), _p(decay), _p(out), bh, decay.shape[0], kdim, vdim, l,
                                  int(block_kdim or kdim))
    return out
