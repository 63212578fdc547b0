"""ctypes loader for the C restatement (oracle/gdn_oracle.c).  TEST INFRASTRUCTURE ONLY."""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libgdn_oracle.so")
_lib = None


def build():
    subprocess.run(["make", "-C", _HERE, "-B", "libgdn_oracle.so"], check=True, capture_output=True)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def to_bf16_bits(x):
    """float32 array of bf16-exact values -> uint16 bit patterns"""
    x = np.ascontiguousarray(x, dtype=np.float32)
    return (x.view(np.uint32) >> np.uint32(16)).astype(np.uint16)


def from_bf16_bits(b):
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)


def decode_step(proj, conv_pool, cw, A_log, dt_bias, ssm_pool, slots, pos, acc64=True, nthreads=1):
    """proj [B,8224], conv_pool [(S+1)*2,3,6144], cw [6144*4]: uint16 bf16 bits; ssm_pool [S+1,16,128,128] float32.
    Pools are updated in place.  Returns y [B,2048] uint16."""
    B = proj.shape[0]
    for a, dt in ((proj, np.uint16), (conv_pool, np.uint16), (cw, np.uint16), (ssm_pool, np.float32)):
        assert a.dtype == dt and a.flags.c_contiguous
    A_log = np.ascontiguousarray(A_log, dtype=np.float32)
    dt_bias = np.ascontiguousarray(dt_bias, dtype=np.float32)
    slots = np.ascontiguousarray(slots, dtype=np.int32)
    pos = np.ascontiguousarray(pos, dtype=np.int32)
    y = np.zeros((B, 2048), np.uint16)
    lib().gdn_oracle_decode_step(_p(proj), _p(conv_pool), _p(cw), _p(A_log), _p(dt_bias), _p(ssm_pool), _p(slots),
                                 _p(pos), _p(y), ctypes.c_int(B), ctypes.c_int(int(acc64)), ctypes.c_int(nthreads))
    return y


def recurrent(q, k, v, g, beta, state, acc64=True, nthreads=1):
    """q,k,v [B,T,16,128] uint16, g [B,T,16] float32, beta [B,T,16] uint16, state [B,16,128,128] float32 (in place)."""
    B, T = q.shape[:2]
    for a, dt in ((q, np.uint16), (k, np.uint16), (v, np.uint16), (beta, np.uint16), (g, np.float32), (state, np.float32)):
        assert a.dtype == dt and a.flags.c_contiguous
    y = np.zeros((B, T, 16, 128), np.uint16)
    lib().gdn_oracle_recurrent(_p(q), _p(k), _p(v), _p(g), _p(beta), _p(state), _p(y), ctypes.c_int(B), ctypes.c_int(T),
                               ctypes.c_int(int(acc64)), ctypes.c_int(nthreads))
    return y
