"""ctypes loader for the C leg of the CPU oracle (oracle/attn_oracle.c).  TEST INFRASTRUCTURE ONLY."""
import ctypes
import os
import subprocess
import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


def build():
    subprocess.check_call(["make", "-s", "-C", _HERE, "-B"])


def lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "libattn_oracle.so")
        if not os.path.exists(path):
            build()
        L = ctypes.CDLL(path)
        L.pa_oracle_attention.restype = ctypes.c_int
        L.pa_oracle_attention.argtypes = [ctypes.c_void_p, ctypes.c_long, ctypes.c_void_p, ctypes.c_void_p,
                                          ctypes.c_int, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                          ctypes.c_int, ctypes.c_long, ctypes.c_void_p, ctypes.c_long, ctypes.c_void_p]
        L.pa_oracle_attention_ref_loops.restype = ctypes.c_int
        L.pa_oracle_attention_ref_loops.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_long,
                                                    ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
        _LIB = L
    return _LIB


def attention(q, k16, v16, base_pos, gate=None, rows=None):
    """Same contract as attn_oracle.attention (f64 result [n_out, nH, hd]); multi-threaded C."""
    q = np.ascontiguousarray(q, dtype=np.float32)
    n, nH, hd = q.shape
    k16 = np.ascontiguousarray(k16, dtype=np.uint16)
    v16 = np.ascontiguousarray(v16, dtype=np.uint16)
    nKV = k16.shape[1]
    assert k16.shape[0] >= base_pos + n and v16.shape == k16.shape
    sel = None if rows is None else np.ascontiguousarray(list(rows), dtype=np.int32)
    n_out = n if sel is None else len(sel)
    out = np.zeros((n_out, nH, hd), dtype=np.float64)
    g = None if gate is None else np.ascontiguousarray(gate, dtype=np.float32).reshape(n, nH * hd)
    rc = lib().pa_oracle_attention(q.ctypes.data, nH * hd, k16.ctypes.data, v16.ctypes.data, n,
                                   None if sel is None else sel.ctypes.data, n_out, nH, nKV, hd, base_pos,
                                   None if g is None else g.ctypes.data, nH * hd, out.ctypes.data)
    if rc != 0:
        raise RuntimeError("pa_oracle_attention failed")
    return out
