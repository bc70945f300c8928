"""ctypes wrapper of the plain-C oracle (oracle/sma_oracle.c).  TEST INFRASTRUCTURE ONLY."""
import ctypes
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "libsma_oracle.so")
_lib = None


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB):
            subprocess.run(["make", "-C", HERE], check=True)
        lib = ctypes.CDLL(LIB)
        vp, ci = ctypes.c_void_p, ctypes.c_int
        lib.oracle_pack_mask.restype = ci
        lib.oracle_pack_mask.argtypes = [vp, vp, ci, ci, ci]
        lib.oracle_attn_fwd.restype = ci
        lib.oracle_attn_fwd.argtypes = [vp, vp, vp, vp, vp, vp, ci, ci, ci, ci, ctypes.c_float]
        _lib = lib
    return _lib


def pack_mask(mask: np.ndarray) -> np.ndarray:
    m = np.ascontiguousarray(np.asarray(mask).astype(np.uint8))
    B, H, N, _ = m.shape
    out = np.empty((B, H, N, (N + 31) // 32), dtype=np.uint32)
    rc = load().oracle_pack_mask(m.ctypes.data, out.ctypes.data, B, H, N)
    assert rc == 0
    return out.view(np.int32)


def attn_fwd(q, k, v, mask, scale):
    """float32 numpy inputs [B,H,N,D], bool mask -> (out float32, lse float32)."""
    q = np.ascontiguousarray(q, dtype=np.float32)
    k = np.ascontiguousarray(k, dtype=np.float32)
    v = np.ascontiguousarray(v, dtype=np.float32)
    m = np.ascontiguousarray(np.asarray(mask).astype(np.uint8))
    B, H, N, D = q.shape
    out = np.empty_like(q)
    lse = np.empty((B, H, N), dtype=np.float32)
    rc = load().oracle_attn_fwd(q.ctypes.data, k.ctypes.data, v.ctypes.data, m.ctypes.data,
                                out.ctypes.data, lse.ctypes.data, B, H, N, D, float(scale))
    assert rc == 0
    return out, lse
