"""numpy front-end to the plain-C oracle (oracle/cottention_oracle.c) -- TEST INFRASTRUCTURE ONLY.

Inputs may carry any leading (batch, head, ...) dimensions; they are flattened to (BH, N, D),
upcast to float64 (exact for fp32/fp16/bf16 values) and the result is returned in float64 with
the caller's leading shape.  Reference lines each routine follows are cited in the C file.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "_build", "libcottention_oracle.so")
_lib = None


def build(force=False):
    """Compile the C oracle with gcc (a few hundred ms)."""
    src = os.path.join(_HERE, "cottention_oracle.c")
    if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src):
        subprocess.run(["make", "-s", "-B", "-C", _HERE], check=True)
    return _LIB_PATH


def _load():
    global _lib
    if _lib is None:
        build()
        lib = ctypes.CDLL(_LIB_PATH)
        dp, lg, it = ctypes.POINTER(ctypes.c_double), ctypes.c_long, ctypes.c_int
        lib.cott_oracle_causal_loop.argtypes = [dp, dp, dp, dp, lg, lg, lg, lg, it]
        lib.cott_oracle_causal_masked.argtypes = [dp, dp, dp, dp, lg, lg, lg, lg, it]
        lib.cott_oracle_causal_bwd.argtypes = [dp] * 7 + [lg] * 4
        lib.cott_oracle_noncausal.argtypes = [dp, dp, dp, dp, lg, lg, lg, lg]
        lib.cott_oracle_noncausal_bwd.argtypes = [dp] * 7 + [lg] * 4
        lib.cott_oracle_decode_step.argtypes = [dp] * 5 + [lg] * 3
        for name in ("causal_loop", "causal_masked", "causal_bwd", "noncausal", "noncausal_bwd", "decode_step"):
            getattr(lib, "cott_oracle_" + name).restype = None
        _lib = lib
    return _lib


def _f64(x):
    if hasattr(x, "detach"):  # torch tensor (any float dtype, CPU)
        x = x.detach().to("cpu").double().numpy()
    return np.ascontiguousarray(np.asarray(x, dtype=np.float64))


def _ptr(a):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_double))


def _flat3(a, b, c):
    a, b, c = _f64(a), _f64(b), _f64(c)
    lead, n, di = a.shape[:-2], a.shape[-2], a.shape[-1]
    dj = c.shape[-1]
    if b.shape != a.shape or c.shape[:-1] != a.shape[:-1]:
        raise ValueError(f"oracle: inconsistent shapes {a.shape} {b.shape} {c.shape}")
    bh = int(np.prod(lead)) if lead else 1
    return a, b, c, lead, bh, n, di, dj


def causal(A, B, C, reversed=False):
    """out[s,j] = sum_i A[s,i] sum_{s'<=s (>=s if reversed)} B[s',i] C[s',j]  (recurrent-loop form)."""
    a, b, c, lead, bh, n, di, dj = _flat3(A, B, C)
    out = np.empty(lead + (n, dj), dtype=np.float64)
    _load().cott_oracle_causal_loop(_ptr(a), _ptr(b), _ptr(c), _ptr(out), bh, n, di, dj, int(bool(reversed)))
    return out


def causal_masked(A, B, C, reversed=False):
    """Same quantity by the masked quadratic form ((A B^T) o tril) C; O(N^2), small inputs."""
    a, b, c, lead, bh, n, di, dj = _flat3(A, B, C)
    out = np.empty(lead + (n, dj), dtype=np.float64)
    _load().cott_oracle_causal_masked(_ptr(a), _ptr(b), _ptr(c), _ptr(out), bh, n, di, dj, int(bool(reversed)))
    return out


def _bwd(fn, Q, K, V, dO):
    q, k, v, lead, bh, n, dk, dv = _flat3(Q, K, V)
    g = _f64(dO)
    if g.shape != v.shape:
        raise ValueError(f"oracle: dO shape {g.shape} != V shape {v.shape}")
    dq, dk_, dv_ = np.empty_like(q), np.empty_like(k), np.empty_like(v)
    fn(_ptr(q), _ptr(k), _ptr(v), _ptr(g), _ptr(dq), _ptr(dk_), _ptr(dv_), bh, n, dk, dv)
    return dq, dk_, dv_


def causal_bwd(Q, K, V, dO):
    """(dQ, dK, dV) of O = causal(Q, K, V) contracted with dO."""
    return _bwd(_load().cott_oracle_causal_bwd, Q, K, V, dO)


def noncausal(A, B, C):
    """out = A (B^T C)."""
    a, b, c, lead, bh, n, di, dj = _flat3(A, B, C)
    out = np.empty(lead + (n, dj), dtype=np.float64)
    _load().cott_oracle_noncausal(_ptr(a), _ptr(b), _ptr(c), _ptr(out), bh, n, di, dj)
    return out


def noncausal_bwd(Q, K, V, dO):
    """(dQ, dK, dV) of O = Q (K^T V) contracted with dO."""
    return _bwd(_load().cott_oracle_noncausal_bwd, Q, K, V, dO)


def decode_step(S, q, k, v):
    """In-place on the float64 state S (..., Dk, Dv): S += k v^T ; returns o = q S (updated S)."""
    if not (isinstance(S, np.ndarray) and S.dtype == np.float64 and S.flags.c_contiguous):
        raise ValueError("oracle.decode_step needs a C-contiguous float64 numpy state (updated in place)")
    q, k, v = _f64(q), _f64(k), _f64(v)
    dk, dv = S.shape[-2], S.shape[-1]
    bh = int(np.prod(S.shape[:-2])) if S.ndim > 2 else 1
    if q.shape[-1] != dk or k.shape != q.shape or v.shape[-1] != dv or q.size != bh * dk or v.size != bh * dv:
        raise ValueError("oracle.decode_step: inconsistent shapes")
    o = np.empty(v.shape, dtype=np.float64)
    _load().cott_oracle_decode_step(_ptr(S), _ptr(q), _ptr(k), _ptr(v), _ptr(o), bh, dk, dv)
    return o
