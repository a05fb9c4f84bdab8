"""ctypes binding of oracle/libssd_oracle.so (plain-C oracle).  TEST INFRASTRUCTURE ONLY."""
import ctypes
import os
import subprocess

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libssd_oracle.so")
_lib = None


def build(force=False):
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(os.path.join(_HERE, "ssd_oracle.c")):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libssd_oracle.so"], stdout=subprocess.DEVNULL)
    return _SO


def lib():
    global _lib
    if _lib is None:
        _lib = ctypes.CDLL(build())
    return _lib


def _f32(t):
    return None if t is None else np.ascontiguousarray(t.detach().float().numpy())


def _i32(t):
    return None if t is None else np.ascontiguousarray(t.detach().to(torch.int32).numpy())


def _p(a, ty=ctypes.c_float):
    return None if a is None else a.ctypes.data_as(ctypes.POINTER(ty))


def chunk_state(B, x, dt, dA_cumsum, seq_idx=None, clamp=True):
    b, L, H, P = x.shape
    G, N = B.shape[2], B.shape[3]
    C, Q = dt.shape[2], dt.shape[3]
    xa, Ba, dta, csa, sa = _f32(x), _f32(B), _f32(dt), _f32(dA_cumsum), _i32(seq_idx)
    out = np.empty((b, C, H, P, N), dtype=np.float32)
    rc = lib().ssd_oracle_chunk_state(_p(xa), _p(Ba), _p(dta), _p(csa), _p(sa, ctypes.c_int32), _p(out),
                                      b, L, H, P, N, G, Q, int(clamp))
    assert rc == 0, rc
    return torch.from_numpy(out)


def state_passing(states, dA_chunk, initial_states=None, seq_idx=None, chunk_size=0):
    b, C, H, dim = states.shape
    L = 0 if seq_idx is None else seq_idx.shape[-1]
    sa, da, ia, qa = _f32(states), _f32(dA_chunk), _f32(initial_states), _i32(seq_idx)
    out = np.empty((b, C, H, dim), dtype=np.float32)
    fin = np.empty((b, H, dim), dtype=np.float32)
    rc = lib().ssd_oracle_state_passing(_p(sa), _p(da), _p(ia), _p(qa, ctypes.c_int32), _p(out), _p(fin),
                                        b, C, H, dim, L, chunk_size or 0)
    assert rc == 0, rc
    return torch.from_numpy(out), torch.from_numpy(fin)


def token_recurrence(x, B, dt_tok, A, chunk_size, initial_states=None, seq_idx=None):
    b, L, H, P = x.shape
    G, N = B.shape[2], B.shape[3]
    C = (L + chunk_size - 1) // chunk_size
    xa, Ba, dta, Aa, ia, qa = _f32(x), _f32(B), _f32(dt_tok), _f32(A), _f32(initial_states), _i32(seq_idx)
    out = np.empty((b, C, H, P, N), dtype=np.float64)
    fin = np.empty((b, H, P, N), dtype=np.float64)
    rc = lib().ssd_oracle_token_recurrence(_p(xa), _p(Ba), _p(dta), _p(Aa), _p(ia), _p(qa, ctypes.c_int32),
                                           _p(out, ctypes.c_double), _p(fin, ctypes.c_double),
                                           b, L, H, P, N, G, chunk_size)
    assert rc == 0, rc
    return torch.from_numpy(out), torch.from_numpy(fin)
