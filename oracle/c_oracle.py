"""ctypes front end of ``liboracle.so`` (the C restatement in dflash_oracle.c).

TEST INFRASTRUCTURE ONLY: used by tests/ (C oracle vs numpy oracle) and by the
``cpu_baseline`` leg of bench.py.  Arrays are float32, C-contiguous.
"""

from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


def build(force: bool = False) -> str:
    path = os.path.join(_HERE, "liboracle.so")
    if force or not os.path.exists(path):
        subprocess.check_call(["make", "-C", _HERE, "-B", "liboracle.so"])
    return path


def lib():
    global _LIB
    if _LIB is None:
        _LIB = C.CDLL(build())
        _LIB.oracle_num_threads.restype = C.c_int
        _LIB.oracle_match_acceptance_length.restype = C.c_int
    return _LIB


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _f32(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.float32)


def num_threads() -> int:
    return lib().oracle_num_threads()


def set_num_threads(n: int) -> None:
    lib().oracle_set_num_threads(C.c_int(n))


def tape_replay(tape, k, g, state, mask=None, *, variant="fused"):
    tape, k, g, state, mask = map(_f32, (tape, k, g, state, mask))
    B, T, Hv, Dv = tape.shape
    Hk, Dk = k.shape[2], k.shape[3]
    out = np.empty_like(state)
    fn = getattr(lib(), f"oracle_tape_replay_{variant}")
    fn(_p(tape), _p(k), _p(g), C.c_int(g.ndim), _p(state), _p(out), _p(mask),
       *map(C.c_int, (B, T, Hk, Hv, Dk, Dv)))
    return out


def gated_delta(q, k, v, g, beta, state, mask=None, *, variant="fused"):
    q, k, v, g, beta, state, mask = map(_f32, (q, k, v, g, beta, state, mask))
    B, T, Hk, Dk = q.shape
    Hv, Dv = v.shape[2], v.shape[3]
    y = np.empty((B, T, Hv, Dv), np.float32)
    tape = np.empty((B, T, Hv, Dv), np.float32)
    out = np.empty_like(state)
    fn = getattr(lib(), f"oracle_gated_delta_{variant}")
    fn(_p(q), _p(k), _p(v), _p(g), C.c_int(g.ndim), _p(beta), _p(state), _p(y), _p(out), _p(tape),
       _p(mask), *map(C.c_int, (B, T, Hk, Hv, Dk, Dv)))
    return y, out, tape


def sdpa_block_causal(q, k, v, scale):
    q, k, v = map(_f32, (q, k, v))
    B, Hq, M, D = q.shape
    Hk, N = k.shape[1], k.shape[2]
    out = np.empty_like(q)
    lse = np.empty((B, Hq, M), np.float32)
    lib().oracle_sdpa_block_causal(_p(q), _p(k), _p(v), C.c_float(scale), _p(out), _p(lse),
                                   *map(C.c_int, (B, Hq, Hk, M, N, D)))
    return out, lse


def match_acceptance_length(drafted, posterior) -> int:
    d = np.ascontiguousarray(drafted, dtype=np.uint32)
    p = np.ascontiguousarray(posterior, dtype=np.uint32)
    return lib().oracle_match_acceptance_length(_p(d), _p(p), C.c_int(d.shape[0]))
