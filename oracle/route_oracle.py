"""ctypes binding of oracle/route_oracle.c (test infrastructure; see that file's header)."""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "libroute_oracle.so")
_lib = None
_I32P = ctypes.POINTER(ctypes.c_int32)


def _p(a):
    return a.ctypes.data_as(_I32P)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            raise RuntimeError(f"{_SO} is not built: run `make -C oracle` (or __graft_entry__.build())")
        _lib = ctypes.CDLL(_SO)
    return _lib


def token_count(routing, num_experts, pad=1):
    r = np.ascontiguousarray(routing, dtype=np.int32)
    counts = np.zeros(num_experts, np.int32)
    expanded = np.zeros(num_experts + 1, np.int32)
    rc = lib().oracle_token_count(_p(r), int(r.size), int(num_experts), int(pad), _p(counts), _p(expanded))
    if rc:
        raise ValueError(f"oracle_token_count rc={rc}")
    return counts, expanded


def token_assign(routing, num_experts, expanded):
    r = np.ascontiguousarray(routing, dtype=np.int32)
    ex = np.ascontiguousarray(expanded, dtype=np.int32)
    P = int(ex[num_experts])
    tok = np.zeros(max(P, 1), np.int32)
    exp = np.zeros(max(P, 1), np.int32)
    rc = lib().oracle_token_assign(_p(r), int(r.size), int(num_experts), _p(ex), _p(tok), _p(exp))
    if rc:
        raise ValueError(f"oracle_token_assign rc={rc}")
    return tok[:P], exp[:P]


def route_build(routing, num_experts):
    r = np.ascontiguousarray(routing, dtype=np.int32)
    T, k = r.shape
    counts = np.zeros((k, num_experts), np.int32)
    offsets = np.zeros((k, num_experts + 1), np.int32)
    token_ids = np.zeros((k, max(T, 1)), np.int32)
    rc = lib().oracle_route_build(_p(r), int(T), int(k), int(num_experts), _p(counts), _p(offsets), _p(token_ids))
    if rc:
        raise ValueError(f"oracle_route_build rc={rc}")
    return counts, offsets, token_ids[:, :T]
