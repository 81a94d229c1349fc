"""ctypes access to the oracle's C ranker (``oracle/ranker.c``) and to the
independent textbook evaluator (``oracle/std_eval.c``).  TEST INFRASTRUCTURE
ONLY.  Build with ``make -C oracle`` (``__graft_entry__.build()`` does)."""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "libp2oracle.so")
_lib = None


def build() -> str:
    subprocess.run(["make", "-C", _HERE], check=True, capture_output=True)
    return _SO


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
        _lib.p2o_rank_planes.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p]
        _lib.p2o_rank_cards.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_void_p]
        _lib.p2o_hist_all7.argtypes = [ctypes.c_void_p]
        _lib.p2o_std_best5.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p]
    return _lib


def rank_planes(planes: np.ndarray) -> np.ndarray:
    """[..., 4, 13] (or [..., 52]) 0/1 planes -> packed int32, rules.py semantics."""
    p = np.ascontiguousarray(np.asarray(planes).astype(np.uint8))
    lead = p.shape[:-2] if p.shape[-1] == 13 else p.shape[:-1]
    p = p.reshape(-1, 52)
    out = np.empty(p.shape[0], dtype=np.int32)
    lib().p2o_rank_planes(p.ctypes.data, p.shape[0], out.ctypes.data)
    return out.reshape(lead)


def rank_cards(cards: np.ndarray) -> np.ndarray:
    """[..., K] card ids -> packed int32, rules_triton.py card-id semantics."""
    c = np.ascontiguousarray(np.asarray(cards).astype(np.int16))
    lead = c.shape[:-1]
    k = c.shape[-1]
    c = c.reshape(-1, k)
    out = np.empty(c.shape[0], dtype=np.int32)
    lib().p2o_rank_cards(c.ctypes.data, c.shape[0], k, out.ctypes.data)
    return out.reshape(lead)


def hist_all7() -> np.ndarray:
    """Category histogram over all C(52,7) hands, index = category 0..9."""
    h = np.zeros(10, dtype=np.uint64)
    lib().p2o_hist_all7(h.ctypes.data)
    return h


def std_best5(cards7: np.ndarray) -> np.ndarray:
    """Textbook best-5-of-7 key (uint32, bigger = stronger) for [N,7] ids."""
    c = np.ascontiguousarray(np.asarray(cards7).astype(np.int16)).reshape(-1, 7)
    out = np.empty(c.shape[0], dtype=np.uint32)
    lib().p2o_std_best5(c.ctypes.data, c.shape[0], out.ctypes.data)
    return out
