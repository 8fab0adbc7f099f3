"""Format-valid Q4_K / Q6_K weight encoders for the tests (ctypes binding of kquant_encoders.c).

Test-input generators, not an oracle: weight blocks are inputs of the projection path, both sides of every parity
test consume the same blocks, and nothing here claims agreement with llama.cpp's offline quantizer.  Q8_0 weights
come from the oracle, whose quantizer the benchmark configuration defines completely.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "kquant_encoders.c")
LIB_PATH = os.path.join(HERE, "libkquant_encoders.so")
Q8_0, Q4_K, Q6_K = 8, 12, 14
ROW_BYTES = {Q4_K: 144, Q6_K: 210}

_lib = None


def build(force: bool = False) -> str:
    stale = (not os.path.exists(LIB_PATH)) or os.path.getmtime(LIB_PATH) < os.path.getmtime(SRC)
    if force or stale:
        subprocess.check_call(["gcc", "-O2", "-std=c11", "-fPIC", "-fopenmp", "-march=x86-64-v3", "-ffp-contract=off",
                               "-Wall", "-Wextra", "-shared", "-o", LIB_PATH, SRC, "-lm"])
    return LIB_PATH


def _load() -> C.CDLL:
    global _lib
    if _lib is None:
        build()
        L = C.CDLL(LIB_PATH)
        L.enc_quantize_rows.restype = C.c_int
        L.enc_quantize_rows.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_int]
        _lib = L
    return _lib


def encode(qtype: int, w: np.ndarray, nthreads: int = 8) -> np.ndarray:
    """float32 [N, K] -> uint8 [N, row_bytes] of GGUF blocks of `qtype`."""
    if qtype == Q8_0:
        from oracle import oracle
        return oracle.quantize(Q8_0, w, nthreads)
    w = np.ascontiguousarray(w, dtype=np.float32)
    n, k = w.shape
    if qtype not in ROW_BYTES or k % 256:
        raise ValueError("Q4_K / Q6_K need K a multiple of 256")
    out = np.zeros((n, k // 256 * ROW_BYTES[qtype]), dtype=np.uint8)
    if _load().enc_quantize_rows(qtype, w.ctypes.data, out.ctypes.data, k, n, nthreads) != 0:
        raise ValueError("encoder refused the shape")
    return out
