"""ctypes binding of the CPU oracle (libqproj_oracle.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the
cpu_baseline leg of the benchmark.  The product package never imports it.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libqproj_oracle.so")

TYPE_Q8_0, TYPE_Q4_K, TYPE_Q6_K = 8, 12, 14
ACT_GGML, ACT_F64, ACT_Q8X32 = 0, 1, 2
TYPE_NAMES = {TYPE_Q8_0: "q8_0", TYPE_Q4_K: "q4_K", TYPE_Q6_K: "q6_K"}
BLOCK_BYTES = {TYPE_Q8_0: 34, TYPE_Q4_K: 144, TYPE_Q6_K: 210}
BLOCK_ELEMS = {TYPE_Q8_0: 32, TYPE_Q4_K: 256, TYPE_Q6_K: 256}


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (no GPU needed)."""
    src = os.path.join(HERE, "qproj_oracle.c")
    stale = (not os.path.exists(LIB_PATH)) or os.path.getmtime(LIB_PATH) < os.path.getmtime(src)
    if force or stale:
        subprocess.check_call(["make", "-C", HERE, "-B", "libqproj_oracle.so"],
                              stdout=subprocess.DEVNULL)
    return LIB_PATH


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        L = C.CDLL(LIB_PATH)
        vp, i64, i32, f32p = C.c_void_p, C.c_int64, C.c_int, C.c_void_p
        L.orc_sizeof_block.restype = C.c_size_t
        L.orc_sizeof_block.argtypes = [i32]
        L.orc_row_bytes.restype = C.c_size_t
        L.orc_row_bytes.argtypes = [i32, i64]
        L.orc_fp16_to_fp32.restype = C.c_float
        L.orc_fp16_to_fp32.argtypes = [C.c_uint16]
        L.orc_fp16_to_fp32_f16c.restype = C.c_float
        L.orc_fp16_to_fp32_f16c.argtypes = [C.c_uint16]
        L.orc_fp32_to_fp16.restype = C.c_uint16
        L.orc_fp32_to_fp16.argtypes = [C.c_float]
        L.orc_fp32_to_fp16_f16c.restype = C.c_uint16
        L.orc_fp32_to_fp16_f16c.argtypes = [C.c_float]
        L.orc_get_scale_min_k4.argtypes = [i32, vp, vp, vp]
        L.orc_pack_scale_min_k4.argtypes = [vp, vp, vp]
        L.orc_dequantize_row.argtypes = [i32, vp, f32p, i64]
        L.orc_quantize_rows.restype = i32
        L.orc_quantize_rows.argtypes = [i32, f32p, vp, i64, i64, i32]
        L.orc_quantize_row_q8_0.argtypes = [f32p, vp, i64]
        L.orc_quantize_row_q8_K.argtypes = [f32p, vp, i64]
        L.orc_quantize_row_q8x32.argtypes = [f32p, vp, i64]
        for name in ("orc_vec_dot_q8_0_q8_0", "orc_vec_dot_q4_K_q8_K", "orc_vec_dot_q6_K_q8_K"):
            getattr(L, name).restype = C.c_float
            getattr(L, name).argtypes = [i64, vp, vp]
        L.orc_vec_dot_q8x32.restype = C.c_float
        L.orc_vec_dot_q8x32.argtypes = [i32, i64, vp, vp]
        L.orc_mul_mat.restype = i32
        L.orc_mul_mat.argtypes = [i32, vp, i64, i64, f32p, i64, f32p, i32, i32]
        L.orc_mul_mat_f64.restype = i32
        L.orc_mul_mat_f64.argtypes = [i32, vp, i64, i64, f32p, i64, vp, i32]
        L.orc_mul_mat_id.restype = i32
        L.orc_mul_mat_id.argtypes = [i32, vp, i64, i64, i64, f32p, i64, vp, i64, i64, f32p, i32, i32]
        L.orc_moe_ffn.restype = i32
        L.orc_moe_ffn.argtypes = [i32, i32, vp, vp, vp, i64, i64, i64, f32p, vp, f32p, i64, i64,
                                  f32p, i32, i32]
        L.orc_time_mul_mat.restype = C.c_double
        L.orc_rms_norm.argtypes = [vp, vp, C.c_float, i64, i64, vp]
        L.orc_rms_norm.restype = None
        L.orc_time_mul_mat.argtypes = [i32, vp, i64, i64, f32p, i64, f32p, i32, i32, i32]
        L.orc_max_threads.restype = i32
        L.orc_has_avx2.restype = i32
        L.orc_mul_mat_avx2.restype = i32
        L.orc_mul_mat_avx2.argtypes = [i32, vp, i64, i64, f32p, i64, f32p, i32]
        L.orc_time_mul_mat_avx2.restype = C.c_double
        L.orc_time_mul_mat_avx2.argtypes = [i32, vp, i64, i64, f32p, i64, f32p, i32, i32]
        _lib = L
    return _lib


def _p(a: np.ndarray) -> int:
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data


def row_bytes(qtype: int, k: int) -> int:
    return int(lib().orc_row_bytes(qtype, k))


def fp16_to_fp32(h: int) -> float:
    return float(lib().orc_fp16_to_fp32(h))


def quantize(qtype: int, w: np.ndarray, nthreads: int = 8) -> np.ndarray:
    """float32 [N, K] -> uint8 [N, row_bytes] of GGUF Q8_0 blocks (quantize_row_q8_0_ref).  The oracle makes no
    Q4_K / Q6_K weight blocks: those are inputs of the path (tests/kquant_encoders.py encodes test inputs)."""
    w = np.ascontiguousarray(w, dtype=np.float32)
    n, k = w.shape
    out = np.zeros((n, row_bytes(qtype, k)), dtype=np.uint8)
    if lib().orc_quantize_rows(qtype, _p(w), _p(out), k, n, nthreads) != 0:
        raise ValueError("the oracle quantizes weights to Q8_0 only (K a multiple of 32)")
    return out


def dequantize(qtype: int, blocks: np.ndarray, k: int) -> np.ndarray:
    """uint8 [N, row_bytes] -> float32 [N, K]."""
    blocks = np.ascontiguousarray(blocks, dtype=np.uint8).reshape(-1, row_bytes(qtype, k))
    out = np.empty((blocks.shape[0], k), dtype=np.float32)
    for r in range(blocks.shape[0]):
        lib().orc_dequantize_row(qtype, _p(blocks[r]), _p(out[r]), k)
    return out


def quantize_q8_K(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    k = x.shape[-1]
    rows = x.reshape(-1, k)
    out = np.zeros((rows.shape[0], k // 256 * 292), dtype=np.uint8)
    for r in range(rows.shape[0]):
        lib().orc_quantize_row_q8_K(_p(rows[r]), _p(out[r]), k)
    return out


def quantize_q8_0_act(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    k = x.shape[-1]
    rows = x.reshape(-1, k)
    out = np.zeros((rows.shape[0], k // 32 * 34), dtype=np.uint8)
    for r in range(rows.shape[0]):
        lib().orc_quantize_row_q8_0(_p(rows[r]), _p(out[r]), k)
    return out


def quantize_q8x32(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    k = x.shape[-1]
    rows = x.reshape(-1, k)
    out = np.zeros((rows.shape[0], k // 32 * 40), dtype=np.uint8)
    for r in range(rows.shape[0]):
        lib().orc_quantize_row_q8x32(_p(rows[r]), _p(out[r]), k)
    return out


def mul_mat(qtype: int, w: np.ndarray, k: int, x: np.ndarray, act: int = ACT_GGML,
            nthreads: int = 8) -> np.ndarray:
    """w: uint8 [N, row_bytes]; x: float32 [M, K] -> float32 [M, N]."""
    w = np.ascontiguousarray(w, dtype=np.uint8)
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, k)
    n = w.size // row_bytes(qtype, k)
    m = x.shape[0]
    y = np.empty((m, n), dtype=np.float32)
    rc = lib().orc_mul_mat(qtype, _p(w), k, n, _p(x), m, _p(y), act, nthreads)
    if rc:
        raise RuntimeError(f"orc_mul_mat failed rc={rc}")
    return y


def mul_mat_f64(qtype: int, w: np.ndarray, k: int, x: np.ndarray, nthreads: int = 8) -> np.ndarray:
    w = np.ascontiguousarray(w, dtype=np.uint8)
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, k)
    n = w.size // row_bytes(qtype, k)
    m = x.shape[0]
    y = np.empty((m, n), dtype=np.float64)
    rc = lib().orc_mul_mat_f64(qtype, _p(w), k, n, _p(x), m, _p(y), nthreads)
    if rc:
        raise RuntimeError(f"orc_mul_mat_f64 failed rc={rc}")
    return y


def mul_mat_id(qtype: int, w_exps: np.ndarray, k: int, n: int, n_expert: int, b: np.ndarray,
               ids: np.ndarray, act: int = ACT_GGML, nthreads: int = 8) -> np.ndarray:
    """b: float32 [B, nb1, K] (nb1 in {1, n_used}); ids: int32 [B, n_used] -> [B, n_used, N]."""
    w_exps = np.ascontiguousarray(w_exps, dtype=np.uint8)
    b = np.ascontiguousarray(b, dtype=np.float32)
    ids = np.ascontiguousarray(ids, dtype=np.int32)
    B, n_used = ids.shape
    nb1 = b.shape[1]
    y = np.empty((B, n_used, n), dtype=np.float32)
    rc = lib().orc_mul_mat_id(qtype, _p(w_exps), k, n, n_expert, _p(b), nb1, _p(ids), n_used, B,
                              _p(y), act, nthreads)
    if rc:
        raise RuntimeError(f"orc_mul_mat_id failed rc={rc}")
    return y


def moe_ffn(type_gu: int, type_down: int, gate: np.ndarray, up: np.ndarray, down: np.ndarray,
            d_model: int, d_ff: int, n_expert: int, x: np.ndarray, ids: np.ndarray,
            weights: np.ndarray, act: int = ACT_GGML, nthreads: int = 8) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    ids = np.ascontiguousarray(ids, dtype=np.int32)
    weights = np.ascontiguousarray(weights, dtype=np.float32)
    B, n_used = ids.shape
    y = np.empty((B, d_model), dtype=np.float32)
    rc = lib().orc_moe_ffn(type_gu, type_down, _p(np.ascontiguousarray(gate)),
                           _p(np.ascontiguousarray(up)), _p(np.ascontiguousarray(down)), d_model,
                           d_ff, n_expert, _p(x), _p(ids), _p(weights), n_used, B, _p(y), act,
                           nthreads)
    if rc:
        raise RuntimeError(f"orc_moe_ffn failed rc={rc}")
    return y


def time_mul_mat(qtype: int, w: np.ndarray, k: int, x: np.ndarray, act: int, nthreads: int,
                 reps: int) -> float:
    w = np.ascontiguousarray(w, dtype=np.uint8)
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, k)
    n = w.size // row_bytes(qtype, k)
    m = x.shape[0]
    y = np.empty((m, n), dtype=np.float32)
    return float(lib().orc_time_mul_mat(qtype, _p(w), k, n, _p(x), m, _p(y), act, nthreads, reps))


def has_avx2() -> bool:
    return bool(lib().orc_has_avx2())


def mul_mat_avx2(qtype: int, w: np.ndarray, k: int, x: np.ndarray, nthreads: int = 8) -> np.ndarray:
    """mul_mat in the ggml activation mode through the AVX2 dot products (the CPU-baseline code path)."""
    w = np.ascontiguousarray(w, dtype=np.uint8)
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, k)
    n = w.size // row_bytes(qtype, k)
    m = x.shape[0]
    y = np.empty((m, n), dtype=np.float32)
    rc = lib().orc_mul_mat_avx2(qtype, _p(w), k, n, _p(x), m, _p(y), nthreads)
    if rc:
        raise RuntimeError(f"orc_mul_mat_avx2 failed rc={rc}")
    return y


def time_mul_mat_avx2(qtype: int, w: np.ndarray, k: int, x: np.ndarray, nthreads: int, reps: int) -> float:
    w = np.ascontiguousarray(w, dtype=np.uint8)
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, k)
    n = w.size // row_bytes(qtype, k)
    m = x.shape[0]
    y = np.empty((m, n), dtype=np.float32)
    t = float(lib().orc_time_mul_mat_avx2(qtype, _p(w), k, n, _p(x), m, _p(y), nthreads, reps))
    if t < 0:
        raise RuntimeError("the oracle was built without AVX2")
    return t


def rms_norm(x: np.ndarray, gamma, eps: float) -> np.ndarray:
    """RMS_NORM then MUL by the norm weights, row by row (gamma None: the norm alone)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    m, k = x.shape
    y = np.empty_like(x)
    g = None if gamma is None else np.ascontiguousarray(gamma, dtype=np.float32)
    lib().orc_rms_norm(_p(x), 0 if g is None else _p(g), C.c_float(eps), m, k, _p(y))
    return y


def max_threads() -> int:
    return int(lib().orc_max_threads())
