"""Independent numpy restatement of the GGUF block formats, written from the
public format description and vectorised over blocks -- a second opinion used
to pin the C oracle (a shared misreading would have to be made twice, in two
different code shapes).  fp16 decoding is numpy's own."""
import numpy as np


def f16(buf: np.ndarray) -> np.ndarray:
    """uint8 [..., 2] little-endian -> float32"""
    return np.ascontiguousarray(buf).view("<f2").astype(np.float32)[..., 0]


def deq_q8_0(blocks: np.ndarray) -> np.ndarray:
    b = blocks.reshape(-1, 34)
    d = f16(b[:, 0:2])
    q = b[:, 2:].view(np.int8).astype(np.float32)
    return (q * d[:, None]).astype(np.float32).reshape(-1)


def unpack_scales_k4(s: np.ndarray):
    """uint8 [nb, 12] -> (sc [nb, 8], mn [nb, 8]) per the 6-bit packing:
    bytes 0-3: low 6 bits = scale 0-3, top 2 bits = high bits of scale 4-7;
    bytes 4-7: low 6 bits = min 0-3, top 2 bits = high bits of min 4-7;
    bytes 8-11: low nibble = low 4 bits of scale 4-7, high nibble = low 4 bits of min 4-7."""
    s = s.astype(np.uint16)
    sc = np.empty((s.shape[0], 8), np.uint16)
    mn = np.empty((s.shape[0], 8), np.uint16)
    sc[:, 0:4] = s[:, 0:4] & 63
    mn[:, 0:4] = s[:, 4:8] & 63
    sc[:, 4:8] = (s[:, 8:12] & 15) | ((s[:, 0:4] >> 6) << 4)
    mn[:, 4:8] = (s[:, 8:12] >> 4) | ((s[:, 4:8] >> 6) << 4)
    return sc.astype(np.uint8), mn.astype(np.uint8)


def q4_K_ints(blocks: np.ndarray):
    """-> q [nb, 256] in 0..15, sc [nb, 8], mn [nb, 8], d [nb], dmin [nb]"""
    b = blocks.reshape(-1, 144)
    d = f16(b[:, 0:2])
    dmin = f16(b[:, 2:4])
    sc, mn = unpack_scales_k4(b[:, 4:16])
    qs = b[:, 16:].reshape(-1, 4, 32)
    q = np.stack([qs & 0xF, qs >> 4], axis=2).reshape(-1, 256)  # chunk c: 32 low then 32 high
    return q, sc, mn, d, dmin


def deq_q4_K(blocks: np.ndarray) -> np.ndarray:
    q, sc, mn, d, dmin = q4_K_ints(blocks)
    dsc = (d[:, None] * sc.astype(np.float32)).astype(np.float32)  # fp32 product
    dmn = (dmin[:, None] * mn.astype(np.float32)).astype(np.float32)
    qf = q.reshape(-1, 8, 32).astype(np.float32)
    prod = (dsc[:, :, None] * qf).astype(np.float32)
    return (prod - dmn[:, :, None]).astype(np.float32).reshape(-1)


def q6_K_ints(blocks: np.ndarray):
    """-> q [nb, 256] in -32..31, sc [nb, 16] int8, d [nb]"""
    b = blocks.reshape(-1, 210)
    ql = b[:, 0:128].reshape(-1, 2, 2, 32)   # half, (first 32 | second 32), l
    qh = b[:, 128:192].reshape(-1, 2, 32)
    sc = b[:, 192:208].view(np.int8)
    d = f16(b[:, 208:210])
    q = np.empty((b.shape[0], 2, 4, 32), np.int16)
    q[:, :, 0] = (ql[:, :, 0] & 0xF) | (((qh >> 0) & 3) << 4)
    q[:, :, 1] = (ql[:, :, 1] & 0xF) | (((qh >> 2) & 3) << 4)
    q[:, :, 2] = (ql[:, :, 0] >> 4) | (((qh >> 4) & 3) << 4)
    q[:, :, 3] = (ql[:, :, 1] >> 4) | (((qh >> 6) & 3) << 4)
    return (q.reshape(-1, 256) - 32).astype(np.int8), sc, d


def deq_q6_K(blocks: np.ndarray) -> np.ndarray:
    q, sc, d = q6_K_ints(blocks)
    dsc = (d[:, None] * sc.astype(np.float32)).astype(np.float32)
    return (dsc[:, :, None] * q.reshape(-1, 16, 16).astype(np.float32)).astype(np.float32).reshape(-1)


def quant_q8_0(x: np.ndarray) -> np.ndarray:
    """Benchmark config 1: d = max|w|/127 stored fp16, q = round(w/d) (half away from zero,
    the multiply by the fp32 reciprocal of the unrounded d)."""
    xb = x.astype(np.float32).reshape(-1, 32)
    amax = np.abs(xb).max(axis=1)
    d = (amax / np.float32(127)).astype(np.float32)
    with np.errstate(divide="ignore"):
        inv = np.where(d != 0, np.float32(1) / d, np.float32(0)).astype(np.float32)
    v = (xb * inv[:, None]).astype(np.float32)
    q = (np.sign(v) * np.floor(np.abs(v).astype(np.float64) + 0.5)).astype(np.int8)
    out = np.empty((xb.shape[0], 34), np.uint8)
    out[:, 0:2] = d.astype("<f2").view(np.uint8).reshape(-1, 2)
    out[:, 2:] = q.view(np.uint8)
    return out.reshape(-1)
