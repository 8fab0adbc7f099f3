"""Synthetic GGUF weights for benchmarks and smoke runs: plain round-to-nearest quantizers written
with torch ops so that multi-gigabyte weight sets are produced on the device in milliseconds.

These are format-valid Q8_0 / Q4_K / Q6_K encoders (min/max affine per sub-block, no error
search), not a re-implementation of llama.cpp's offline quantizer: model files arrive already
quantized, so the projection path never quantizes weights.  Q8_0 follows the benchmark's own
definition exactly (d = max|w|/127 as fp16, q = round(w/d)).
"""
from __future__ import annotations

import torch

TYPE_Q8_0, TYPE_Q4_K, TYPE_Q6_K = 8, 12, 14


def _round_half_away(v: torch.Tensor) -> torch.Tensor:
    return torch.sign(v) * torch.floor(v.abs() + 0.5)


def _f16_bytes(v: torch.Tensor) -> torch.Tensor:
    return v.to(torch.float16).contiguous().view(torch.uint8).reshape(*v.shape, 2)


def quantize_q8_0(w: torch.Tensor) -> torch.Tensor:
    n, k = w.shape
    xb = w.float().reshape(n, k // 32, 32)
    amax = xb.abs().amax(dim=2)
    d = amax / 127.0
    inv = torch.where(d != 0, 1.0 / d, torch.zeros_like(d))
    q = _round_half_away(xb * inv[..., None]).to(torch.int8)
    out = torch.empty((n, k // 32, 34), dtype=torch.uint8, device=w.device)
    out[..., 0:2] = _f16_bytes(d)
    out[..., 2:] = q.view(torch.uint8)
    return out.reshape(n, -1)


def quantize_q4_k(w: torch.Tensor) -> torch.Tensor:
    n, k = w.shape
    nb = k // 256
    x = w.float().reshape(n, nb, 8, 32)
    lo = torch.clamp(x.amin(dim=3), max=0.0)
    hi = x.amax(dim=3)
    scale = (hi - lo) / 15.0                      # >= 0
    mn = -lo                                      # >= 0
    max_scale = scale.amax(dim=2, keepdim=True)
    max_min = mn.amax(dim=2, keepdim=True)
    inv_s = torch.where(max_scale > 0, 63.0 / max_scale, torch.zeros_like(max_scale))
    inv_m = torch.where(max_min > 0, 63.0 / max_min, torch.zeros_like(max_min))
    ls = torch.clamp(torch.round(inv_s * scale), 0, 63).to(torch.int32)
    lm = torch.clamp(torch.round(inv_m * mn), 0, 63).to(torch.int32)
    d = (max_scale / 63.0).to(torch.float16)
    dmin = (max_min / 63.0).to(torch.float16)
    dsc = d.float() * ls.float()
    dmn = dmin.float() * lm.float()
    safe = torch.where(dsc != 0, dsc, torch.ones_like(dsc))
    q = torch.where(dsc[..., None] != 0, torch.round((x + dmn[..., None]) / safe[..., None]),
                    torch.zeros_like(x))
    q = torch.clamp(q, 0, 15).to(torch.uint8)     # [n, nb, 8, 32]
    out = torch.empty((n, nb, 144), dtype=torch.uint8, device=w.device)
    out[..., 0:2] = _f16_bytes(d[..., 0])
    out[..., 2:4] = _f16_bytes(dmin[..., 0])
    sc = torch.zeros((n, nb, 12), dtype=torch.int32, device=w.device)
    sc[..., 0:4] = ls[..., 0:4] | ((ls[..., 4:8] >> 4) << 6)
    sc[..., 4:8] = lm[..., 0:4] | ((lm[..., 4:8] >> 4) << 6)
    sc[..., 8:12] = (ls[..., 4:8] & 0xF) | ((lm[..., 4:8] & 0xF) << 4)
    out[..., 4:16] = sc.to(torch.uint8)
    qc = q.reshape(n, nb, 4, 2, 32)               # chunk, (low | high), l
    out[..., 16:] = (qc[..., 0, :] | (qc[..., 1, :] << 4)).reshape(n, nb, 128)
    return out.reshape(n, -1)


def quantize_q6_k(w: torch.Tensor) -> torch.Tensor:
    n, k = w.shape
    nb = k // 256
    x = w.float().reshape(n, nb, 16, 16)
    idx = x.abs().argmax(dim=3, keepdim=True)
    mx = torch.gather(x, 3, idx)[..., 0]          # signed value of the largest magnitude
    scale = mx / -32.0
    sidx = scale.abs().argmax(dim=2, keepdim=True)
    max_scale = torch.gather(scale, 2, sidx)      # [n, nb, 1]
    zero = max_scale.abs() < 1e-15
    iscale = torch.where(zero, torch.zeros_like(max_scale), -128.0 / torch.where(zero, torch.ones_like(max_scale), max_scale))
    d = torch.where(zero, torch.zeros_like(iscale), 1.0 / torch.where(zero, torch.ones_like(iscale), iscale)).to(torch.float16)
    sc = torch.clamp(torch.round(iscale * scale), -128, 127).to(torch.int32)
    dsc = d.float() * sc.float()
    safe = torch.where(dsc != 0, dsc, torch.ones_like(dsc))
    q = torch.where(dsc[..., None] != 0, torch.round(x / safe[..., None]), torch.zeros_like(x))
    L = (torch.clamp(q, -32, 31) + 32).to(torch.uint8).reshape(n, nb, 2, 4, 32)   # half, group, l
    out = torch.empty((n, nb, 210), dtype=torch.uint8, device=w.device)
    ql = torch.empty((n, nb, 2, 2, 32), dtype=torch.uint8, device=w.device)
    ql[..., 0, :] = (L[..., 0, :] & 0xF) | ((L[..., 2, :] & 0xF) << 4)
    ql[..., 1, :] = (L[..., 1, :] & 0xF) | ((L[..., 3, :] & 0xF) << 4)
    qh = (L[..., 0, :] >> 4) | ((L[..., 1, :] >> 4) << 2) | ((L[..., 2, :] >> 4) << 4) | ((L[..., 3, :] >> 4) << 6)
    out[..., 0:128] = ql.reshape(n, nb, 128)
    out[..., 128:192] = qh.reshape(n, nb, 64)
    out[..., 192:208] = sc.to(torch.int8).view(torch.uint8)
    out[..., 208:210] = _f16_bytes(d[..., 0])
    return out.reshape(n, -1)


def quantize(qtype: int, w: torch.Tensor) -> torch.Tensor:
    if qtype == TYPE_Q8_0:
        return quantize_q8_0(w)
    if qtype == TYPE_Q4_K:
        return quantize_q4_k(w)
    if qtype == TYPE_Q6_K:
        return quantize_q6_k(w)
    raise ValueError(f"unsupported type {qtype}")


def random_weight(qtype: int, n: int, k: int, seed: int, device, std: float = 0.02,
                  rows_per_pass: int = 4096) -> torch.Tensor:
    """N(0, std) weights quantized to `qtype`; uint8 [n, row_bytes] on `device`."""
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    parts = []
    for r0 in range(0, n, rows_per_pass):
        r = min(rows_per_pass, n - r0)
        w = torch.randn((r, k), generator=g, device=device, dtype=torch.float32) * std
        parts.append(quantize(qtype, w))
    return torch.cat(parts, dim=0).contiguous()
