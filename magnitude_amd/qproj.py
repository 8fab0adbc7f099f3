"""Host-side mirror of the projection operators, over the qproj C ABI (include/qproj.h).

The operator names and argument meaning follow the ggml graph ops that Magnitude's engine
reaches through its one native call per scheduler step
(/root/reference/inference/crates/icn-engine/src/lib.rs:2264): ``mul_mat`` is GGML_OP_MUL_MAT,
``mul_mat_id`` is GGML_OP_MUL_MAT_ID, ``moe_ffn`` is llama.cpp's build_moe_ffn.  torch is used
only to own device memory; every computation is a HIP kernel inside libqproj.so.  There is no
CPU or torch fallback: a missing library or a failing call raises.
"""
from __future__ import annotations

import ctypes as C
import os
from typing import Optional, Sequence

import numpy as np
import torch

TYPE_Q8_0, TYPE_Q4_K, TYPE_Q6_K = 8, 12, 14
ACT_GGML, ACT_F32, ACT_Q8X32 = 0, 1, 2
TYPE_NAMES = {TYPE_Q8_0: "Q8_0", TYPE_Q4_K: "Q4_K", TYPE_Q6_K: "Q6_K"}
BLOCK_BYTES = {TYPE_Q8_0: 34, TYPE_Q4_K: 144, TYPE_Q6_K: 210}
BLOCK_ELEMS = {TYPE_Q8_0: 32, TYPE_Q4_K: 256, TYPE_Q6_K: 256}

STATUS_NAMES = {0: "OK", 1: "INVALID_ARG", 2: "HIP", 3: "OOM", 4: "UNSUPPORTED", 5: "NO_DEVICE"}

# QPROJ_LIBRARY points at another build of the same library (e.g. an instrumented one)
LIB_PATH = os.environ.get("QPROJ_LIBRARY") or os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib",
                                                           "libqproj.so")

# every symbol include/qproj.h declares: (restype, argtypes)
_vp, _i64, _i32, _sz = C.c_void_p, C.c_int64, C.c_int, C.c_size_t
SYMBOLS = {
    "qproj_device_count": (_i32, [C.POINTER(C.c_int)]),
    "qproj_ctx_create": (_i32, [_i32, _vp, C.POINTER(_vp)]),
    "qproj_ctx_destroy": (_i32, [_vp]),
    "qproj_sync": (_i32, [_vp]),
    "qproj_last_error": (C.c_char_p, [_vp]),
    "qproj_stream": (_vp, [_vp]),
    "qproj_row_bytes": (_sz, [_i32, _i64]),
    "qproj_upload": (_i32, [_vp, _i32, _i64, _i64, _i64, _vp, C.POINTER(_vp)]),
    "qproj_upload_from_device": (_i32, [_vp, _i32, _i64, _i64, _i64, _vp, C.POINTER(_vp)]),
    "qproj_download": (_i32, [_vp, _vp, _vp]),
    "qproj_weight_free": (_i32, [_vp, _vp]),
    "qproj_weight_info": (_i32, [_vp, C.POINTER(C.c_int), C.POINTER(_i64), C.POINTER(_i64),
                                 C.POINTER(_i64), C.POINTER(_sz)]),
    "qproj_dequantize": (_i32, [_vp, _vp, _vp]),
    "qproj_act_bytes": (_sz, [_i32, _i32, _i64, _i64]),
    "qproj_quantize_activations": (_i32, [_vp, _i32, _i32, _vp, _i64, _i64, _vp]),
    "qproj_rms_norm": (_i32, [_vp, _vp, _vp, C.c_float, _i64, _i64, _vp]),
    "qproj_ffn_gate_up": (_i32, [_vp, _vp, _vp, _vp, _i64, _vp, _i32]),
    "qproj_rms_norm_ffn_gate_up": (_i32, [_vp, _vp, _vp, _vp, _vp, C.c_float, _i64, _vp, _i32]),
    "qproj_rms_norm_mul_mat": (_i32, [_vp, _i32, _vp, _vp, _vp, C.c_float, _i64, _vp, _i32]),
    "qproj_rms_norm_quantize": (_i32, [_vp, _i32, _i32, _vp, _vp, C.c_float, _i64, _i64, _vp]),
    "qproj_ffn": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, C.c_float, _i32, _i64, _vp, _i32]),
    "qproj_mul_mat": (_i32, [_vp, _vp, _vp, _i64, _vp, _i32]),
    "qproj_mul_mat_multi": (_i32, [_vp, _i32, C.POINTER(_vp), _vp, _i64, C.POINTER(_vp), _i32]),
    "qproj_mul_mat_multi_noalloc": (_i32, [_vp, _i32, C.POINTER(_vp), _vp, _i64, C.POINTER(_vp), _i32]),
    "qproj_workspace_bytes": (_sz, [_i32, _i64, _i32, C.POINTER(_i64), _i64, _i32, C.POINTER(C.c_int)]),
    "qproj_mul_mat_quantized": (_i32, [_vp, _i32, C.POINTER(_vp), _vp, _i32, _i64, C.POINTER(_vp)]),
    "qproj_mul_mat_id": (_i32, [_vp, _vp, _vp, _i64, _vp, _i64, _i64, _vp, _i32]),
    "qproj_moe_ffn": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _vp, _i32]),
    "qproj_plan_mul_mat": (_i32, [_i32, _i64, _i32, C.POINTER(_i64), _i64, _i32, _i32, C.c_char_p, _sz]),
    "qproj_plan_moe_ffn": (_i32, [_i32, _i32, _i64, _i64, _i64, _i64, _i64, C.c_char_p, _sz]),
    "qproj_version": (C.c_char_p, []),
    "qproj_probe_eligibility": (_i32, [_vp]),
}

PROBE_MAX_DEVICES = 16


class Eligibility(C.Structure):
    """struct qproj_eligibility of include/qproj.h"""
    _fields_ = [("state", C.c_int), ("driver_api", C.c_int), ("runtime_api", C.c_int), ("n_devices", C.c_int),
                ("architectures", (C.c_char * 32) * PROBE_MAX_DEVICES),
                ("hardware_labels", (C.c_char * 256) * PROBE_MAX_DEVICES),
                ("runtime_library", C.c_char * 1024), ("diagnostic", C.c_char * 244)]


class QprojError(RuntimeError):
    def __init__(self, status: int, message: str):
        super().__init__(f"qproj status {status} ({STATUS_NAMES.get(status, '?')}): {message}")
        self.status = status


_lib = None


def load_library(path: Optional[str] = None) -> C.CDLL:
    """dlopen libqproj.so and bind every declared entry point; raises if it is not built."""
    global _lib
    if _lib is not None and path is None:
        return _lib
    p = path or LIB_PATH
    if not os.path.exists(p):
        raise FileNotFoundError(
            f"{p} is missing: build it with `make -C magnitude_amd/csrc` (hipcc, gfx950). "
            "There is no fallback path.")
    lib = C.CDLL(p)
    for name, (res, args) in SYMBOLS.items():
        fn = getattr(lib, name)  # AttributeError if the library does not export it
        fn.restype = res
        fn.argtypes = args
    if path is None:
        _lib = lib
    return lib


def _probe() -> Eligibility:
    e = Eligibility()
    st = load_library().qproj_probe_eligibility(C.byref(e))
    if st:
        raise QprojError(st, "qproj_probe_eligibility")
    return e


def probe_eligibility() -> dict:
    """The backend eligibility entry a HIP backend would add to the server's report, in exactly the contract's
    serialised shape (/root/reference/inference/crates/icn-contracts/src/bootstrap_protocol.rs:14-39: tag
    "state" in lowercase, camelCase fields, unknown fields denied): {"state": "usable", "driverApi",
    "architectures", "driverLibrary"} or {"state": "absent" | "failed", "diagnostic"}."""
    e = _probe()
    if e.state == 0:
        return {"state": "usable", "driverApi": e.driver_api,
                "architectures": [e.architectures[i].value.decode() for i in range(e.n_devices)],
                "driverLibrary": e.runtime_library.decode(errors="replace")}
    return {"state": "absent" if e.state == 1 else "failed", "diagnostic": e.diagnostic.decode(errors="replace")}


def probe_hardware() -> dict:
    """What the probe learns beside the contract entry: one hardware label per device and the runtime version
    (the reference keeps its hardware labels beside the report as well,
    /root/reference/inference/crates/icn-server/src/cuda_driver.rs:78).  Empty lists when no device is usable."""
    e = _probe()
    n = e.n_devices if e.state == 0 else 0
    return {"runtimeApi": e.runtime_api if e.state == 0 else 0,
            "hardwareLabels": [e.hardware_labels[i].value.decode(errors="replace") for i in range(n)]}


NOALLOC_SCRATCH_BYTES = 64 << 20


def workspace_bytes(qtype: int, k: int, ns: Sequence[int], m: int, act: int = ACT_GGML) -> int:
    """Scratch bytes mul_mat_multi reserves for this shape; raises when the library's walk of its own dispatch
    finds a launcher that the reserved scratch would not satisfy.  Needs no GPU."""
    arr = (_i64 * len(ns))(*ns)
    st = C.c_int(0)
    nbytes = int(load_library().qproj_workspace_bytes(qtype, k, len(ns), arr, m, act, C.byref(st)))
    if st.value:
        raise QprojError(st.value, f"qproj_workspace_bytes(type {qtype}, K {k}, N {list(ns)}, M {m}, act {act})")
    return nbytes


def plan_mul_mat(qtype: int, k: int, ns: Sequence[int], m: int, act: int = ACT_GGML, with_norm: bool = False) -> str:
    """The launches mul_mat_multi (or rms_norm_mul_mat) makes for this shape, one line each, as the launchers
    themselves describe them in a dry run of the dispatch; the last line is the scratch reserved.  Needs no GPU."""
    arr = (_i64 * len(ns))(*ns)
    buf = C.create_string_buffer(8192)
    st = load_library().qproj_plan_mul_mat(qtype, k, len(ns), arr, m, act, 1 if with_norm else 0, buf, len(buf))
    if st:
        raise QprojError(st, f"qproj_plan_mul_mat(type {qtype}, K {k}, N {list(ns)}, M {m}, act {act}): " + buf.value.decode())
    return buf.value.decode()


def plan_moe_ffn(gate_type: int, down_type: int, d_model: int, d_ff: int, n_expert: int, n_used: int, batch: int) -> str:
    """The launches moe_ffn makes for this shape (see plan_mul_mat)."""
    buf = C.create_string_buffer(8192)
    st = load_library().qproj_plan_moe_ffn(gate_type, down_type, d_model, d_ff, n_expert, n_used, batch, buf, len(buf))
    if st:
        raise QprojError(st, f"qproj_plan_moe_ffn({gate_type}, {down_type}, {d_model}, {d_ff}, {n_expert}, {n_used}, {batch}): " + buf.value.decode())
    return buf.value.decode()


def row_bytes(qtype: int, k: int) -> int:
    return int(load_library().qproj_row_bytes(qtype, k))


def _ptr(t: torch.Tensor) -> int:
    if not t.is_cuda:
        raise ValueError("device tensor expected")
    if not t.is_contiguous():
        raise ValueError("contiguous tensor expected")
    return t.data_ptr()


class Weight:
    """A quantized weight resident on the device (N rows of K weights, E experts)."""

    def __init__(self, ctx: "Context", handle: int, qtype: int, k: int, n: int, n_expert: int):
        self.ctx, self.handle, self.qtype, self.K, self.N, self.E = ctx, handle, qtype, k, n, n_expert

    @property
    def gguf_bytes(self) -> int:
        return self.E * self.N * (self.K // BLOCK_ELEMS[self.qtype]) * BLOCK_BYTES[self.qtype]

    def free(self) -> None:
        if self.handle:
            self.ctx.lib.qproj_weight_free(self.ctx.handle, self.handle)
            self.handle = 0

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Context:
    """One device + one HIP stream.  Not thread-safe, like the engine's single executor thread."""

    def __init__(self, device: int = 0, stream: Optional[int] = None):
        self.lib = load_library()
        h = _vp()
        st = self.lib.qproj_ctx_create(device, _vp(stream) if stream else None, C.byref(h))
        if st:
            raise QprojError(st, "qproj_ctx_create failed (is a gfx950 device visible?)")
        self.handle = h.value
        self.device = device
        self._held = []     # contiguous copies handed to launches that may still be pending (dropped in sync())

    def close(self) -> None:
        if getattr(self, "handle", 0):
            self.lib.qproj_ctx_destroy(self.handle)
            self.handle = 0

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def _check(self, status: int) -> None:
        if status:
            raise QprojError(status, self.lib.qproj_last_error(self.handle).decode())

    @property
    def stream(self) -> int:
        return int(self.lib.qproj_stream(self.handle) or 0)

    def sync(self) -> None:
        self._check(self.lib.qproj_sync(self.handle))
        self._held.clear()

    def _cptr(self, t: torch.Tensor) -> int:
        """Device address of t made contiguous.  A copy made for that is kept alive until the next sync(): the launch
        that reads it runs on the context's own stream, which torch's allocator does not track, so a temporary freed
        when the ctypes call returns could be handed out again while the kernel is still reading it."""
        c = t.contiguous()
        if c is not t:
            self._held.append(c)
        return _ptr(c)

    # ---- weights -------------------------------------------------------------------------
    def upload(self, qtype: int, k: int, n: int, gguf: np.ndarray, n_expert: int = 1) -> Weight:
        """gguf: host uint8 array holding n_expert*n rows of k weights in GGUF block layout."""
        buf = np.ascontiguousarray(gguf, dtype=np.uint8)
        want = n_expert * n * row_bytes(qtype, k)
        if want == 0 or buf.size != want:
            raise ValueError(f"expected {want} bytes of {TYPE_NAMES.get(qtype, qtype)} blocks, got {buf.size}")
        h = _vp()
        self._check(self.lib.qproj_upload(self.handle, qtype, k, n, n_expert, buf.ctypes.data, C.byref(h)))
        return Weight(self, h.value, qtype, k, n, n_expert)

    def upload_from_device(self, qtype: int, k: int, n: int, gguf: torch.Tensor, n_expert: int = 1) -> Weight:
        want = n_expert * n * row_bytes(qtype, k)
        if gguf.dtype != torch.uint8 or gguf.numel() != want:
            raise ValueError(f"expected {want} uint8 bytes on the device")
        torch.cuda.current_stream().synchronize()
        h = _vp()
        self._check(self.lib.qproj_upload_from_device(self.handle, qtype, k, n, n_expert, _ptr(gguf), C.byref(h)))
        return Weight(self, h.value, qtype, k, n, n_expert)

    def download(self, w: Weight) -> np.ndarray:
        out = np.empty(w.gguf_bytes, dtype=np.uint8)
        self._check(self.lib.qproj_download(self.handle, w.handle, out.ctypes.data))
        return out

    def dequantize(self, w: Weight) -> torch.Tensor:
        out = torch.empty((w.E * w.N, w.K), dtype=torch.float32, device=f"cuda:{self.device}")
        torch.cuda.current_stream().synchronize()
        self._check(self.lib.qproj_dequantize(self.handle, w.handle, _ptr(out)))
        self.sync()
        return out

    # ---- activations ---------------------------------------------------------------------
    def quantize_activations(self, x: torch.Tensor, kind: int, wtype: int) -> dict:
        """Runs the activation quantizer and returns its planes as torch tensors."""
        x = x.contiguous()
        m, k = x.shape
        nbytes = int(self.lib.qproj_act_bytes(kind, wtype, m, k))
        if nbytes == 0:
            raise ValueError("bad activation shape or kind")
        buf = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
        torch.cuda.current_stream().synchronize()
        self._check(self.lib.qproj_quantize_activations(self.handle, kind, wtype, _ptr(x), m, k, _ptr(buf)))
        self.sync()
        al = lambda v: (v + 255) // 256 * 256
        per256 = kind == ACT_GGML and wtype != TYPE_Q8_0
        dblk = 256 if per256 else 32
        off_d = al(m * k)
        off_aux = off_d + al(m * (k // dblk) * 4)
        out = {
            "qs": buf[:m * k].view(torch.int8).view(m, k),
            "d": buf[off_d:off_d + m * (k // dblk) * 4].view(torch.float32).view(m, k // dblk),
        }
        if per256:
            out["bsums"] = buf[off_aux:off_aux + m * (k // 16) * 2].view(torch.int16).view(m, k // 16)
            off_ms = off_aux + al(m * (k // 16) * 2)
            out["msum"] = buf[off_ms:off_ms + m * (k // 256) * 32].view(torch.float16).view(m, k // 256, 2, 8)
            off_rs = off_ms + al(m * (k // 256) * 32)
            out["rs"] = buf[off_rs:off_rs + m * 4].view(torch.float32)
        elif kind == ACT_Q8X32:
            out["isum"] = buf[off_aux:off_aux + m * (k // 32) * 4].view(torch.int32).view(m, k // 32)
            off_ms = off_aux + al(m * (k // 32) * 4)
            out["msum"] = buf[off_ms:off_ms + m * (k // 256) * 32].view(torch.float16).view(m, k // 256, 2, 8)
            off_rs = off_ms + al(m * (k // 256) * 32)
            out["rs"] = buf[off_rs:off_rs + m * 4].view(torch.float32)
        return out

    # ---- operators -----------------------------------------------------------------------
    def mul_mat(self, w: Weight, x: torch.Tensor, act: int = ACT_GGML, out: Optional[torch.Tensor] = None,
                sync: bool = True) -> torch.Tensor:
        """GGML_OP_MUL_MAT: x f32 [M, K] -> y f32 [M, N]."""
        x2 = x.reshape(-1, w.K)
        if x2.dtype != torch.float32:
            raise ValueError("activations must be float32")
        m = x2.shape[0]
        y = out if out is not None else torch.empty((m, w.N), dtype=torch.float32, device=x.device)
        if sync:
            torch.cuda.current_stream().synchronize()
        self._check(self.lib.qproj_mul_mat(self.handle, w.handle, self._cptr(x2), m, _ptr(y), act))
        if sync:
            self.sync()
        return y

    def mul_mat_multi(self, ws: Sequence[Weight], x: torch.Tensor, act: int = ACT_GGML,
                      outs: Optional[Sequence[torch.Tensor]] = None, sync: bool = True, noalloc: bool = False):
        """Several MUL_MATs sharing one activation (q/k/v or gate/up) in one launch.  noalloc: through the entry
        point that keeps its scratch in the library's fixed buffer and allocates nothing (the outputs must be
        passed in then, or they are made here before the call)."""
        x2 = x.reshape(-1, ws[0].K).contiguous()
        m = x2.shape[0]
        ys = list(outs) if outs is not None else [
            torch.empty((m, w.N), dtype=torch.float32, device=x.device) for w in ws]
        n = len(ws)
        wa = (_vp * n)(*[w.handle for w in ws])
        ya = (_vp * n)(*[_ptr(y) for y in ys])
        if sync:
            torch.cuda.current_stream().synchronize()
        fn = self.lib.qproj_mul_mat_multi_noalloc if noalloc else self.lib.qproj_mul_mat_multi
        self._check(fn(self.handle, n, wa, _ptr(x2), m, ya, act))
        if sync:
            self.sync()
        return ys

    def rms_norm(self, x: torch.Tensor, gamma: Optional[torch.Tensor], eps: float,
                 out: Optional[torch.Tensor] = None, sync: bool = True) -> torch.Tensor:
        """GGML_OP_RMS_NORM followed by GGML_OP_MUL with the norm weights (gamma None: the norm alone)."""
        x = x.contiguous()
        m, k = x.shape
        y = out if out is not None else torch.empty_like(x)
        if sync:
            torch.cuda.current_stream().synchronize()
        self._check(self.lib.qproj_rms_norm(self.handle, _ptr(x), 0 if gamma is None else self._cptr(gamma),
                                            C.c_float(eps), m, k, _ptr(y)))
        if sync:
            self.sync()
        return y

    def rms_norm_quantize_raw(self, x: torch.Tensor, gamma: Optional[torch.Tensor], eps: float, kind: int, wtype: int,
                              out: Optional[torch.Tensor] = None, sync: bool = True) -> torch.Tensor:
        """Norm, weight multiply and activation quantizer in one launch; the buffer feeds mul_mat_quantized."""
        x = x.contiguous()
        m, k = x.shape
        nbytes = int(self.lib.qproj_act_bytes(kind, wtype, m, k))
        if nbytes == 0:
            raise ValueError("bad activation shape or kind")
        buf = out if out is not None else torch.empty(nbytes, dtype=torch.uint8, device=x.device)
        if sync:
            torch.cuda.current_stream().synchronize()
        self._check(self.lib.qproj_rms_norm_quantize(self.handle, kind, wtype, _ptr(x),
                                                     0 if gamma is None else self._cptr(gamma),
                                                     C.c_float(eps), m, k, _ptr(buf)))
        if sync:
            self.sync()
        return buf

    def rms_norm_mul_mat(self, ws: Sequence[Weight], x: torch.Tensor, gamma: Optional[torch.Tensor], eps: float,
                         act: int = ACT_GGML, outs: Optional[Sequence[torch.Tensor]] = None, sync: bool = True):
        """RMS norm (+ norm weights) and the MUL_MATs that share the normalised rows (q/k/v, gate/up)."""
        x2 = x.reshape(-1, ws[0].K).contiguous()
        m = x2.shape[0]
        ys = list(outs) if outs is not None else [
            torch.empty((m, w.N), dtype=torch.float32, device=x.device) for w in ws]
        n = len(ws)
        wa = (_vp * n)(*[w.handle for w in ws])
        ya = (_vp * n)(*[_ptr(y) for y in ys])
        if sync:
            torch.cuda.current_stream().synchronize()
        self._check(self.lib.qproj_rms_norm_mul_mat(self.handle, n, wa, _ptr(x2),
                                                    0 if gamma is None else self._cptr(gamma),
                                                    C.c_float(eps), m, ya, act))
        if sync:
            self.sync()
        return ys

    def ffn_gate_up(self, gate: Weight, up: Weight, x: torch.Tensor, act: int = ACT_GGML,
                    gamma: Optional[torch.Tensor] = None, eps: Optional[float] = None,
                    out: Optional[torch.Tensor] = None, sync: bool = True) -> torch.Tensor:
        """h = silu(gate . x) * (up . x); with eps given, behind an RMS norm (gamma: the norm weights or None)."""
        x2 = x.reshape(-1, gate.K).contiguous()
        m = x2.shape[0]
        h = out if out is not None else torch.empty((m, gate.N), dtype=torch.float32, device=x.device)
        if sync:
            torch.cuda.current_stream().synchronize()
        if eps is None:
            self._check(self.lib.qproj_ffn_gate_up(self.handle, gate.handle, up.handle, _ptr(x2), m, _ptr(h), act))
        else:
            self._check(self.lib.qproj_rms_norm_ffn_gate_up(self.handle, gate.handle, up.handle, _ptr(x2),
                                                            0 if gamma is None else self._cptr(gamma),
                                                            C.c_float(eps), m, _ptr(h), act))
        if sync:
            self.sync()
        return h

    def quantize_activations_raw(self, x: torch.Tensor, kind: int, wtype: int,
                                 out: Optional[torch.Tensor] = None, sync: bool = True) -> torch.Tensor:
        """Activation quantizer into one opaque device buffer, for mul_mat_quantized."""
        x = x.contiguous()
        m, k = x.shape
        nbytes = int(self.lib.qproj_act_bytes(kind, wtype, m, k))
        if nbytes == 0:
            raise ValueError("bad activation shape or kind")
        buf = out if out is not None else torch.empty(nbytes, dtype=torch.uint8, device=x.device)
        if sync:
            torch.cuda.current_stream().synchronize()
        self._check(self.lib.qproj_quantize_activations(self.handle, kind, wtype, _ptr(x), m, k, _ptr(buf)))
        if sync:
            self.sync()
        return buf

    def mul_mat_quantized(self, ws: Sequence[Weight], act: torch.Tensor, kind: int, m: int,
                          outs: Sequence[torch.Tensor], sync: bool = True):
        """MUL_MAT over activations quantized beforehand (shared by all of `ws`)."""
        n = len(ws)
        wa = (_vp * n)(*[w.handle for w in ws])
        ya = (_vp * n)(*[_ptr(y) for y in outs])
        if sync:
            torch.cuda.current_stream().synchronize()
        self._check(self.lib.qproj_mul_mat_quantized(self.handle, n, wa, _ptr(act), kind, m, ya))
        if sync:
            self.sync()
        return outs

    def ffn(self, gate: Weight, up: Weight, down: Weight, x: torch.Tensor, act: int = ACT_GGML,
            gamma: Optional[torch.Tensor] = None, eps: Optional[float] = None, out: Optional[torch.Tensor] = None,
            sync: bool = True) -> torch.Tensor:
        """down . (silu(gate . x') * (up . x')), x' = rms_norm(x) * gamma when eps is given: the dense feed-forward."""
        x = x.contiguous()
        m = x.shape[0]
        y = out if out is not None else torch.empty((m, down.N), dtype=torch.float32, device=x.device)
        if sync:
            torch.cuda.current_stream().synchronize()
        self._check(self.lib.qproj_ffn(self.handle, gate.handle, up.handle, down.handle, _ptr(x),
                                       0 if gamma is None else self._cptr(gamma),
                                       C.c_float(0.0 if eps is None else eps), 0 if eps is None else 1, m, _ptr(y), act))
        if sync:
            self.sync()
        return y

    def mul_mat_id(self, w: Weight, x: torch.Tensor, ids: torch.Tensor, act: int = ACT_GGML,
                   sync: bool = True) -> torch.Tensor:
        """GGML_OP_MUL_MAT_ID: x f32 [B, nb1, K] (nb1 in {1, n_used}); ids i32 [B, n_used]
        -> f32 [B, n_used, N]."""
        if ids.dtype != torch.int32 or x.dtype != torch.float32:
            raise ValueError("ids must be int32 and x float32")
        b, n_used = ids.shape
        nb1 = x.shape[1]
        y = torch.empty((b, n_used, w.N), dtype=torch.float32, device=x.device)
        if sync:
            torch.cuda.current_stream().synchronize()
        self._check(self.lib.qproj_mul_mat_id(self.handle, w.handle, self._cptr(x), nb1,
                                              self._cptr(ids), n_used, b, _ptr(y), act))
        if sync:
            self.sync()
        return y

    def moe_ffn(self, gate: Weight, up: Weight, down: Weight, x: torch.Tensor, ids: torch.Tensor,
                weights: torch.Tensor, act: int = ACT_GGML, out: torch.Tensor = None,
                sync: bool = True) -> torch.Tensor:
        """y[b] = sum_j weights[b, j] * down_e(silu(gate_e x_b) * up_e x_b), e = ids[b, j]."""
        if ids.dtype != torch.int32 or x.dtype != torch.float32 or weights.dtype != torch.float32:
            raise ValueError("ids must be int32, x and weights float32")
        if ids.dim() != 2 or tuple(weights.shape) != tuple(ids.shape) or x.shape[0] != ids.shape[0]:
            raise ValueError("ids and weights must be [B, n_used] and x [B, d_model]")
        b, n_used = ids.shape
        y = out if out is not None else torch.empty((b, gate.K), dtype=torch.float32, device=x.device)
        if sync:
            torch.cuda.current_stream().synchronize()
        self._check(self.lib.qproj_moe_ffn(self.handle, gate.handle, up.handle, down.handle,
                                           self._cptr(x), self._cptr(ids),
                                           self._cptr(weights), n_used, b, _ptr(y), act))
        if sync:
            self.sync()
        return y
