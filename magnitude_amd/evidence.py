"""Result records in the shapes the reference's own tooling decodes.

* `backend_ops_row` / `backend_ops_sql`: the 16 fields of llama.cpp's `test-backend-ops perf --output sql`
  rows, which the reference's qualification lane parses
  (inference/crates/icn-parity/src/decode.rs:547-564, sample row :1421).
* `measurement`: a parity `measurement{name, unit, samples[]}` object with every raw sample kept
  (inference/parity/schemas/evidence.schema.json:147-165, parity/README.md:110).
* `calibration_metric`: one entry of the hardware calibration the engine's performance estimator
  consumes (inference/crates/icn-server/src/main.rs:1313-1325; `estimate_generation_performance`,
  icn-hardware/src/lib.rs:1508): bytes per second and launch overhead per tensor type.
* `llama_bench_record`: the result object of the engine's llama-bench style probe
  (inference/crates/icn-engine/src/parity_probe.rs:1352-1424: operation names :53-56, prompt loop
  :1427-1469, generation loop :1471-1504), for a driver that runs the same prompt-processing /
  token-generation schedule over the projections only.
"""
from __future__ import annotations

import statistics
import time

BACKEND_OPS_FIELDS = ("test_time", "build_commit", "backend_name", "op_name", "op_params", "test_mode",
                      "supported", "passed", "error_message", "time_us", "flops", "bandwidth_gb_s",
                      "memory_kb", "n_runs", "device_description", "backend_reg_name")
GGML_TYPE_NAMES = {8: "q8_0", 12: "q4_K", 14: "q6_K"}
MEASUREMENT_UNITS = ("ns", "us", "ms", "s", "tokens/s", "bytes/s", "GB/s", "FLOP/s", "bytes", "count", "ratio")


def mul_mat_params(qtype: int, n_rows: int, m: int, k: int) -> str:
    """op_params of a MUL_MAT case in test-backend-ops' naming: m = weight rows, n = activation rows."""
    return (f"type_a={GGML_TYPE_NAMES[qtype]},type_b=f32,m={n_rows},n={m},k={k},bs=[1,1],nr=[1,1],"
            f"per=[0,1,2,3],k_v=0,o=1")


def mul_mat_id_params(qtype: int, n_rows: int, k: int, n_expert: int, n_used: int, batch: int) -> str:
    return (f"type_a={GGML_TYPE_NAMES[qtype]},type_b=f32,n_mats={n_expert},n_used={n_used},b=0,"
            f"m={n_rows},n={batch},k={k}")


def backend_ops_row(op_name: str, op_params: str, samples_us, flops: float, bytes_moved: float, memory_kb: int,
                    device: str, build_commit: str = "qproj", backend_name: str = "ROCm0",
                    backend_reg_name: str = "qproj-hip", passed: bool = True, error: str = "") -> dict:
    """flops = operations of one run, bytes_moved = algorithmic bytes of one run; time_us is the mean sample."""
    t = statistics.fmean(samples_us)
    return {
        "test_time": time.strftime("%Y-%m-%dT%H:%M:%SZ", time.gmtime()),
        "build_commit": build_commit,
        "backend_name": backend_name,
        "op_name": op_name,
        "op_params": op_params,
        "test_mode": "perf",
        "supported": "1",
        "passed": "1" if passed else "0",
        "error_message": error,
        "time_us": f"{t:.6f}",
        "flops": f"{flops / (t * 1e-6):.6f}",
        "bandwidth_gb_s": f"{bytes_moved / (t * 1e-6) / 1e9:.6f}",
        "memory_kb": str(int(memory_kb)),
        "n_runs": str(len(samples_us)),
        "device_description": device,
        "backend_reg_name": backend_reg_name,
    }


def backend_ops_sql(row: dict) -> str:
    def q(v):
        return "'" + str(v).replace("'", "''") + "'"
    return ("INSERT INTO test_backend_ops (" + ", ".join(BACKEND_OPS_FIELDS) + ") VALUES (" +
            ", ".join(q(row[f]) for f in BACKEND_OPS_FIELDS) + ");")


def measurement(name: str, unit: str, samples) -> dict:
    if unit not in MEASUREMENT_UNITS:
        raise ValueError(f"unit {unit!r} is not one of the evidence schema's units")
    return {"name": name, "unit": unit, "samples": [float(s) for s in samples]}


def calibration_metric(tensor_type: int, routed: bool, bytes_per_launch: float, samples_us, launch_us: float,
                       backend: str = "ROCm", device_id: str = "0") -> dict:
    """bytes_per_second from the median sample; relative_spread = (max - min) / median;
    stable when the spread stays under 10 %."""
    med = statistics.median(samples_us)
    spread = (max(samples_us) - min(samples_us)) / med if med > 0 else 0.0
    return {
        "backend_type": 1,
        "backend": backend,
        "device_id": device_id,
        "tensor_type": int(tensor_type),
        "routed": bool(routed),
        "bytes_per_second": bytes_per_launch / (med * 1e-6),
        "launch_microseconds": float(launch_us),
        "relative_spread": float(spread),
        "sample_count": len(samples_us),
        "measured_microseconds": int(round(sum(samples_us))),
        "stable": bool(spread < 0.10),
    }


LLAMA_BENCH_OPERATIONS = ("llama-bench.prompt-processing", "llama-bench.token-generation",
                          "llama-bench.prompt-generation")


def llama_bench_record(operation: str, prompt_tokens: int, prompt_calls: int, generation_tokens: int,
                       generation_calls: int, durations_ns, effective_configuration: dict, devices,
                       producer: str = "magnitude_amd/projection-only") -> dict:
    """One record per measured case; every repetition keeps its own duration and tokens/s sample
    (the probe measures one repetition per call, a harness collects them)."""
    if operation not in LLAMA_BENCH_OPERATIONS:
        raise ValueError(f"unknown operation {operation!r}")
    durations_ns = [float(d) for d in durations_ns]
    if not durations_ns or min(durations_ns) <= 0:
        raise ValueError("measured duration was zero")
    tokens = int(prompt_tokens) + int(generation_tokens)
    shape_ok = {"llama-bench.prompt-processing": prompt_tokens > 0 and generation_tokens == 0,
                "llama-bench.token-generation": prompt_tokens == 0 and generation_tokens > 0,
                "llama-bench.prompt-generation": prompt_tokens > 0 and generation_tokens > 0}[operation]
    if not shape_ok:
        raise ValueError(f"token counts do not fit {operation}")
    cfg = dict(effective_configuration)
    cfg.setdefault("n_prompt", int(prompt_tokens))
    cfg.setdefault("n_gen", int(generation_tokens))
    return {
        "schemaVersion": 1,
        "output": {
            "operation": operation,
            "measuredPromptTokens": int(prompt_tokens),
            "measuredPromptDecodeCalls": int(prompt_calls),
            "measuredGenerationTokens": int(generation_tokens),
            "measuredGenerationDecodeCalls": int(generation_calls),
            "preparedContextDepthTokens": 0,
            "preparedContextDepthDecodeCalls": 0,
            "measurementRepetitions": len(durations_ns),
            "measuredTokens": tokens,
            "tokenSchedule": "synthetic-activations",   # projections see activations, never token ids
        },
        "measurements": [
            measurement("duration", "ns", durations_ns),
            measurement("tokens_per_second", "tokens/s", [tokens * 1e9 / d for d in durations_ns]),
        ],
        "effectiveConfiguration": cfg,
        "devices": list(devices),
        "producerVersion": producer,
    }
