"""The evidence emitters produce rows the reference's decoders accept in shape: 16 SQL fields in
the pinned order (icn-parity/src/decode.rs:547-564), measurement units from the evidence schema,
calibration entries with the fields of main.rs:1313-1325."""
import re

import pytest

from magnitude_amd import evidence as ev


def test_backend_ops_sql_row_shape():
    row = ev.backend_ops_row("MUL_MAT", ev.mul_mat_params(12, 14336, 1, 4096), [15.0, 16.0, 17.0],
                             flops=2 * 14336 * 4096, bytes_moved=33_100_000, memory_kb=32256, device="MI355X")
    assert tuple(row) == ev.BACKEND_OPS_FIELDS
    sql = ev.backend_ops_sql(row)
    assert sql.startswith("INSERT INTO test_backend_ops (test_time, build_commit, backend_name, op_name,")
    values = re.search(r"VALUES \((.*)\);$", sql).group(1)
    fields = re.findall(r"'((?:[^']|'')*)'", values)
    assert len(fields) == 16
    assert fields[3] == "MUL_MAT" and fields[5] == "perf" and fields[6] == "1" and fields[7] == "1"
    assert float(fields[9]) == pytest.approx(16.0)
    assert float(fields[11]) == pytest.approx(33_100_000 / 16e-6 / 1e9, rel=1e-6)
    assert fields[13] == "3"
    assert "type_a=q4_K,type_b=f32,m=14336,n=1,k=4096" in fields[4]


def test_quotes_are_escaped():
    row = ev.backend_ops_row("MUL_MAT", "x", [1.0], 1, 1, 1, device="AMD 'Instinct'")
    assert "'AMD ''Instinct'''" in ev.backend_ops_sql(row)


def test_measurement_units_follow_the_schema():
    m = ev.measurement("gate_up", "us", [1, 2, 3])
    assert m == {"name": "gate_up", "unit": "us", "samples": [1.0, 2.0, 3.0]}
    with pytest.raises(ValueError):
        ev.measurement("x", "furlongs", [1])


def test_calibration_metric_fields():
    c = ev.calibration_metric(12, False, 66_191_360, [15.0, 15.5, 16.0], launch_us=2.0)
    assert set(c) == {"backend_type", "backend", "device_id", "tensor_type", "routed", "bytes_per_second",
                      "launch_microseconds", "relative_spread", "sample_count", "measured_microseconds", "stable"}
    assert c["bytes_per_second"] == pytest.approx(66_191_360 / 15.5e-6)
    assert c["sample_count"] == 3 and c["stable"] and c["relative_spread"] == pytest.approx(1.0 / 15.5)


def test_llama_bench_record_has_the_probe_result_shape():
    """Field names and nesting of inference/crates/icn-engine/src/parity_probe.rs:1395-1424; one
    duration and one tokens/s sample per repetition, tokens/s = tokens * 1e9 / ns (:1357)."""
    from magnitude_amd import evidence
    rec = evidence.llama_bench_record("llama-bench.prompt-processing", 512, 1, 0, 0, [2.0e6, 4.0e6],
                                      {"batch_size": 512}, [{"name": "gpu"}])
    assert rec["schemaVersion"] == 1
    assert set(rec) == {"schemaVersion", "output", "measurements", "effectiveConfiguration", "devices", "producerVersion"}
    out = rec["output"]
    assert out["operation"] == "llama-bench.prompt-processing"
    assert (out["measuredPromptTokens"], out["measuredPromptDecodeCalls"]) == (512, 1)
    assert (out["measuredGenerationTokens"], out["measuredGenerationDecodeCalls"]) == (0, 0)
    assert out["measuredTokens"] == 512 and out["measurementRepetitions"] == 2
    names = [(m["name"], m["unit"]) for m in rec["measurements"]]
    assert names == [("duration", "ns"), ("tokens_per_second", "tokens/s")]
    assert rec["measurements"][1]["samples"] == [512 * 1e9 / 2.0e6, 512 * 1e9 / 4.0e6]
    assert rec["effectiveConfiguration"]["n_prompt"] == 512 and rec["effectiveConfiguration"]["n_gen"] == 0
    tg = evidence.llama_bench_record("llama-bench.token-generation", 0, 0, 128, 128, [1.0e8], {}, [])
    assert tg["output"]["measuredTokens"] == 128 and tg["measurements"][1]["samples"] == [1280.0]
    with pytest.raises(ValueError):
        evidence.llama_bench_record("llama-bench.token-generation", 512, 1, 0, 0, [1.0], {}, [])   # wrong shape for the operation
    with pytest.raises(ValueError):
        evidence.llama_bench_record("llama-bench.prompt-processing", 512, 1, 0, 0, [0.0], {}, [])  # zero duration
    with pytest.raises(ValueError):
        evidence.llama_bench_record("decode", 1, 1, 0, 0, [1.0], {}, [])
