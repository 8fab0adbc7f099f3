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


# ---------------------------------------------------------------- against the reference-held sample row

def _decode_backend_ops_sql(text):
    """The reference decoder's rules for `test-backend-ops perf --output sql` rows, restated
    (icn-parity/src/decode.rs:542-640 and the value parser at :731-762): lines starting with the INSERT prefix,
    values single-quoted with '' as the escape, exactly 16 of them in the pinned field order, test_mode perf, a
    resolved tool / backend identity, booleans as 1/0/true/false, numeric fields that parse, and a supported row
    with passed, a finite positive time and n_runs > 0."""
    import math
    rows = []
    for line in text.splitlines():
        if not line.startswith("INSERT INTO test_backend_ops"):
            continue
        before, sep, suffix = line.partition("VALUES (")
        assert sep and suffix.endswith(");"), "malformed backend-ops SQL INSERT"
        body, values, i = suffix[:-2], [], 0
        while True:
            while i < len(body) and (body[i].isspace() or body[i] == ","):
                i += 1
            if i >= len(body):
                break
            assert body[i] == "'", "backend-ops SQL values must be single-quoted"
            i += 1
            value = ""
            while True:
                assert i < len(body), "unterminated backend-ops SQL value"
                if body[i] == "'" and i + 1 < len(body) and body[i + 1] == "'":
                    value += "'"
                    i += 2
                elif body[i] == "'":
                    i += 1
                    break
                else:
                    value += body[i]
                    i += 1
            values.append(value)
        assert len(values) == 16
        f = dict(zip(ev.BACKEND_OPS_FIELDS, values))
        assert f["test_mode"] == "perf"
        assert f["build_commit"].strip() and f["backend_name"].strip()
        assert f["backend_name"].lower() not in ("unknown", "auto")
        as_bool = {"1": True, "true": True, "0": False, "false": False}
        supported, passed = as_bool[f["supported"]], as_bool[f["passed"]]
        time_us, flops, bw = float(f["time_us"]), float(f["flops"]), float(f["bandwidth_gb_s"])
        memory_kb, n_runs = int(f["memory_kb"]), int(f["n_runs"])
        assert memory_kb >= 0 and n_runs >= 0 and "-" not in f["memory_kb"] + f["n_runs"]      # u64 in the reference
        if supported:
            assert passed and math.isfinite(time_us) and time_us > 0.0 and n_runs > 0
        rows.append((before, f, time_us, flops, bw))
    assert rows, "backend-ops SQL contains no result rows"
    return rows


def _golden_row():
    import os
    return open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "backend_ops_row.sql")).read()


def test_the_reference_held_sample_row_decodes():
    (before, f, time_us, flops, bw), = _decode_backend_ops_sql(_golden_row())
    assert f["op_name"] == "SOFT_MAX" and f["backend_name"] == "MTL0" and f["build_commit"] == "9e3b928fd"
    assert (time_us, flops, bw) == (222.961055, 0.0, 2.737648)
    assert f["device_description"] == "" and f["backend_reg_name"] == ""


def test_emitted_rows_have_the_sample_rows_column_list_quoting_and_value_syntax():
    golden = _golden_row().strip()
    g_before, g_f, *_ = _decode_backend_ops_sql(golden)[0]
    rows = [ev.backend_ops_row("MUL_MAT", ev.mul_mat_params(12, 28672, 1, 4096), [14.6, 14.7, 14.9], flops=2.0 * 28672 * 4096,
                               bytes_moved=66_191_360, memory_kb=64640, device="AMD Instinct MI355X"),
            ev.backend_ops_row("MUL_MAT_ID", ev.mul_mat_id_params(12, 768, 2048, 128, 8, 64), [114.0], flops=1.0,
                               bytes_moved=334e6, memory_kb=326000, device="it's a 'quoted' name")]
    text = "\n".join(ev.backend_ops_sql(r) for r in rows)
    decoded = _decode_backend_ops_sql(text)
    assert len(decoded) == 2
    for (before, f, time_us, flops, bw), row in zip(decoded, rows):
        assert before == g_before                                   # the statement up to VALUES, byte for byte
        assert list(f) == list(g_f) == list(ev.BACKEND_OPS_FIELDS)
        assert f["device_description"] == row["device_description"]  # the '' escape round-trips
        # the same value syntax as the sample: fixed notation with six decimals, integers bare, booleans 1/0
        for key in ("time_us", "flops", "bandwidth_gb_s"):
            assert re.fullmatch(r"\d+\.\d{6}", f[key]) and re.fullmatch(r"\d+\.\d{6}", g_f[key])
        for key in ("memory_kb", "n_runs"):
            assert re.fullmatch(r"\d+", f[key]) and re.fullmatch(r"\d+", g_f[key])
        assert f["supported"] == g_f["supported"] == "1" and f["passed"] == "1"
        assert re.fullmatch(r"\d{4}-\d\d-\d\dT\d\d:\d\d:\d\dZ", f["test_time"]) and re.fullmatch(r"\d{4}-\d\d-\d\dT\d\d:\d\d:\d\dZ", g_f["test_time"])
    assert text.endswith(");") and golden.endswith(");")
