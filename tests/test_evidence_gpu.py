"""Evidence rows made from measurements of the MI355X itself: the SQL row the reference's backend-ops decoder would
accept (column list and value syntax of the row it holds in its own test, tests/golden/backend_ops_row.sql) and the
fit-calibration entry, with the figures in them consistent with the samples they were made from."""
import math
import os
import sys

import numpy as np
import pytest

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
from test_evidence_cpu import _decode_backend_ops_sql, _golden_row   # the reference decoder's rules, restated


def test_rows_from_a_measured_projection_decode_like_the_reference_sample():
    from magnitude_amd import ACT_GGML, Context, evidence, synth
    from magnitude_amd.qproj import TYPE_Q4_K
    stream = torch.cuda.Stream()
    ctx = Context(0, stream=stream.cuda_stream)
    try:
        n, k = 2048, 4096
        w = ctx.upload_from_device(TYPE_Q4_K, k, n, synth.random_weight(TYPE_Q4_K, n, k, seed=3, device="cuda"))
        x = torch.randn((1, k), device="cuda")
        y = torch.empty((1, n), device="cuda")
        for _ in range(3):
            ctx.mul_mat(w, x, ACT_GGML, out=y, sync=False)
        ctx.sync()
        samples_us = []
        for _ in range(20):
            with torch.cuda.stream(stream):
                a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a.record(stream)
                ctx.mul_mat(w, x, ACT_GGML, out=y, sync=False)
                b.record(stream)
            b.synchronize()
            samples_us.append(a.elapsed_time(b) * 1e3)
        assert all(0.5 < s < 5000 for s in samples_us)
        byts = n * k * 144 // 256 + 4 * (k + n)
        device = torch.cuda.get_device_properties(0).name
        row = evidence.backend_ops_row("MUL_MAT", evidence.mul_mat_params(TYPE_Q4_K, n, 1, k), samples_us,
                                       flops=2.0 * n * k, bytes_moved=byts, memory_kb=byts // 1024, device=device)
        (before, f, time_us, flops, bw), = _decode_backend_ops_sql(evidence.backend_ops_sql(row))
        g_before, g_f, *_ = _decode_backend_ops_sql(_golden_row())[0]
        assert before == g_before and list(f) == list(g_f)
        assert min(samples_us) - 1e-3 <= time_us <= max(samples_us) + 1e-3
        assert math.isclose(time_us, float(np.mean(samples_us)), rel_tol=1e-6, abs_tol=1e-5)
        assert math.isclose(bw, byts / (time_us * 1e-6) / 1e9, rel_tol=1e-4)
        assert math.isclose(flops, 2.0 * n * k / (time_us * 1e-6), rel_tol=1e-4)
        assert 1.0 < bw < 8000.0                       # a memory rate under the HBM peak
        assert f["n_runs"] == "20" and f["device_description"] == device and device.strip()
        assert "type_a=q4_K" in f["op_params"] and f"m={n}" in f["op_params"] and f"k={k}" in f["op_params"]
        cal = evidence.calibration_metric(TYPE_Q4_K, False, byts, samples_us, launch_us=2.0)
        assert cal["sample_count"] == 20 and cal["measured_microseconds"] == int(round(sum(samples_us)))
        assert math.isclose(cal["bytes_per_second"], byts / (float(np.median(samples_us)) * 1e-6), rel_tol=1e-9)
        assert cal["relative_spread"] >= 0.0 and cal["stable"] == (cal["relative_spread"] < 0.10)
        w.free()
    finally:
        ctx.close()
