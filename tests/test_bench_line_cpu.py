"""The last stdout line of bench.py must be one compact JSON object (the driver keeps only a tail of
stdout): every contract field, the roofline and CPU-baseline objects, one headline per leg, under 4 KB
whatever the legs hold; tables and raw samples go to the details file, as the reference keeps raw
samples in evidence files (inference/parity/README.md:110)."""
import json

import bench
from magnitude_amd import evidence


def full_result(nshapes=9, nsamples=400):
    samples = [14.7 + 0.001 * i for i in range(nsamples)]
    per = {k: {"us_per_launch": 6.3123456, "bytes_per_launch": 14196736, "GBps": 2260.123456, "frac_hbm_peak": 0.28251}
           for k in ("qkv", "o", "down")}
    shapes = [{"type": "Q4_K", "M": m, "K": k, "N": n, "gemm_ms": 0.5281234, "quantize_ms": 0.0171234,
               "gemm_tops": 911.6123, "end_to_end_tops": 880.123, "frac_int8_peak": 0.18232}
              for m in (512, 2048, 4096) for (k, n) in ((4096, 14336), (14336, 4096), (4096, 4096))][:nshapes]
    ggml_shapes = shapes + [dict(s, type="Q6_K") for s in shapes[:3]] + [dict(s, type="Q8_0") for s in shapes[:3]]
    cfg = {"scope": "projection operators only"}
    devs = [{"name": "AMD Instinct MI355X", "backend": "ROCm", "index": 0}]
    out = {
        "metric": "Q4_K GEMV achieved HBM GB/s (% peak) + prefill GEMM TOPS, 8B shapes", "value": 3714.123456, "unit": "GB/s",
        "n_gpus": 1, "steps": 20, "warmup": 5, "ms_per_step": 1.19123456, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "int8", "dtype_note": "x" * 200, "data": "synthetic: " + "y" * 100,
        "config": {"workload": "configs[1]: " + "w" * 150, "layers": 32, "act_mode": "ggml", "launches_per_layer": "4 " + "z" * 100,
                   "launch_route": "eager", "hip_graph": False},
        "ms_per_step_by_route": {"eager": 1.19, "hip_graph": 1.23}, "pct_hbm_peak": 46.4265, "tokens_per_s_projection_only": 839.51,
        "bytes_per_step": 4421000000,
        "step_stats": bench.summarize([1.19 + 0.001 * (i % 5) for i in range(20)]),
        "launch_us": bench.summarize([1.77, 1.78, 1.76]),
        "roofline": {"bound": "hbm", "achieved": 4520.123456, "peak": 8000.0, "unit": "GB/s", "frac": 0.565015432,
                     "traffic": 66509926, "traffic_source": "profiles/decode_gate_up_q4k.txt (" + "s" * 80 + ")",
                     "kernel": "gemv_decode_kernel<Q4_K, M=1>: " + "k" * 100, "bytes_per_launch": 66191360,
                     "us_per_launch": 14.6434343, "mad_us": 0.0512345, "rel_mad": 0.0034987, "samples": 30, "launches_timed": 960,
                     "launch_us": 1.7712345, "streaming_probe_us": [11.3, 12.5], "other_kernels": per},
        "verify": {"note": "n", "shapes": [{"M": m, "group": g, "us_per_launch": 20.912345, "us_rows_quantized_earlier": 16.812345,
                                            "GBps": 3200.5, "frac_hbm_peak": 0.4}
                                           for m in (2, 4, 8, 16) for g in ("gate_up", "down")]},
        "q8_0": {"shape": "4096x4096, M=1", "us_per_launch": 6.07123, "GBps": 2940.12, "frac_hbm_peak": 0.3675},
        "norm": {"M=1": {"separate_us": 17.9, "fused_us": 16.2, "fused_swiglu_us": 16.3}},
        "prefill": {"act_format": "per-32", "mfma": "m", "headline_tops": 520.123, "headline_frac_int8_peak": 0.104,
                    "headline_rel_mad": 0.0041234, "samples_per_shape": 30, "bound": "valu", "floor_tops": 704.0,
                    "floor": "5000 x 32 / (16 + 4 x 52.8): 48 of 52.8 vector instr. per matrix instr. are the per-32 flush",
                    "peak_tops": 5000.0, "shapes": shapes},
        "prefill_ggml_acts": {"act_format": "q8k", "mfma": "m" * 200, "headline_tops": 911.6, "headline_frac_int8_peak": 0.1823,
                              "headline_rel_mad": 0.0061234, "samples_per_shape": 30, "shapes": ggml_shapes},
        "moe": {"experts": 128, "batches": [{"B": b, "distinct_experts_mean": 51.5, "calls_in_rotation": 12, "bytes_cycled": 1019215872,
                                             "ms": 0.0551234, "rel_mad": 0.0071234, "GBps": 2581.123, "frac_hbm_peak": 0.32,
                                             "cache_resident": {"ms": 0.05, "GBps": 2800.0, "bytes": 137000000}} for b in (1, 8, 64)],
                "note": "n" * 300},
        "cpu_baseline": {"value": 9.912345, "unit": "GB/s", "cores": 16, "kind": "port", "sample": "s" * 160, "host_cpus": 128,
                         "host_physical_cores": 64, "host_logical_cpus": 128, "thread_policy": "physical-cores, at most the box's 16-CPU share",
                         "rel_mad": 0.0123456, "one_thread_GBps": 0.68123, "isa": "AVX2"},
        "llama_bench": [evidence.llama_bench_record("llama-bench.prompt-processing", 512, 1, 0, 0, [12.3e6] * 5, cfg, devs),
                        evidence.llama_bench_record("llama-bench.token-generation", 0, 0, 128, 128, [157e6] * 5, cfg, devs)],
    }
    row = evidence.backend_ops_row("MUL_MAT", evidence.mul_mat_params(12, 28672, 1, 4096), samples, flops=1.0,
                                   bytes_moved=66191360, memory_kb=64640, device="AMD Instinct MI355X")
    out["evidence"] = {"backend_ops": [row] * 40, "measurements": [evidence.measurement("decode.gate_up.launch", "us", samples)] * 8,
                       "calibration": [evidence.calibration_metric(12, False, 66191360, samples, launch_us=2.0)] * 8}
    return out


def test_final_line_is_compact_and_complete():
    out = full_result()
    assert len(json.dumps(out)) > 30000               # the full record is what broke the driver's parse
    text = bench.compact_line(out, "gpurun_out/bench_details.json")
    assert "\n" not in text and len(text) <= bench.MAX_LINE_BYTES == 4000
    line = json.loads(text)
    for k in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling", "vs_baseline",
              "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert k in line, k
    assert line["value"] == 3714.12 and line["ms_per_step"] == 1.19123 and line["vs_baseline"] is None
    assert "workload" in line["config"] and "model" not in line["config"]
    rf = line["roofline"]
    assert rf["bound"] == "hbm" and rf["peak"] == 8000.0 and rf["unit"] == "GB/s" and rf["traffic"] == 66509926
    assert abs(rf["frac"] - rf["achieved"] / rf["peak"]) < 1e-3
    assert {"kernel", "bytes_per_launch", "us_per_launch", "traffic_source"} <= set(rf)
    cb = line["cpu_baseline"]
    assert {"value", "unit", "cores", "kind", "sample"} <= set(cb) and cb["kind"] == "port"
    assert line["prefill_q8x32"]["headline_tops"] == 520.1 and line["prefill_q8k"]["headline_tops"] == 911.6
    assert line["llama_bench_projections_only"]["pp512_tok_s"] == round(512e9 / 12.3e6)
    assert line["moe_ffn"]["B64"]["us"] == 55.1
    assert "evidence" not in line and line["details"] == "gpurun_out/bench_details.json"
    # the spread of every headline figure rides on the line: median + MAD over raw samples, as the reference's
    # comparator summarizes a measurement (inference/crates/icn-parity/src/compare.rs:727-766)
    vs = line["value_stats"]
    assert vs["n"] == 20 and vs["median_ms"] == 1.192 and vs["mad_ms"] == 0.001 and 0 < vs["rel_mad"] < 0.01
    assert rf["mad_us"] == 0.0512 and rf["rel_mad"] == 0.0035 and rf["samples"] == 30 and rf["launch_us"] == 1.7712
    assert rf["streaming_probe_us"] == [11.3, 12.5]
    assert line["prefill_q8x32"]["rel_mad"] == 0.0041 and line["prefill_q8k"]["rel_mad"] == 0.0061
    assert line["prefill_q8x32"]["samples"] == 30 and line["prefill_q8k"]["samples"] == 30
    # config 4's own format is bounded by the vector ALU: the line says so, with the floor, and keeps frac against 5 POPS
    assert line["prefill_q8x32"]["bound"] == "valu" and line["prefill_q8x32"]["floor_tops"] == 704.0
    assert "floor" in line["prefill_q8x32"] and line["prefill_q8x32"]["peak_tops"] == 5000.0
    assert line["moe_ffn"]["B64"]["rel_mad"] == 0.0071
    assert cb["host_physical_cores"] == 64 and cb["cores"] == 16 and "physical-cores" in cb["thread_policy"] and cb["rel_mad"] == 0.0123
    assert line["verify_us_rows_quantized_earlier"]["M16_down"] == 16.81


def test_final_line_sheds_tables_before_contract_fields():
    out = full_result()
    out["prefill_ggml_acts"]["shapes"] = [dict(s, M=s["M"] + i) for i in range(12)            # an absurdly long table
                                          for s in out["prefill_ggml_acts"]["shapes"]]
    text = bench.compact_line(out)
    line = json.loads(text)
    assert len(text) <= bench.MAX_LINE_BYTES
    assert line["roofline"]["frac"] and line["cpu_baseline"]["value"] and line["value"]
    assert line["prefill_q8k"]["headline_tops"] == 911.6 and "tops" not in line["prefill_q8k"]


def test_summary_statistics_are_the_reference_comparators():
    # median: mean of the two middle samples of an even count; MAD: median of the absolute deviations from it
    assert bench.median([3.0, 1.0, 2.0]) == 2.0 and bench.median([4.0, 1.0, 3.0, 2.0]) == 2.5
    st = bench.summarize([10.0, 12.0, 11.0, 30.0, 9.0])
    assert st == {"median": 11.0, "mad": 1.0, "rel_mad": 1.0 / 11.0, "n": 5}
    assert bench.MIN_SAMPLES >= 30 and bench.MIN_WARMUP >= 5
    phys, logical = bench.physical_cores()
    assert 1 <= phys <= logical


def test_only_the_step_leg():
    out = {k: v for k, v in full_result().items() if k in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step",
                                                          "higher_is_better", "scaling", "vs_baseline", "dtype", "data", "config")}
    line = json.loads(bench.compact_line(out))
    assert line["value"] == 3714.12 and "roofline" not in line


def test_traffic_figure_is_withheld_when_the_kernel_sources_changed(tmp_path, monkeypatch):
    traffic, source = bench.measured_traffic()
    digest = bench.source_digest(*bench.DECODE_KERNEL_SOURCES)
    if traffic is not None:
        assert digest in source
    else:
        assert "stale" in source or "not recorded" in source
    monkeypatch.setattr(bench, "source_digest", lambda *a: "0" * 16)
    traffic, source = bench.measured_traffic()
    assert traffic is None and ("stale" in source or "not recorded" in source)
