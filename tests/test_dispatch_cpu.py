"""The scratch the library reserves for a MUL_MAT covers what the kernel launchers it picks ask for.

qproj_workspace_bytes walks the library's own dispatch (the code that serves qproj_mul_mat_multi) without
launching: every launcher works out its demand from the variables that pick its split and refuses a buffer that is
too small, so a sizing rule and a dispatch rule that disagree show up here, on the CPU, as a non-zero status --
not as a write past a device buffer."""
import itertools

import pytest

from magnitude_amd import qproj

Q8_0, Q4_K, Q6_K = 8, 12, 14
GGML, F32, Q8X32 = 0, 1, 2

MS = [1, 2, 3, 4, 5, 8, 9, 15, 16, 17, 20, 31, 32, 33, 47, 48, 63, 64, 65, 96, 127, 128, 129, 200, 255, 256, 333, 511, 512,
      513, 1000, 1024, 2048, 4096]
KS = [256, 512, 768, 1024, 2048, 3072, 4096, 5120, 6144, 8192, 11008, 14336, 28672]
NS = [(1,), (5,), (32,), (77,), (128,), (256,), (1024,), (4096,), (14336,), (4096, 1024, 1024), (14336, 14336), (768, 768),
      (130, 5), (1024, 1024, 1024, 1024), (32000,)]


@pytest.mark.parametrize("qtype", [Q4_K, Q6_K, Q8_0])
def test_every_launcher_is_satisfied_by_the_reserved_scratch(qtype):
    checked = 0
    for m, k, ns in itertools.product(MS, KS, NS):
        nbytes = qproj.workspace_bytes(qtype, k, ns, m, GGML)       # raises on a launcher that would be refused
        if m <= 2 or (m <= 4 and (k <= 4096 or (qtype == Q8_0 and k <= 20480))):   # (four Q8_0 rows of K <= 20480 fit the kernel's LDS)
            assert nbytes == 0, (m, k, ns)                            # decode regime: the kernel quantizes its own rows
        else:
            assert nbytes >= qproj.load_library().qproj_act_bytes(GGML, qtype, m, k) > 0
        checked += 1
    assert checked == len(MS) * len(KS) * len(NS)


def test_q8_0_rows_of_whole_blocks_only():
    for m, k in itertools.product([1, 3, 16, 17, 64, 100, 512], [32, 96, 288, 1056, 4096 + 32]):
        qproj.workspace_bytes(Q8_0, k, (77,), m, GGML)


def test_per32_and_fp32_modes():
    for m, k, ns in itertools.product([1, 3, 17, 64, 200, 512, 2048], [256, 4096, 14336], [(4096,), (14336,), (130,)]):
        nbytes = qproj.workspace_bytes(Q4_K, k, ns, m, Q8X32)
        assert nbytes >= qproj.load_library().qproj_act_bytes(Q8X32, Q4_K, m, k)
        assert qproj.workspace_bytes(Q4_K, k, ns, m, F32) == 0
    with pytest.raises(qproj.QprojError):
        qproj.workspace_bytes(Q6_K, 4096, (4096,), 64, Q8X32)        # the per-32 path is built for Q4_K weights


def test_known_sizes():
    al = lambda v: (v + 255) // 256 * 256
    planes = lambda m, k: al(m * k) + al(m * (k // 256) * 4) + al(m * (k // 16) * 2) + al(m * (k // 256) * 32) + al(m * 4)
    # down projection of the 8B layer at 512 tokens: 64 tiles of 128 tokens x 256 rows for 256 compute units, K is cut in four
    assert qproj.workspace_bytes(Q6_K, 14336, (4096,), 512, GGML) == planes(512, 14336) + 4 * 512 * 4096 * 4
    # gate/up at 4096 tokens: the grid is full, nothing beyond the activation planes
    assert qproj.workspace_bytes(Q4_K, 4096, (14336, 14336), 4096, GGML) == planes(4096, 4096)
    # small batch, K = 14336 at 16 rows: per-chunk results of the small-batch kernel
    assert qproj.workspace_bytes(Q6_K, 14336, (4096,), 16, GGML) > planes(16, 14336)


def test_bad_shapes_are_refused():
    lib = qproj.load_library()
    import ctypes as C
    st = C.c_int(0)
    arr = (C.c_int64 * 1)(4096)
    assert lib.qproj_workspace_bytes(Q4_K, 4100, 1, arr, 4, GGML, C.byref(st)) == 0 and st.value == 1
    assert lib.qproj_workspace_bytes(2, 4096, 1, arr, 4, GGML, C.byref(st)) == 0 and st.value == 1
    assert lib.qproj_workspace_bytes(Q4_K, 4096, 5, arr, 4, GGML, C.byref(st)) == 0 and st.value == 1
    assert lib.qproj_workspace_bytes(Q4_K, 4096, 1, None, 4, GGML, None) == 0


def test_the_8b_layer_fits_the_fixed_scratch_up_to_512_tokens():
    """The allocation-free entry point keeps its scratch in a fixed 64 MiB buffer: every projection group of the
    8B-class layer must fit for the batches the engine issues (n_batch 512,
    /root/reference/inference/crates/icn-engine/src/lib.rs:93-96)."""
    groups = [(Q4_K, 4096, (4096, 1024, 1024)), (Q4_K, 4096, (4096,)), (Q4_K, 4096, (14336, 14336)), (Q6_K, 14336, (4096,))]
    for m in (1, 2, 4, 8, 16, 64, 128, 512):
        for qt, k, ns in groups:
            assert qproj.workspace_bytes(qt, k, ns, m, GGML) <= qproj.NOALLOC_SCRATCH_BYTES, (m, qt, k, ns)
    assert qproj.workspace_bytes(Q6_K, 14336, (4096,), 4096, GGML) > qproj.NOALLOC_SCRATCH_BYTES   # and larger ones are refused


# ---------------------------------------------------------------------------------------------------------------
# The routing table: which kernel, tile, grid and cuts of K serve every shape of the benchmark configurations.  The
# lines are written by the launchers themselves in a dry run of the dispatch (qproj_plan_mul_mat / qproj_plan_moe_ffn),
# so an edit of a routing threshold shows up as a diff of tests/golden/dispatch_plan.txt.
# Regenerate after a deliberate change with:  QPROJ_UPDATE_PLAN=1 python -m pytest tests/test_dispatch_cpu.py -k routing_table
def routing_table() -> str:
    out = []

    def dense(title, qtype, k, ns, m, act=GGML, with_norm=False):
        out.append(f"## {title}: {'Q8_0' if qtype == Q8_0 else 'Q4_K' if qtype == Q4_K else 'Q6_K'} K={k} N={list(ns)} M={m} "
                   f"act={'ggml' if act == GGML else 'f32' if act == F32 else 'q8x32'}{' +rms_norm' if with_norm else ''}")
        out.append(qproj.plan_mul_mat(qtype, k, ns, m, act, with_norm).rstrip())

    layer = [("q/k/v", Q4_K, 4096, (4096, 1024, 1024)), ("o", Q4_K, 4096, (4096,)), ("gate/up", Q4_K, 4096, (14336, 14336)),
             ("down", Q6_K, 14336, (4096,))]
    dense("config 1", Q8_0, 4096, (4096,), 1)
    for name, qt, k, ns in layer:
        dense(f"config 2 {name}", qt, k, ns, 1)
    dense("config 2 norm + q/k/v", Q4_K, 4096, (4096, 1024, 1024), 1, with_norm=True)
    dense("config 2 norm + gate/up", Q4_K, 4096, (14336, 14336), 1, with_norm=True)
    for m in (2, 4, 8, 16):
        for name, qt, k, ns in layer:
            dense(f"config 3 {name}", qt, k, ns, m)
    for m in (512, 2048, 4096):
        for k, n in ((4096, 14336), (14336, 4096), (4096, 4096)):
            dense("config 4 (per-32 activations)", Q4_K, k, (n,), m, Q8X32)
            dense("config 4 (ggml activations)", Q4_K, k, (n,), m)
        dense("config 4 (ggml activations) down", Q6_K, 14336, (4096,), m)
        dense("config 4 (ggml activations) config 1's matrix", Q8_0, 4096, (4096,), m)
    for name, qt, k, ns in layer:
        dense(f"prompt batch of the engine (512 tokens) {name}", qt, k, ns, 512)
    for b in (1, 8, 64):
        out.append(f"## config 5: 128 experts, top-8, d_model 2048, d_ff 768, Q4_K, B={b}")
        out.append(qproj.plan_moe_ffn(Q4_K, Q4_K, 2048, 768, 128, 8, b).rstrip())
    return "\n".join(out) + "\n"


def test_routing_table_of_the_benchmark_configurations_is_pinned():
    import os
    path = os.path.join(os.path.dirname(__file__), "golden", "dispatch_plan.txt")
    table = routing_table()
    if os.environ.get("QPROJ_UPDATE_PLAN"):
        with open(path, "w") as f:
            f.write(table)
    with open(path) as f:
        pinned = f.read()
    assert table == pinned, "the dispatch changed: review the diff, then regenerate tests/golden/dispatch_plan.txt"
    # every shape is served (no refusal) and the decode regime stays one launch
    assert "refused" not in table
    first = table.split("## config 2 q/k/v")[1].split("##")[0]
    assert first.count("gemv_decode_kernel") == 1 and "quantizer:" not in first


def test_plan_reports_a_refused_call():
    with pytest.raises(qproj.QprojError):
        qproj.plan_mul_mat(Q6_K, 4096, (4096,), 64, Q8X32)
