"""C-ABI checks that need no GPU: the library loads, exports every declared symbol, and its
argument validation / size arithmetic answers without touching a device."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    from magnitude_amd import qproj
    if not os.path.exists(qproj.LIB_PATH):
        pytest.fail(f"{qproj.LIB_PATH} not built (make -C magnitude_amd/csrc)")
    return qproj.load_library()


def test_every_declared_symbol_is_exported_and_bound(lib):
    from magnitude_amd import qproj
    header = open(os.path.join(ROOT, "include", "qproj.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)  # declarations only, not prose
    declared = set(re.findall(r"\b(qproj_[a-z_0-9]+)\s*\(", header))
    assert declared, "no declarations found"
    assert declared == set(qproj.SYMBOLS), (declared ^ set(qproj.SYMBOLS))
    for name in declared:
        assert getattr(lib, name) is not None


def test_version_and_sizes(lib):
    assert lib.qproj_version().decode().endswith("gfx950")
    assert lib.qproj_row_bytes(8, 4096) == 128 * 34
    assert lib.qproj_row_bytes(12, 4096) == 16 * 144
    assert lib.qproj_row_bytes(14, 14336) == 56 * 210
    assert lib.qproj_row_bytes(12, 4100) == 0
    assert lib.qproj_row_bytes(2, 4096) == 0      # Q4_0 is not a type this path carries
    # activation buffer sizes: planes are 256-byte aligned
    assert lib.qproj_act_bytes(0, 12, 1, 4096) == 4096 + 256 + 512 + 512 + 256   # qs | d | bsums | fp16 min-term plane | row normalisers
    assert lib.qproj_act_bytes(0, 8, 1, 4096) == 4096 + 512
    assert lib.qproj_act_bytes(2, 12, 2, 4096) == 8192 + 1024 + 1024 + 1024 + 256   # qs | d | isum | fp16 min-term plane | row normalisers
    assert lib.qproj_act_bytes(0, 12, 1, 4000) == 0
    assert lib.qproj_act_bytes(1, 12, 1, 4096) == 0  # fp32 activations are not quantized
    # the per-32 format keeps one min-term record per 256 weights of a row: K must be whole super-blocks, or the
    # quantizer would write records the msum plane has no room for
    for k in (32, 288, 4096 + 32):
        assert lib.qproj_act_bytes(2, 12, 1000, k) == 0
        assert lib.qproj_act_bytes(0, 12, 1000, k) == 0
    assert lib.qproj_act_bytes(0, 8, 1, 288) == 512 + 256   # Q8_0 blocks need K % 32 only


def test_null_and_no_device_errors_do_not_crash(lib):
    n = C.c_int(-1)
    rc = lib.qproj_device_count(C.byref(n))
    assert rc in (0, 5)
    assert lib.qproj_device_count(None) == 1
    assert lib.qproj_ctx_create(0, None, None) == 1
    assert lib.qproj_sync(None) == 1
    assert lib.qproj_mul_mat(None, None, None, 1, None, 0) == 1
    assert lib.qproj_last_error(None) == b"null context"
    assert lib.qproj_ctx_destroy(None) == 0
    assert lib.qproj_weight_free(None, None) == 0
    if rc == 5:  # no GPU here: creating a context reports it instead of aborting
        h = C.c_void_p()
        assert lib.qproj_ctx_create(0, None, C.byref(h)) == 5
        assert not h.value


def test_eligibility_probe_answers_in_the_contract_shape(lib):
    """Mirrors cuda_driver.rs inspect() / backend_eligibility.rs cuda(): usable lists one architecture per
    device, absent and failed carry a bounded single-line diagnostic; never crashes without a GPU."""
    from magnitude_amd import qproj
    assert lib.qproj_probe_eligibility(None) == 1
    assert C.sizeof(qproj.Eligibility) == 16 + 16 * 32 + 16 * 256 + 1024 + 244
    r = qproj.probe_eligibility()
    assert r["state"] in ("usable", "absent", "failed")
    n = C.c_int(0)
    rc = lib.qproj_device_count(C.byref(n))
    if r["state"] == "usable":
        assert rc == 0 and n.value >= 1
        # exactly the contract's fields: its deserialiser denies unknown ones (bootstrap_protocol.rs:16-21)
        assert set(r) == {"state", "driverApi", "architectures", "driverLibrary"}
        assert r["driverApi"] > 0 and "gfx950" in r["architectures"]
        hw = qproj.probe_hardware()
        assert len(r["architectures"]) == len(hw["hardwareLabels"]) >= n.value and hw["runtimeApi"] > 0
        assert r["driverLibrary"]
    else:
        assert rc == 5      # whatever keeps the probe from "usable" also keeps contexts from being created
        assert set(r) == {"state", "diagnostic"}
        assert qproj.probe_hardware() == {"runtimeApi": 0, "hardwareLabels": []}
        d = r["diagnostic"]
        assert 0 < len(d) <= 240 and "\n" not in d and "\r" not in d


def test_product_code_never_touches_the_oracle():
    """The shipped package and the benchmark's GPU leg must not import or link the CPU oracle."""
    pkg = os.path.join(ROOT, "magnitude_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp", "Makefile")):
                text = open(os.path.join(dirpath, f), errors="ignore").read()
                assert "oracle" not in text.lower(), os.path.join(dirpath, f)
