"""GPU parity: the HIP kernels behind the C ABI against the CPU oracle on identical seeded inputs.

Bars: dequantized weights and quantized activations bit-exact; fp32 outputs of the
quantized-activation modes against the oracle in the same mode within 2e-5 (the integer partial
sums are exact on both sides, only the fp32 association differs -- ggml's own SIMD paths differ
from its scalar path in the same way); fp32-activation mode against the fp64 dot within 1e-4.
Both are far inside the stated gate (max relative error 1e-3, max abs 1e-2 where |y| < 1),
which is asserted as well.
"""
import numpy as np
import pytest
import torch

from kquant_encoders import encode

pytestmark = pytest.mark.gpu

Q8_0, Q4_K, Q6_K = 8, 12, 14
TYPES = [Q8_0, Q4_K, Q6_K]


@pytest.fixture(scope="module")
def ctx():
    from magnitude_amd import Context
    assert torch.cuda.is_available(), "these tests need the MI355X"
    c = Context(0)
    yield c
    c.close()


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def gate(got, want):
    """north-star gate: rel <= 1e-3 where |y| >= 1, abs <= 1e-2 where |y| < 1"""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    big = np.abs(want) >= 1
    if big.any():
        assert np.max(np.abs(got[big] - want[big]) / np.abs(want[big])) <= 1e-3
    if (~big).any():
        assert np.max(np.abs(got[~big] - want[~big])) <= 1e-2


def close(got, want, tol):
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    err = np.abs(got - want) / np.maximum(1.0, np.abs(want))
    assert err.max() <= tol, f"max scaled error {err.max():.3e} at {np.unravel_index(err.argmax(), err.shape)}"


def finite_halves(rng, n):
    h = rng.integers(0, 65536, n).astype(np.uint16)
    h[(h & 0x7c00) == 0x7c00] &= 0xbfff
    return h.view(np.uint8).reshape(n, 2)


def random_blocks(rng, qtype, nb):
    size = {Q8_0: 34, Q4_K: 144, Q6_K: 210}[qtype]
    b = rng.integers(0, 256, (nb, size), dtype=np.uint8)
    if qtype == Q8_0:
        b[:, 0:2] = finite_halves(rng, nb)
    elif qtype == Q4_K:
        b[:, 0:2] = finite_halves(rng, nb)
        b[:, 2:4] = finite_halves(rng, nb)
    else:
        b[:, 208:210] = finite_halves(rng, nb)
    return b


_weight_cache = {}


def make_weight(orc, qtype, n, k, seed):
    key = (qtype, n, k, seed)
    if key not in _weight_cache:
        _weight_cache[key] = _make_weight(orc, qtype, n, k, seed)
    return _weight_cache[key]


def _make_weight(orc, qtype, n, k, seed):
    rng = np.random.default_rng(seed)
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    return encode(qtype, w)


# ---------------------------------------------------------------- dequantize / upload

@pytest.mark.parametrize("qtype", TYPES)
def test_dequantize_bit_exact_random_byte_patterns(ctx, orc, qtype):
    """Arbitrary bytes (every scale/min/nibble combination, fp16 subnormals included)."""
    rng = np.random.default_rng(40 + qtype)
    rows, bpr = 64, {Q8_0: 128, Q4_K: 16, Q6_K: 16}[qtype]
    k = bpr * orc.BLOCK_ELEMS[qtype]
    blocks = random_blocks(rng, qtype, rows * bpr).reshape(rows, -1)
    w = ctx.upload(qtype, k, rows, blocks)
    got = ctx.dequantize(w).cpu().numpy()
    want = orc.dequantize(qtype, blocks, k)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert np.array_equal(ctx.download(w), blocks.reshape(-1))


@pytest.mark.parametrize("qtype", TYPES)
def test_dequantize_bit_exact_quantizer_output(ctx, orc, qtype):
    blocks = make_weight(orc, qtype, 96, 2048, seed=qtype)
    w = ctx.upload(qtype, 2048, 96, blocks)
    got = ctx.dequantize(w).cpu().numpy()
    assert np.array_equal(got.view(np.uint32), orc.dequantize(qtype, blocks, 2048).view(np.uint32))


def test_eligibility_probe_reports_the_gfx950_device(ctx):
    """On a box with the GPU the probe is "usable", names the architecture the library is built for and
    agrees with torch about the device."""
    from magnitude_amd import qproj
    r = qproj.probe_eligibility()
    assert r["state"] == "usable", r
    assert set(r) == {"state", "driverApi", "architectures", "driverLibrary"}   # the contract denies unknown fields
    hw = qproj.probe_hardware()
    assert r["driverApi"] > 0 and hw["runtimeApi"] > 0
    assert r["architectures"][0] == "gfx950"
    assert len(r["architectures"]) == len(hw["hardwareLabels"]) == torch.cuda.device_count()
    assert hw["hardwareLabels"][0].strip() == hw["hardwareLabels"][0] != ""
    assert "amdhip64" in r["driverLibrary"]


def test_upload_rejects_bad_arguments(ctx, orc):
    from magnitude_amd import QprojError
    blocks = make_weight(orc, Q4_K, 4, 256, seed=1)
    with pytest.raises(ValueError):
        ctx.upload(Q4_K, 256, 5, blocks)            # byte count does not match
    with pytest.raises((ValueError, QprojError)):
        ctx.upload(2, 256, 4, blocks)               # Q4_0: not carried by this path
    with pytest.raises((ValueError, QprojError)):
        ctx.upload(Q4_K, 100, 4, blocks)


def test_empty_batches_are_accepted_and_touch_nothing(ctx, orc):
    """A scheduler step may carry no rows for a layer (ggml computes a MUL_MAT with ne1 = 0 as a no-op): M = 0 and
    B = 0 return success without writing; negative counts are refused."""
    import ctypes as C
    from magnitude_amd import ACT_GGML
    QPROJ_ERR_INVALID_ARG = 1   # include/qproj.h
    k, n, e = 256, 64, 4
    w = ctx.upload(Q4_K, k, n, make_weight(orc, Q4_K, n, k, seed=3))
    we = ctx.upload(Q4_K, k, n, make_weight(orc, Q4_K, n * e, k, seed=4), n_expert=e)
    x = torch.ones((4, k), device="cuda")
    y = torch.full((4, n), 7.0, device="cuda")
    ids = torch.zeros((4, 2), dtype=torch.int32, device="cuda")
    wa = (C.c_void_p * 1)(w.handle)
    ya = (C.c_void_p * 1)(y.data_ptr())
    lib, h = ctx.lib, ctx.handle
    assert lib.qproj_mul_mat(h, w.handle, x.data_ptr(), 0, y.data_ptr(), ACT_GGML) == 0
    assert lib.qproj_mul_mat_multi(h, 1, wa, x.data_ptr(), 0, ya, ACT_GGML) == 0
    assert lib.qproj_mul_mat_id(h, we.handle, x.data_ptr(), 1, ids.data_ptr(), 2, 0, y.data_ptr(), ACT_GGML) == 0
    ctx.sync()
    assert bool((y == 7.0).all())
    assert lib.qproj_mul_mat(h, w.handle, x.data_ptr(), -1, y.data_ptr(), ACT_GGML) == QPROJ_ERR_INVALID_ARG
    assert lib.qproj_mul_mat_id(h, we.handle, x.data_ptr(), 1, ids.data_ptr(), 2, -1, y.data_ptr(), ACT_GGML) == QPROJ_ERR_INVALID_ARG
    assert bool((y == 7.0).all())
    w.free()
    we.free()


# ---------------------------------------------------------------- activation quantizers

def activation_cases(rng, m, k):
    x = rng.standard_normal((m, k)).astype(np.float32)
    x[0, 0:256] = 0.0                       # zero super-block
    x[0, 300] = 3.0
    x[0, 310] = -3.0                        # tie in magnitude: the first one wins
    x[-1, 5] *= 20.0                        # outlier channel
    x[-1, 512:544] = np.float32(1e-30)      # tiny block
    x[1 % m, 64:96] = 0.5                   # constant block: exact .5 quotients for roundf
    return x


# 128 rows and more take the one-launch route (a workgroup per row writes codes, sums and the min-term plane);
# fewer rows the quantizer launch followed by the min-term launch: the same bytes either way
@pytest.mark.parametrize("m,k", [(5, 2048), (131, 6144)])
def test_quantize_q8_K_bit_exact(ctx, orc, m, k):
    from magnitude_amd import ACT_GGML
    rng = np.random.default_rng(50)
    x = activation_cases(rng, m, k)
    got = ctx.quantize_activations(dev(x), ACT_GGML, Q4_K)
    raw = orc.quantize_q8_K(x).reshape(m, k // 256, 292)
    want_d = raw[:, :, 0:4].copy().view(np.float32)[:, :, 0]
    want_q = raw[:, :, 4:260].view(np.int8).reshape(m, k)
    want_b = raw[:, :, 260:292].copy().view(np.int16).reshape(m, k // 16)
    assert np.array_equal(got["qs"].cpu().numpy(), want_q)
    assert np.array_equal(got["d"].cpu().numpy().view(np.uint32), want_d.view(np.uint32))
    assert np.array_equal(got["bsums"].cpu().numpy(), want_b)
    # the tiled kernels' extra planes: rs = the largest power of two not above the row's largest d (1 for a zero
    # row), and (d / rs) * (sum of each 32 codes) / 16 as an fp16 high part and the fp16 of what the high part leaves
    # (numpy's float16 rounds to nearest even like the device)
    dmax = np.abs(want_d).max(axis=1)       # a Q8_K scale carries a sign
    rs = np.where(dmax > 0, np.float32(2.0) ** np.floor(np.log2(np.maximum(dmax, np.float32(1e-37)))), np.float32(1.0)).astype(np.float32)
    assert np.array_equal(got["rs"].cpu().numpy().view(np.uint32), rs.view(np.uint32))
    v = (want_d / rs[:, None])[:, :, None] * want_b.reshape(m, k // 256, 8, 2).sum(-1).astype(np.float32) * np.float32(0.0625)
    hi = v.astype(np.float16)
    lo = (v - hi.astype(np.float32)).astype(np.float16)
    ms = got["msum"].cpu().numpy()
    assert np.array_equal(ms[:, :, 0], hi)      # as values: a zero sum under a negative scale may come as +0 or -0
    assert np.array_equal(ms[:, :, 1], lo)


def test_quantize_q8_0_activations_bit_exact(ctx, orc):
    from magnitude_amd import ACT_GGML
    rng = np.random.default_rng(51)
    m, k = 3, 1056  # not a multiple of 256: rows straddle the 256-element wave chunks
    x = activation_cases(rng, m, k)
    got = ctx.quantize_activations(dev(x), ACT_GGML, Q8_0)
    raw = orc.quantize_q8_0_act(x).reshape(m, k // 32, 34)
    want_d = raw[:, :, 0:2].copy().view(np.float16)[:, :, 0].astype(np.float32)
    want_q = raw[:, :, 2:].view(np.int8).reshape(m, k)
    assert np.array_equal(got["qs"].cpu().numpy(), want_q)
    assert np.array_equal(got["d"].cpu().numpy().view(np.uint32), want_d.view(np.uint32))


@pytest.mark.parametrize("m,k", [(7, 1024), (129, 4608), (2, 200704)])   # the last: too long a row for the one-launch route
def test_quantize_q8x32_bit_exact(ctx, orc, m, k):
    from magnitude_amd import ACT_Q8X32
    rng = np.random.default_rng(52)
    x = activation_cases(rng, m, k)
    got = ctx.quantize_activations(dev(x), ACT_Q8X32, Q4_K)
    raw = orc.quantize_q8x32(x).reshape(m, k // 32, 40)
    assert np.array_equal(got["qs"].cpu().numpy(), raw[:, :, 8:].view(np.int8).reshape(m, k))
    assert np.array_equal(got["d"].cpu().numpy().view(np.uint32), raw[:, :, 0:4].copy().view(np.uint32)[:, :, 0])
    assert np.array_equal(got["isum"].cpu().numpy(), raw[:, :, 4:8].copy().view(np.int32)[:, :, 0])
    # the prefill kernel's extra planes: rs (power of two under the row's largest d) and (d / rs) * isum / 16 as an
    # fp16 high part and the fp16 of the rest
    d32 = raw[:, :, 0:4].copy().view(np.float32)[:, :, 0]
    dmax = d32.max(axis=1)
    rs = np.where(dmax > 0, np.float32(2.0) ** np.floor(np.log2(np.maximum(dmax, np.float32(1e-37)))), np.float32(1.0)).astype(np.float32)
    assert np.array_equal(got["rs"].cpu().numpy().view(np.uint32), rs.view(np.uint32))
    v = (d32 / rs[:, None]) * raw[:, :, 4:8].copy().view(np.int32)[:, :, 0].astype(np.float32) * np.float32(0.0625)
    hi = v.astype(np.float16)
    lo = (v - hi.astype(np.float32)).astype(np.float16)
    ms = got["msum"].cpu().numpy()
    assert np.array_equal(ms[:, :, 0], hi.reshape(m, k // 256, 8))
    assert np.array_equal(ms[:, :, 1], lo.reshape(m, k // 256, 8))


def test_quantize_q8x32_rejects_rows_that_are_not_whole_super_blocks(ctx):
    """The per-32 format keeps one min-term record per 256 weights of a row; with K % 256 != 0 the quantizer
    would write records the msum plane has no room for, so the ABI refuses before anything is launched."""
    from magnitude_amd import ACT_Q8X32
    for m, k in ((1000, 32), (3, 288)):
        assert ctx.lib.qproj_act_bytes(ACT_Q8X32, Q4_K, m, k) == 0
        x = torch.zeros((m, k), device="cuda")
        buf = torch.empty(m * k * 4 + 4096, dtype=torch.uint8, device="cuda")
        rc = ctx.lib.qproj_quantize_activations(ctx.handle, ACT_Q8X32, Q4_K, x.data_ptr(), m, k, buf.data_ptr())
        assert rc == 1                      # QPROJ_ERR_INVALID_ARG
        assert b"shape" in ctx.lib.qproj_last_error(ctx.handle)


# ---------------------------------------------------------------- mul_mat, decode and small M

SHAPES = {  # (K, N): 8B-layer K values at reduced N, plus ragged row counts and a short K
    Q8_0: [(4096, 384), (1056, 77)],
    Q4_K: [(4096, 512), (14336, 64), (768, 203), (256, 9)],
    Q6_K: [(14336, 256), (4096, 130), (256, 5)],
}


@pytest.mark.parametrize("qtype", TYPES)
@pytest.mark.parametrize("m", [1, 2, 3, 4, 8, 16, 19])
def test_mul_mat_ggml_mode_matches_oracle(ctx, orc, qtype, m):
    from magnitude_amd import ACT_GGML
    for (k, n) in SHAPES[qtype]:
        blocks = make_weight(orc, qtype, n, k, seed=1000 + k + n)
        rng = np.random.default_rng(m * 7 + k)
        x = rng.standard_normal((m, k)).astype(np.float32)
        w = ctx.upload(qtype, k, n, blocks)
        got = ctx.mul_mat(w, dev(x), ACT_GGML).cpu().numpy()
        want = orc.mul_mat(qtype, blocks, k, x, orc.ACT_GGML)
        close(got, want, 2e-5)
        gate(got, want)
        w.free()


@pytest.mark.parametrize("qtype,k,ns", [(Q4_K, 4096, (4097,)), (Q4_K, 2048, (3001, 1000)), (Q6_K, 2048, (3000,)),
                                        (Q8_0, 4096, (5000,)), (Q4_K, 4096, (6143, 6145))])
def test_small_batch_row_groups_of_fewer_than_32_rows(ctx, orc, qtype, k, ns):
    """A grid of the small-batch kernel that would leave compute units without a workgroup is evened out with row
    groups of 24..31 rows (the spare columns of the matrix instruction repeat a row and are not stored).  Shapes whose
    plan says so, with ragged last groups and two matrices in one launch, against the oracle; rows past the end of a
    matrix stay untouched."""
    import re
    from magnitude_amd import ACT_GGML, qproj
    for m in (5, 8, 16, 27):
        plan = qproj.plan_mul_mat(qtype, k, list(ns), m, ACT_GGML)
        rows = [int(r) for r in re.findall(r"row group(?:\(s\))? of (\d+) rows", plan)]
        assert rows and all(24 <= r < 32 for r in rows), plan
        ws, blocks = [], []
        for i, n in enumerate(ns):
            blocks.append(make_weight(orc, qtype, n, k, seed=2400 + k + n + i))
            ws.append(ctx.upload(qtype, k, n, blocks[-1]))
        rng = np.random.default_rng(m + k + ns[0])
        x = rng.standard_normal((m, k)).astype(np.float32)
        # outputs inside larger buffers: what lies behind them must not change
        bufs = [torch.full((m * n + 64,), 7.0, dtype=torch.float32, device="cuda") for n in ns]
        outs = [b[: m * n].view(m, n) for b, n in zip(bufs, ns)]
        ctx.mul_mat_multi(ws, dev(x), ACT_GGML, outs=outs)
        for b, o, n, blk in zip(bufs, outs, ns, blocks):
            want = orc.mul_mat(qtype, blk, k, x, orc.ACT_GGML)
            close(o.cpu().numpy(), want, 2e-5)
            assert bool((b[m * n:] == 7.0).all())
        for w in ws:
            w.free()


@pytest.mark.parametrize("qtype,k,n", [(Q4_K, 4096, 512), (Q4_K, 14336, 203), (Q4_K, 256, 9), (Q8_0, 4096, 384),
                                       (Q8_0, 14336, 77), (Q6_K, 4096, 130), (Q6_K, 14336, 256)])
def test_rows_17_to_32_on_the_small_batch_kernel(ctx, orc, qtype, k, n):
    """Between the 16 rows of a verify batch and the tiled kernels: 17..32 rows take ONE pass of 32 rows of the
    small-batch matrix-core kernel - every token row of the matrix instruction carries a row of its own, K is
    staged in shorter chunks (two chunks add themselves to the cleared output).  Against the oracle, and a row's
    result does not depend on how many rows ride along in the pass (bitwise); the first tiled row counts beyond
    ride along against the oracle."""
    from magnitude_amd import ACT_GGML
    blocks = make_weight(orc, qtype, n, k, seed=1700 + k + n)
    w = ctx.upload(qtype, k, n, blocks)
    rng = np.random.default_rng(k + n)
    x = rng.standard_normal((63, k)).astype(np.float32)
    x[:, rng.integers(0, k, 4)] *= 20.0
    want = orc.mul_mat(qtype, blocks, k, x, orc.ACT_GGML)
    got32 = ctx.mul_mat(w, dev(x[:32]), ACT_GGML).cpu().numpy()
    for m in (17, 25, 31, 32, 33, 47, 63):
        got = ctx.mul_mat(w, dev(x[:m]), ACT_GGML).cpu().numpy()
        close(got, want[:m], 2e-5)
        gate(got, want[:m])
        if m <= 32:
            assert np.array_equal(got, got32[:m]), m
    w.free()


@pytest.mark.parametrize("qtype", [Q4_K, Q6_K, Q8_0])
@pytest.mark.parametrize("m,k,n", [(48, 4096, 256), (130, 768, 203), (200, 14336, 128), (333, 256, 40)])
def test_mul_mat_ggml_mode_prefill_sized_batches(ctx, orc, qtype, m, k, n):
    """Large M in the ggml activation format: the prefill matrix-core kernels (Q4_K: two int8 chains
    per super-block; Q6_K: one K=16 product per sub-block, integer scale on the vector ALU; Q8_0: one
    product per block of 32, both scales applied in fp32) against the oracle's integer arithmetic
    with ggml's activation blocks, ragged M and N included."""
    from magnitude_amd import ACT_GGML
    blocks = make_weight(orc, qtype, n, k, seed=1500 + k + n)
    rng = np.random.default_rng(m + k)
    x = rng.standard_normal((m, k)).astype(np.float32)
    x[:, rng.integers(0, k, 8)] *= 30.0          # outlier channels, as transformer activations have
    w = ctx.upload(qtype, k, n, blocks)
    got = ctx.mul_mat(w, dev(x), ACT_GGML).cpu().numpy()
    want = orc.mul_mat(qtype, blocks, k, x, orc.ACT_GGML)
    close(got, want, 2e-5)
    gate(got, want)
    # a row of the big batch is the small-batch kernel's row up to fp32 summation order
    few = ctx.mul_mat(w, dev(x[:5]), ACT_GGML).cpu().numpy()
    close(got[:5], few, 2e-5)
    w.free()


@pytest.mark.parametrize("m,k,n", [(1000, 256, 6200), (900, 768, 6200)])
def test_mul_mat_ggml_mode_q4k_wide_tiles(ctx, orc, m, k, n):
    """Q4_K with enough 128-token x 256-row tiles (>= 192) to take the wide prefill kernel: one and three
    super-blocks of K (the late-converting waves prepare a next super-block that does not exist after the
    last), a ragged last token tile and a last column tile in which six of the eight waves have no rows."""
    from magnitude_amd import ACT_GGML
    blocks = make_weight(orc, Q4_K, n, k, seed=1700 + k + n)
    rng = np.random.default_rng(m + k)
    x = rng.standard_normal((m, k)).astype(np.float32)
    x[:, rng.integers(0, k, 8)] *= 30.0
    w = ctx.upload(Q4_K, k, n, blocks)
    got = ctx.mul_mat(w, dev(x), ACT_GGML).cpu().numpy()
    want = orc.mul_mat(Q4_K, blocks, k, x, orc.ACT_GGML)
    close(got, want, 2e-5)
    gate(got, want)
    w.free()


@pytest.mark.parametrize("qtype", TYPES)
@pytest.mark.parametrize("m", [1, 3, 4, 6])
def test_mul_mat_f32_mode_matches_fp64_dot(ctx, orc, qtype, m):
    from magnitude_amd import ACT_F32
    for (k, n) in SHAPES[qtype]:
        blocks = make_weight(orc, qtype, n, k, seed=2000 + k + n)
        rng = np.random.default_rng(m * 11 + k)
        x = rng.standard_normal((m, k)).astype(np.float32)
        w = ctx.upload(qtype, k, n, blocks)
        got = ctx.mul_mat(w, dev(x), ACT_F32).cpu().numpy()
        want = orc.mul_mat_f64(qtype, blocks, k, x)
        close(got, want, 1e-4)
        gate(got, want)
        w.free()


@pytest.mark.parametrize("qtype", TYPES)
def test_small_m_rows_equal_the_m1_result(ctx, orc, qtype):
    """Speculative-verify batches: a row's result does not depend on how many rows ride along
    (bitwise, for every M the matrix-core kernel serves), and agrees with the M=1 decode kernel,
    which sums the same exact integer dots in another fp32 order."""
    from magnitude_amd import ACT_GGML
    k, n = SHAPES[qtype][0]
    blocks = make_weight(orc, qtype, n, k, seed=3000)
    w = ctx.upload(qtype, k, n, blocks)
    rng = np.random.default_rng(77)
    x = dev(rng.standard_normal((16, k)).astype(np.float32))
    single = torch.cat([ctx.mul_mat(w, x[i:i + 1], ACT_GGML) for i in range(16)]).cpu().numpy()
    full = ctx.mul_mat(w, x, ACT_GGML).cpu().numpy()
    close(full, single, 2e-5)
    decode_rows = 4 if k <= 4096 or qtype == Q8_0 else 2
    for m in (2, 3, 4, 5, 8, 11):
        got = ctx.mul_mat(w, x[:m], ACT_GGML).cpu().numpy()
        # the decode kernel serves up to 2 rows (4 with K <= 4096 and for Q8_0), the matrix-core kernel the rest up to 16:
        # bitwise within each
        assert np.array_equal(got, (single if m <= decode_rows else full)[:m]), m


@pytest.mark.parametrize("qtype,k,n,ms", [(Q6_K, 14336, 4096, (3, 4, 8, 16, 24)), (Q4_K, 14336, 4096, (5, 8, 21)),
                                            (Q8_0, 14336, 2048, (5, 8)), (Q6_K, 14336, 1056, (7,))])
def test_two_k_chunks_add_themselves_like_the_summing_launch(ctx, qtype, k, n, ms):
    """Small batches of long rows: the matrix-core kernel cuts K in chunks.  With exactly two chunks (the 8B down
    projection at 3..8 rows) the quantizer launch of qproj_mul_mat clears the output rows and both chunks add their
    partial results to them; activations quantized beforehand (qproj_mul_mat_quantized) keep the partial results in
    scratch and the launch that sums them in chunk order.  0 + a + b = a + b in either order, so the two routes must
    agree bit for bit - whatever the output buffer held before, and on a second call into the same buffer."""
    from magnitude_amd import ACT_GGML, synth
    w = ctx.upload_from_device(qtype, k, n, synth.random_weight(qtype, n, k, seed=8100 + n, device="cuda"))
    g = torch.Generator(device="cuda")
    g.manual_seed(12)
    for m in ms:
        x = torch.randn((m, k), generator=g, device="cuda")
        out = torch.full((m, n), float("nan"), device="cuda")
        ctx.mul_mat(w, x, ACT_GGML, out=out)
        first = out.clone()
        ctx.mul_mat(w, x, ACT_GGML, out=out)
        ref = ctx.mul_mat_quantized([w], ctx.quantize_activations_raw(x, ACT_GGML, qtype), ACT_GGML, m,
                                    [torch.full((m, n), float("nan"), device="cuda")])[0]
        assert torch.isfinite(ref).all()
        assert torch.equal(first, ref), m
        assert torch.equal(out, ref), m
        want = (ctx.dequantize(w).double() @ x.double().T).T
        rel = ((ref.double() - want).norm() / want.norm()).item()
        assert rel < 2e-2, (m, rel)   # int8 activations against the fp64 product of the dequantized weights
    w.free()


def test_outputs_that_overlap_the_activations_keep_the_storing_route(ctx):
    """Where two K parts add themselves to the output, the launch that quantizes x also clears y - so y would be
    written while x is still being read.  A call whose output overlaps its input must therefore not take that route:
    the quantizer reads all of x first, the projection stores y afterwards, and the result is that of a call with
    separate buffers.  (8 rows of the 14336 -> 4096 Q6_K matrix: the small-batch kernel with two K chunks; 192 rows of
    4096 x 4096 Q4_K: two K stretches of a tile.)"""
    from magnitude_amd import ACT_GGML, synth
    for qtype, k, n, m in ((Q6_K, 14336, 4096, 8), (Q4_K, 4096, 4096, 192)):
        w = ctx.upload_from_device(qtype, k, n, synth.random_weight(qtype, n, k, seed=8300 + m, device="cuda"))
        g = torch.Generator(device="cuda")
        g.manual_seed(m)
        x = torch.randn((m, k), generator=g, device="cuda")
        want = ctx.mul_mat(w, x, ACT_GGML)
        buf = torch.empty(max(m * k, m * n) + 64, device="cuda")
        xa = buf[: m * k].view(m, k)
        xa.copy_(x)
        ya = buf[: m * n].view(m, n)                      # the output starts where the input starts
        ctx.mul_mat(w, xa, ACT_GGML, out=ya)
        assert torch.allclose(ya, want, rtol=1e-5, atol=1e-6), (qtype, m)   # (the two routes differ in fp32 order only)
        xa.copy_(x)
        yt = buf[64: 64 + m * n].view(m, n)               # ... and a shifted overlap
        ctx.mul_mat(w, xa, ACT_GGML, out=yt)
        assert torch.allclose(yt, want, rtol=1e-5, atol=1e-6), (qtype, m, "shifted")
        w.free()


@pytest.mark.parametrize("m,k,ns", [(192, 4096, (4096,)), (64, 4096, (14336,)), (256, 14336, (4096,)),
                                     (192, 4096, (4096, 1024, 1024)), (130, 4096, (14336, 14336))])
def test_two_k_stretches_of_a_tile_add_themselves(ctx, m, k, ns):
    """Tiled Q4_K products on grids that leave compute units idle cut K into stretches.  Exactly two stretches, in a
    call that quantizes its own activations, add their partial tiles to output rows that the quantizer launch
    cleared (no scratch, no adding pass); qproj_mul_mat_quantized keeps partial tiles and the pass.  Same integer
    sums, another fp32 order across the stretches: equal within a few ulp, the same on every call whatever the
    output held before, and right against the fp64 product of the dequantized weights."""
    from magnitude_amd import ACT_GGML, synth
    ws = [ctx.upload_from_device(Q4_K, k, n, synth.random_weight(Q4_K, n, k, seed=8300 + i, device="cuda"))
          for i, n in enumerate(ns)]
    g = torch.Generator(device="cuda")
    g.manual_seed(m)
    x = torch.randn((m, k), generator=g, device="cuda")
    outs = [torch.full((m, n), float("nan"), device="cuda") for n in ns]
    ctx.mul_mat_multi(ws, x, ACT_GGML, outs=outs)
    first = [o.clone() for o in outs]
    ctx.mul_mat_multi(ws, x, ACT_GGML, outs=outs)
    ref = ctx.mul_mat_quantized(ws, ctx.quantize_activations_raw(x, ACT_GGML, Q4_K), ACT_GGML, m,
                                [torch.full((m, n), float("nan"), device="cuda") for n in ns])
    for w, a, b, r in zip(ws, first, outs, ref):
        assert torch.isfinite(a).all() and torch.equal(a, b)
        scale = r.abs().max().item()
        assert (a - r).abs().max().item() <= 2e-6 * scale
        want = (ctx.dequantize(w).double() @ x.double().T).T
        rel = ((a.double() - want).norm() / want.norm()).item()
        assert rel < 2e-2, rel
        w.free()


def test_mul_mat_multi_equals_separate_calls(ctx, orc):
    from magnitude_amd import ACT_GGML
    k = 4096
    ns = [512, 128, 128]
    ws = [ctx.upload(Q4_K, k, n, make_weight(orc, Q4_K, n, k, seed=4000 + i)) for i, n in enumerate(ns)]
    x = dev(np.random.default_rng(5).standard_normal((1, k)).astype(np.float32))
    ys = ctx.mul_mat_multi(ws, x, ACT_GGML)
    for w, y in zip(ws, ys):
        assert torch.equal(y, ctx.mul_mat(w, x, ACT_GGML))


@pytest.mark.parametrize("m", [48, 130, 512])
@pytest.mark.parametrize("ns", [(520, 130, 77), (1024, 256), (4096, 1024, 1024)])
def test_mul_mat_multi_prefill_batches_equal_separate_calls(ctx, orc, ns, m):
    """Prefill-sized batches: q/k/v (or gate/up) share one launch of the 64-token kernel, each matrix on its own
    run of workgroups with idle ones in between -- bitwise what the matrices give one by one, ragged edges
    included, and the oracle's values."""
    from magnitude_amd import ACT_GGML
    k = 1024
    blocks = [make_weight(orc, Q4_K, n, k, seed=4100 + n) for n in ns]
    ws = [ctx.upload(Q4_K, k, n, b) for n, b in zip(ns, blocks)]
    x = np.random.default_rng(m + len(ns)).standard_normal((m, k)).astype(np.float32)
    ys = ctx.mul_mat_multi(ws, dev(x), ACT_GGML)
    for w, b, y in zip(ws, blocks, ys):
        assert torch.equal(y, ctx.mul_mat(w, dev(x), ACT_GGML))
    close(ys[-1].cpu().numpy(), orc.mul_mat(Q4_K, blocks[-1], k, x, orc.ACT_GGML), 5e-5)
    for w in ws:
        w.free()


@pytest.mark.parametrize("qtype", TYPES)
def test_mul_mat_special_inputs(ctx, orc, qtype):
    """zero in -> zero out; power-of-two scaling is exact; a one-hot row picks a dequantized column."""
    from magnitude_amd import ACT_F32, ACT_GGML
    k, n = (1024, 40)
    blocks = make_weight(orc, qtype, n, k, seed=5000)
    w = ctx.upload(qtype, k, n, blocks)
    x = np.random.default_rng(6).standard_normal((1, k)).astype(np.float32)
    y1 = ctx.mul_mat(w, dev(x), ACT_GGML)
    assert torch.equal(ctx.mul_mat(w, dev(4 * x), ACT_GGML), 4 * y1)
    assert not ctx.mul_mat(w, dev(0 * x), ACT_GGML).any()
    wd = orc.dequantize(qtype, blocks, k)
    for kk in (0, 17, 255, 256, 700, 1023):
        e = np.zeros((1, k), np.float32)
        e[0, kk] = 2.0
        got = ctx.mul_mat(w, dev(e), ACT_F32).cpu().numpy()[0]
        assert np.allclose(got, 2.0 * wd[:, kk], rtol=1e-6, atol=1e-9), kk


# ---------------------------------------------------------------- prefill GEMM (int8 MFMA)

@pytest.mark.parametrize("m,k,n", [(128, 4096, 256), (200, 1024, 384), (512, 512, 130), (33, 14336, 128)])
def test_prefill_gemm_q8x32_matches_oracle(ctx, orc, m, k, n):
    from magnitude_amd import ACT_Q8X32
    blocks = make_weight(orc, Q4_K, n, k, seed=6000 + m)
    rng = np.random.default_rng(m + k)
    x = rng.standard_normal((m, k)).astype(np.float32)
    cols = rng.choice(k, max(1, k // 100), replace=False)
    x[:, cols] *= 20.0                                    # outlier channels
    w = ctx.upload(Q4_K, k, n, blocks)
    got = ctx.mul_mat(w, dev(x), ACT_Q8X32).cpu().numpy()
    want = orc.mul_mat(Q4_K, blocks, k, x, orc.ACT_Q8X32)
    close(got, want, 5e-5)
    gate(got, want)


# ---------------------------------------------------------------- MUL_MAT_ID and the MoE FFN

@pytest.fixture(scope="module")
def moe(orc):
    d_model, d_ff, E = 2048, 768, 16
    rng = np.random.default_rng(8)
    q = lambda rows, cols, s: encode(Q4_K, (np.random.default_rng(s).standard_normal((E * rows, cols)) * 0.02).astype(np.float32)).reshape(E, rows, -1)
    return dict(d_model=d_model, d_ff=d_ff, E=E, gate=q(d_ff, d_model, 81), up=q(d_ff, d_model, 82),
                down=q(d_model, d_ff, 83), rng=rng)


def routing(rng, B, top, E):
    ids = np.stack([rng.permutation(E)[:top] for _ in range(B)]).astype(np.int32)
    logits = rng.standard_normal((B, top)).astype(np.float32)
    e = np.exp(logits - logits.max(axis=1, keepdims=True))
    return ids, (e / e.sum(axis=1, keepdims=True)).astype(np.float32)


# B = 1: a workgroup set per pair (no grouping pass); B = 3: grouped, activations quantized in the
# kernel prologue; B = 8, 64: grouped, separate quantizer launch
@pytest.mark.parametrize("B", [1, 3, 8, 64])
def test_mul_mat_id_matches_oracle(ctx, orc, moe, B):
    from magnitude_amd import ACT_GGML
    E, k, n, top = moe["E"], moe["d_model"], moe["d_ff"], 8
    rng = np.random.default_rng(90 + B)
    ids, _ = routing(rng, B, top, E)
    w = ctx.upload(Q4_K, k, n, moe["up"], n_expert=E)
    x1 = rng.standard_normal((B, 1, k)).astype(np.float32)
    got = ctx.mul_mat_id(w, dev(x1), dev(ids), ACT_GGML).cpu().numpy()
    want = orc.mul_mat_id(Q4_K, moe["up"], k, n, E, x1, ids)
    close(got, want, 2e-5)
    xt = rng.standard_normal((B, top, k)).astype(np.float32)   # one activation row per slot
    got = ctx.mul_mat_id(w, dev(xt), dev(ids), ACT_GGML).cpu().numpy()
    close(got, orc.mul_mat_id(Q4_K, moe["up"], k, n, E, xt, ids), 2e-5)


@pytest.mark.parametrize("E,B", [(16, 600), (16, 1100), (512, 500)])
def test_mul_mat_id_grouping_of_many_pairs(ctx, orc, E, B):
    """The three ways the grouping pass sorts pairs by expert, on small expert matrices so that the oracle
    stays quick: 4800 pairs (ranks inside blocks of 64 pairs, several blocks per wave), 8800 pairs (more
    than the per-block path holds: sweeps over the ids in global memory) and 4000 pairs over 512 experts
    (block table too large for LDS: sweeps over ids staged in LDS).  Experts get hundreds of rows each, so
    the grouped kernel also runs its several-passes-per-expert loop."""
    from magnitude_amd import ACT_GGML
    k, n, top = 256, 32, 8
    blocks = encode(Q4_K, (np.random.default_rng(E + B).standard_normal((E * n, k)) * 0.02).astype(np.float32)).reshape(E, n, -1)
    rng = np.random.default_rng(7 * E + B)
    ids, _ = routing(rng, B, top, E)
    w = ctx.upload(Q4_K, k, n, blocks, n_expert=E)
    x = rng.standard_normal((B, 1, k)).astype(np.float32)
    got = ctx.mul_mat_id(w, dev(x), dev(ids), ACT_GGML).cpu().numpy()
    want = orc.mul_mat_id(Q4_K, blocks, k, n, E, x, ids)
    close(got, want, 2e-5)
    w.free()


def test_mul_mat_id_reports_bad_expert_ids(ctx, orc, moe):
    from magnitude_amd import ACT_GGML, QprojError
    E, k, n = moe["E"], moe["d_model"], moe["d_ff"]
    w = ctx.upload(Q4_K, k, n, moe["up"], n_expert=E)
    ids = np.array([[0, E]], dtype=np.int32)
    x = np.zeros((1, 1, k), np.float32)
    with pytest.raises(QprojError):
        ctx.mul_mat_id(w, dev(x), dev(ids), ACT_GGML)
    ids[0, 1] = 1                                            # the context stays usable
    ctx.mul_mat_id(w, dev(x), dev(ids), ACT_GGML)
    # the same through the grouping pass (more than 16 pairs)
    ids = np.tile(np.arange(8, dtype=np.int32), (3, 1))
    ids[2, 5] = -1
    x = np.zeros((3, 1, k), np.float32)
    with pytest.raises(QprojError):
        ctx.mul_mat_id(w, dev(x), dev(ids), ACT_GGML)
    ids[2, 5] = 5
    ctx.mul_mat_id(w, dev(x), dev(ids), ACT_GGML)


@pytest.mark.parametrize("B", [1, 3, 8, 64])
def test_moe_ffn_matches_oracle(ctx, orc, moe, B):
    from magnitude_amd import ACT_GGML
    E, d_model, d_ff, top = moe["E"], moe["d_model"], moe["d_ff"], 8
    rng = np.random.default_rng(95 + B)
    ids, wts = routing(rng, B, top, E)
    x = rng.standard_normal((B, d_model)).astype(np.float32)
    g = ctx.upload(Q4_K, d_model, d_ff, moe["gate"], n_expert=E)
    u = ctx.upload(Q4_K, d_model, d_ff, moe["up"], n_expert=E)
    d = ctx.upload(Q4_K, d_ff, d_model, moe["down"], n_expert=E)
    got = ctx.moe_ffn(g, u, d, dev(x), dev(ids), dev(wts), ACT_GGML).cpu().numpy()
    want = orc.moe_ffn(Q4_K, Q4_K, moe["gate"], moe["up"], moe["down"], d_model, d_ff, E, x, ids, wts,
                       orc.ACT_GGML)
    # the intermediate is re-quantized to int8: a last-bit difference in silu/expf can move one
    # code by one step, so this bar is looser than the single-projection one
    close(got, want, 2e-4)
    gate(got, want)
    # B=1 top-8 equals eight independent projections + weighted sum
    if B == 1:
        ws = [ctx.upload(Q4_K, d_model, d_ff, moe["gate"][e]) for e in ids[0]]
        gsep = torch.cat([ctx.mul_mat(wv, dev(x), ACT_GGML) for wv in ws]).cpu().numpy()
        gid = ctx.mul_mat_id(g, dev(x[:, None, :]), dev(ids), ACT_GGML).cpu().numpy()[0]
        close(gsep, gid, 2e-5)   # decode kernel vs grouped matrix-core kernel: same integer dots, other fp32 order


@pytest.mark.parametrize("E,B", [(72, 64), (128, 64), (72, 160)])
def test_moe_ffn_many_experts(ctx, orc, moe, E, B):
    """The FFN at the expert counts of the 128-expert configuration, where the grouped launches take their
    many-workgroup shapes (8 staged rows a pass at E = 128, 16 at E = 72; 32 with more than 16 pairs an expert,
    a prompt-sized batch: E = 72, 160 tokens) and the quantizer of x rides in the grouping launch."""
    from magnitude_amd import ACT_GGML
    d_model, d_ff, top = moe["d_model"], moe["d_ff"], 8
    rng = np.random.default_rng(300 + E + B)
    pick = rng.integers(0, moe["E"], size=E)          # the fixture's 16 experts, repeated
    gate_b, up_b, down_b = (np.ascontiguousarray(moe[k][pick]) for k in ("gate", "up", "down"))
    ids, wts = routing(rng, B, top, E)
    ids[5] = ids[4]                                    # two tokens with the same experts: more than one pair an expert for sure
    x = rng.standard_normal((B, d_model)).astype(np.float32)
    g = ctx.upload(Q4_K, d_model, d_ff, gate_b, n_expert=E)
    u = ctx.upload(Q4_K, d_model, d_ff, up_b, n_expert=E)
    d = ctx.upload(Q4_K, d_ff, d_model, down_b, n_expert=E)
    got = ctx.moe_ffn(g, u, d, dev(x), dev(ids), dev(wts), ACT_GGML).cpu().numpy()
    want = orc.moe_ffn(Q4_K, Q4_K, gate_b, up_b, down_b, d_model, d_ff, E, x, ids, wts, orc.ACT_GGML)
    # one int8 code of the re-quantized intermediate moving by a step (last bit of expf) shows up as ~7e-4 of the
    # output scale in one element of 131072 here; everything else sits below 1e-6
    close(got, want, 1e-3)
    gate(got, want)
    assert np.median(np.abs(got - want)) <= 1e-6 * np.abs(want).max()


@pytest.mark.parametrize("B,E", [(1, 128), (2, 128), (4, 128), (8, 128), (16, 128), (2, 16), (5, 40),
                                 (11, 128), (12, 128), (20, 128), (24, 128), (32, 256)])
def test_moe_ffn_few_tokens_take_an_expert_per_pair(ctx, orc, moe, B, E):
    """Decode-sized batches (no more pairs than experts, half as many again for small experts, 256 at most; or up
    to 16 pairs): the route that needs no grouping pass - a set of workgroups per pair reads ids[p] itself,
    quantizes the pair's activation row, and the down projection adds a token's pairs with their routing weights
    in slot order.  One unit a wave at one token, several pipelined units a wave at eight; from 11 tokens on a
    set of gate / up workgroups serves the eight pairs of a token, whose activation row it stages once."""
    from magnitude_amd import ACT_GGML
    d_model, d_ff, top = moe["d_model"], moe["d_ff"], 8
    rng = np.random.default_rng(700 + 10 * B + E)
    pick = rng.integers(0, moe["E"], size=E)          # the fixture's 16 experts, repeated
    gate_b, up_b, down_b = (np.ascontiguousarray(moe[k][pick]) for k in ("gate", "up", "down"))
    ids, wts = routing(rng, B, top, E)
    if B > 1:
        ids[1, :3] = ids[0, :3]                        # experts that come twice are simply read twice
    x = rng.standard_normal((B, d_model)).astype(np.float32)
    g = ctx.upload(Q4_K, d_model, d_ff, gate_b, n_expert=E)
    u = ctx.upload(Q4_K, d_model, d_ff, up_b, n_expert=E)
    d = ctx.upload(Q4_K, d_ff, d_model, down_b, n_expert=E)
    got = ctx.moe_ffn(g, u, d, dev(x), dev(ids), dev(wts), ACT_GGML).cpu().numpy()
    want = orc.moe_ffn(Q4_K, Q4_K, gate_b, up_b, down_b, d_model, d_ff, E, x, ids, wts, orc.ACT_GGML)
    close(got, want, 1e-3)      # a re-quantized code of the intermediate may move by one step (last bit of expf)
    gate(got, want)
    assert np.median(np.abs(got - want)) <= 1e-6 * np.abs(want).max()
    for t in (g, u, d):
        t.free()


@pytest.mark.parametrize("d_model,d_ff,top,B,down_t", [(1024, 1280, 3, 2, Q6_K), (4096, 256, 1, 1, Q4_K), (256, 4096, 2, 3, Q6_K),
                                                        (1280, 768, 8, 1, Q4_K), (2048, 512, 16, 1, Q6_K), (768, 1024, 5, 3, Q4_K)])
def test_moe_ffn_expert_per_pair_shapes(ctx, orc, d_model, d_ff, top, B, down_t):
    """The same route over the row lengths it maps differently: 1 to 16 whole rows a wave step (K = 4096 .. 256),
    steps whose lanes do not fill the wave (K = 768, 1280: 5 and 3 rows of 12 and 20 lanes), row counts that leave
    the last step ragged, 1 to 16 pairs a token, Q6_K down experts."""
    from magnitude_amd import ACT_GGML
    E = 24
    rng = np.random.default_rng(d_model + d_ff + top)
    enc = lambda t, rows, cols: encode(t, (rng.standard_normal((E * rows, cols)) * 0.03).astype(np.float32)).reshape(E, rows, -1)
    gate_b, up_b, down_b = enc(Q4_K, d_ff, d_model), enc(Q4_K, d_ff, d_model), enc(down_t, d_model, d_ff)
    ids, wts = routing(rng, B, top, E)
    x = rng.standard_normal((B, d_model)).astype(np.float32)
    g = ctx.upload(Q4_K, d_model, d_ff, gate_b, n_expert=E)
    u = ctx.upload(Q4_K, d_model, d_ff, up_b, n_expert=E)
    d = ctx.upload(down_t, d_ff, d_model, down_b, n_expert=E)
    got = ctx.moe_ffn(g, u, d, dev(x), dev(ids), dev(wts), ACT_GGML).cpu().numpy()
    want = orc.moe_ffn(Q4_K, down_t, gate_b, up_b, down_b, d_model, d_ff, E, x, ids, wts, orc.ACT_GGML)
    close(got, want, 1e-3)
    gate(got, want)
    assert np.median(np.abs(got - want)) <= 2e-6 * np.abs(want).max()
    for t in (g, u, d):
        t.free()


@pytest.mark.parametrize("B,down_t", [(1, Q4_K), (2, Q6_K)])
def test_moe_ffn_expert_per_pair_long_rows(ctx, orc, B, down_t):
    """Experts whose rows are longer than one 4096-weight step (17 and 18 super-blocks: a full step and a ragged
    one): a unit is one row walked step by step, the last step's idle lanes add nothing."""
    from magnitude_amd import ACT_GGML
    d_model, d_ff, E, top = 4352, 4608, 3, 2
    rng = np.random.default_rng(17 + B)
    enc = lambda t, rows, cols: encode(t, (rng.standard_normal((E * rows, cols)) * 0.02).astype(np.float32)).reshape(E, rows, -1)
    gate_b, up_b, down_b = enc(Q4_K, d_ff, d_model), enc(Q4_K, d_ff, d_model), enc(down_t, d_model, d_ff)
    ids, wts = routing(rng, B, top, E)
    x = rng.standard_normal((B, d_model)).astype(np.float32)
    g = ctx.upload(Q4_K, d_model, d_ff, gate_b, n_expert=E)
    u = ctx.upload(Q4_K, d_model, d_ff, up_b, n_expert=E)
    d = ctx.upload(down_t, d_ff, d_model, down_b, n_expert=E)
    got = ctx.moe_ffn(g, u, d, dev(x), dev(ids), dev(wts), ACT_GGML).cpu().numpy()
    want = orc.moe_ffn(Q4_K, down_t, gate_b, up_b, down_b, d_model, d_ff, E, x, ids, wts, orc.ACT_GGML)
    close(got, want, 1e-3)
    gate(got, want)
    assert np.median(np.abs(got - want)) <= 2e-6 * np.abs(want).max()
    xs = rng.standard_normal((B, top, d_ff)).astype(np.float32)          # MUL_MAT_ID alone, a row per slot
    got = ctx.mul_mat_id(d, dev(xs), dev(ids), ACT_GGML).cpu().numpy()
    close(got, orc.mul_mat_id(down_t, down_b, d_ff, d_model, E, xs, ids), 2e-5)
    for t in (g, u, d):
        t.free()


def test_moe_ffn_expert_per_pair_many_tokens_one_expert_each(ctx, orc):
    """100 tokens that name one expert each (no more pairs than experts): more groups than a round of workgroups
    gives one workgroup a token, which then walks all 2304 output rows and adds them in passes of its threads."""
    from magnitude_amd import ACT_GGML
    d_model, d_ff, E, B, base = 2304, 256, 100, 100, 6
    rng = np.random.default_rng(4242)
    enc = lambda rows, cols: encode(Q4_K, (rng.standard_normal((base * rows, cols)) * 0.03).astype(np.float32)).reshape(base, rows, -1)
    pick = rng.integers(0, base, size=E)
    gate_b, up_b, down_b = (np.ascontiguousarray(t[pick]) for t in (enc(d_ff, d_model), enc(d_ff, d_model), enc(d_model, d_ff)))
    ids = rng.permutation(E)[:B].astype(np.int32).reshape(B, 1)
    wts = rng.uniform(0.5, 1.5, size=(B, 1)).astype(np.float32)
    x = rng.standard_normal((B, d_model)).astype(np.float32)
    g = ctx.upload(Q4_K, d_model, d_ff, gate_b, n_expert=E)
    u = ctx.upload(Q4_K, d_model, d_ff, up_b, n_expert=E)
    d = ctx.upload(Q4_K, d_ff, d_model, down_b, n_expert=E)
    got = ctx.moe_ffn(g, u, d, dev(x), dev(ids), dev(wts), ACT_GGML).cpu().numpy()
    want = orc.moe_ffn(Q4_K, Q4_K, gate_b, up_b, down_b, d_model, d_ff, E, x, ids, wts, orc.ACT_GGML)
    close(got, want, 1e-3)
    gate(got, want)
    assert np.median(np.abs(got - want)) <= 2e-6 * np.abs(want).max()
    for t in (g, u, d):
        t.free()


@pytest.mark.parametrize("qtype,k,n", [(Q4_K, 768, 100), (Q6_K, 1280, 37), (Q4_K, 4096, 5), (Q6_K, 256, 333)])
def test_mul_mat_id_expert_per_pair_ragged_rows(ctx, orc, qtype, k, n):
    """MUL_MAT_ID alone on that route: row counts that are no multiple of the rows a step covers, a shared activation
    row per token and one per slot, and an id that names no expert (reported, the context stays usable)."""
    from magnitude_amd import ACT_GGML, QprojError
    E, top, B = 12, 4, 3
    rng = np.random.default_rng(k + n)
    blocks = encode(qtype, (rng.standard_normal((E * n, k)) * 0.05).astype(np.float32)).reshape(E, n, -1)
    w = ctx.upload(qtype, k, n, blocks, n_expert=E)
    ids, _ = routing(rng, B, top, E)
    for rows in (1, top):
        x = rng.standard_normal((B, rows, k)).astype(np.float32)
        got = ctx.mul_mat_id(w, dev(x), dev(ids), ACT_GGML).cpu().numpy()
        close(got, orc.mul_mat_id(qtype, blocks, k, n, E, x, ids), 2e-5)
    bad = ids.copy()
    bad[1, 2] = E
    with pytest.raises(QprojError):
        ctx.mul_mat_id(w, dev(x), dev(bad), ACT_GGML)
    got = ctx.mul_mat_id(w, dev(x), dev(ids), ACT_GGML).cpu().numpy()
    close(got, orc.mul_mat_id(qtype, blocks, k, n, E, x, ids), 2e-5)
    w.free()


@pytest.mark.parametrize("qtype,k,n", [(Q4_K, 2048, 768), (Q6_K, 768, 300), (Q4_K, 8192, 40)])
def test_mul_mat_id_pairs_of_a_token_share_a_staged_row(ctx, orc, qtype, k, n):
    """MUL_MAT_ID alone with more pairs than half the compute units have workgroups for: the pairs of a token share
    a set of workgroups that stages the token's activation row once (rows = 1), while with a row per slot every
    pair keeps its own set."""
    from magnitude_amd import ACT_GGML
    E, top, B = 128, 8, 11
    rng = np.random.default_rng(k + n + 5)
    blocks = encode(qtype, (rng.standard_normal((E * n, k)) * 0.05).astype(np.float32)).reshape(E, n, -1)
    w = ctx.upload(qtype, k, n, blocks, n_expert=E)
    ids, _ = routing(rng, B, top, E)
    ids[3, :4] = ids[2, :4]
    for rows in (1, top):
        x = rng.standard_normal((B, rows, k)).astype(np.float32)
        got = ctx.mul_mat_id(w, dev(x), dev(ids), ACT_GGML).cpu().numpy()
        close(got, orc.mul_mat_id(qtype, blocks, k, n, E, x, ids), 2e-5)
    w.free()


@pytest.mark.parametrize("qtype,k,n", [(Q4_K, 8448, 200), (Q6_K, 14336, 96), (Q8_0, 5120, 130)])
def test_mul_mat_id_long_expert_rows_go_in_chunks(ctx, orc, qtype, k, n):
    """Experts with rows of more than 4096 weights (a Mixtral-class down projection) and several pairs an expert:
    the grouped matrix-core kernel stages K in chunks - one set of workgroups a chunk, a pass adds the chunks'
    results in order - instead of leaving the call to the vector-ALU kernel.  8 and 16 staged rows a pass, a
    ragged last chunk, one activation row per token and one per slot."""
    from magnitude_amd import ACT_GGML
    E, top = 6, 2
    rng = np.random.default_rng(k + n)
    blocks = encode(qtype, (rng.standard_normal((E * n, k)) * 0.05).astype(np.float32)).reshape(E, n, -1)
    w = ctx.upload(qtype, k, n, blocks, n_expert=E)
    for B in (8, 24, 60):
        ids, _ = routing(rng, B, top, E)
        for rows in (1, top):
            x = rng.standard_normal((B, rows, k)).astype(np.float32)
            got = ctx.mul_mat_id(w, dev(x), dev(ids), ACT_GGML).cpu().numpy()
            close(got, orc.mul_mat_id(qtype, blocks, k, n, E, x, ids), 2e-5)
    w.free()


@pytest.mark.parametrize("E,top,B,d_model,d_ff", [(4, 2, 24, 512, 8192), (4, 2, 24, 8192, 512), (4, 2, 24, 5120, 4352),
                                                  (16, 2, 12, 8192, 512)])
def test_moe_ffn_long_rows_go_in_chunks(ctx, orc, E, top, B, d_model, d_ff):
    """The FFN with rows of more than 4096 weights on the grouped route: a long intermediate row (the down
    projection walks its K in chunks), a long model row (gate and up take a chunked launch each and the quantizer
    in front of the down projection forms the swiglu - or an elementwise launch, where the down launch quantizes
    its own rows: the last case), and both."""
    from magnitude_amd import ACT_GGML
    rng = np.random.default_rng(7 * d_model + E)
    enc = lambda t, rows, cols: encode(t, (rng.standard_normal((E * rows, cols)) * 0.03).astype(np.float32)).reshape(E, rows, -1)
    gate_b, up_b, down_b = enc(Q4_K, d_ff, d_model), enc(Q4_K, d_ff, d_model), enc(Q6_K, d_model, d_ff)
    ids, wts = routing(rng, B, top, E)
    x = rng.standard_normal((B, d_model)).astype(np.float32)
    g = ctx.upload(Q4_K, d_model, d_ff, gate_b, n_expert=E)
    u = ctx.upload(Q4_K, d_model, d_ff, up_b, n_expert=E)
    d = ctx.upload(Q6_K, d_ff, d_model, down_b, n_expert=E)
    got = ctx.moe_ffn(g, u, d, dev(x), dev(ids), dev(wts), ACT_GGML).cpu().numpy()
    want = orc.moe_ffn(Q4_K, Q6_K, gate_b, up_b, down_b, d_model, d_ff, E, x, ids, wts, orc.ACT_GGML)
    # (seeded so that no int8 code of a re-quantized intermediate row sits on a rounding tie against the host's expf:
    # such a code moves every output of its token by up to 2e-3 of the scale at these weight magnitudes - seen with
    # another seed, and taken apart there: these gate / up products, swiglu on the host and the oracle's down projection
    # agree with the call to 2e-6)
    close(got, want, 1e-3)
    gate(got, want)
    assert np.median(np.abs(got - want)) <= 2e-6 * np.abs(want).max()
    for t in (g, u, d):
        t.free()


# ---------------------------------------------------------------- RMS norm in front of the projections

@pytest.mark.parametrize("m,k", [(1, 4096), (5, 14336), (3, 20480), (7, 288), (64, 4096)])
def test_rms_norm_matches_oracle(ctx, orc, m, k):
    """RMS_NORM + MUL by the norm weights: the sum of squares is taken in double on both sides and only
    its order differs (a different last bit of the double can move the float scale by one ulp once in a
    few hundred thousand rows), every other step is the same float operation: equal to the last bit here."""
    rng = np.random.default_rng(m * 31 + k)
    x = (rng.standard_normal((m, k)) * rng.uniform(0.05, 20.0, (m, 1))).astype(np.float32)
    g = (1.0 + 0.1 * rng.standard_normal(k)).astype(np.float32)
    got = ctx.rms_norm(dev(x), dev(g), 1e-5).cpu().numpy()
    np.testing.assert_array_max_ulp(got, orc.rms_norm(x, g, 1e-5), maxulp=1)
    got = ctx.rms_norm(dev(x), None, 1e-6).cpu().numpy()
    np.testing.assert_array_max_ulp(got, orc.rms_norm(x, None, 1e-6), maxulp=1)


@pytest.mark.parametrize("m,k", [(1, 4096), (5, 14336), (3, 20480), (130, 4096)])
@pytest.mark.parametrize("qtype", [Q4_K, Q8_0])
def test_rms_norm_quantize_writes_the_bytes_of_the_two_calls(ctx, orc, qtype, m, k):
    """The fused launch must leave exactly the activation planes that qproj_rms_norm followed by
    qproj_quantize_activations leaves (all planes, compared as raw bytes), for ggml's format of the
    weight type and for the per-32 prefill format; a projection fed from them equals the unfused one."""
    from magnitude_amd import ACT_GGML, ACT_Q8X32
    rng = np.random.default_rng(m * 17 + k + qtype)
    x = dev((rng.standard_normal((m, k)) * rng.uniform(0.05, 20.0, (m, 1))).astype(np.float32))
    g = dev((1.0 + 0.1 * rng.standard_normal(k)).astype(np.float32))
    normed = ctx.rms_norm(x, g, 1e-5)
    for kind in ([ACT_GGML, ACT_Q8X32] if qtype == Q4_K else [ACT_GGML]):
        two = ctx.quantize_activations_raw(normed, kind, qtype)
        one = ctx.rms_norm_quantize_raw(x, g, 1e-5, kind, qtype)
        assert one.shape == two.shape
        n_qs = m * k
        assert torch.equal(one[:n_qs], two[:n_qs]), "codes differ"
        assert torch.equal(one, two) or _planes_equal(ctx, one, two, kind, qtype, m, k), f"planes differ (kind {kind})"
    n = 96
    blocks = make_weight(orc, qtype, n, k, seed=1900 + k + n)
    w = ctx.upload(qtype, k, n, blocks)
    fused = ctx.rms_norm_quantize_raw(x, g, 1e-5, ACT_GGML, qtype)
    y1 = ctx.mul_mat_quantized([w], fused, ACT_GGML, m, [torch.empty((m, n), device="cuda")])[0]
    y2 = ctx.mul_mat_quantized([w], ctx.quantize_activations_raw(normed, ACT_GGML, qtype), ACT_GGML, m,
                               [torch.empty((m, n), device="cuda")])[0]
    assert torch.equal(y1, y2)
    want = orc.mul_mat(qtype, blocks, k, orc.rms_norm(x.cpu().numpy(), g.cpu().numpy(), 1e-5), orc.ACT_GGML)
    close(y1.cpu().numpy(), want, 2e-5)
    w.free()


@pytest.mark.parametrize("qtype", TYPES)
@pytest.mark.parametrize("m", [1, 2, 4, 8, 200])
def test_rms_norm_mul_mat_equals_the_separate_calls(ctx, orc, qtype, m):
    """norm -> projections in one call: the decode kernel normalises in its prologue (M = 1, 2 while the row
    fits the prefetched pieces: K = 4096 and 14336 at M = 1, 4096 at M = 2), everything else runs the fused
    norm + quantizer launch and then the projection.  Bit for bit the result of qproj_rms_norm followed by
    qproj_mul_mat_multi, for ggml's activation format, the per-32 format and fp32 activations."""
    from magnitude_amd import ACT_GGML, ACT_Q8X32, ACT_F32
    for k, n in ((4096, 160), (14336, 96)):
        blocks = make_weight(orc, qtype, n, k, seed=2100 + k + n + qtype)
        w1 = ctx.upload(qtype, k, n, blocks)
        w2 = ctx.upload(qtype, k, n, make_weight(orc, qtype, n, k, seed=2200 + k + n + qtype))
        rng = np.random.default_rng(m + k + qtype)
        x = dev((rng.standard_normal((m, k)) * rng.uniform(0.1, 10.0, (m, 1))).astype(np.float32))
        g = dev((1.0 + 0.1 * rng.standard_normal(k)).astype(np.float32))
        normed = ctx.rms_norm(x, g, 1e-5)
        acts = [ACT_GGML] + ([ACT_Q8X32] if qtype == Q4_K and m >= 48 else []) + ([ACT_F32] if m <= 4 else [])
        for act in acts:
            want = ctx.mul_mat_multi([w1, w2], normed, act)
            got = ctx.rms_norm_mul_mat([w1, w2], x, g, 1e-5, act)
            for a, b in zip(got, want):
                assert torch.equal(a, b), f"act {act} K {k}"
        if m == 1:   # and against the CPU restatement of the whole chain
            ref = orc.mul_mat(qtype, blocks, k, orc.rms_norm(x.cpu().numpy(), g.cpu().numpy(), 1e-5), orc.ACT_GGML)
            close(ctx.rms_norm_mul_mat([w1], x, g, 1e-5, ACT_GGML)[0].cpu().numpy(), ref, 2e-5)
            got = ctx.rms_norm_mul_mat([w1], x, None, 1e-6, ACT_GGML)[0]
            assert torch.equal(got, ctx.mul_mat(w1, ctx.rms_norm(x, None, 1e-6), ACT_GGML))
        w1.free()
        w2.free()


@pytest.mark.parametrize("qtype", TYPES)
@pytest.mark.parametrize("m", [1, 2, 5, 130])
def test_ffn_gate_up_swiglu(ctx, orc, qtype, m):
    """h = silu(gate . x) * (up . x): for M <= 2 the decode kernel walks row r of both tensors in one wave and
    applies the product when it stores; larger batches take the two projections and an elementwise pass.
    Checked against the separate projections (same dot products: only the last bit of expf may differ from
    torch's) and against the CPU restatement; the form behind an RMS norm against the unfused chain."""
    from magnitude_amd import ACT_GGML
    for k, n in ((4096, 224), (14336, 72)):
        gate_b = make_weight(orc, qtype, n, k, seed=2300 + k + n + qtype)
        up_b = make_weight(orc, qtype, n, k, seed=2400 + k + n + qtype)
        wg, wu = ctx.upload(qtype, k, n, gate_b), ctx.upload(qtype, k, n, up_b)
        rng = np.random.default_rng(m + k + 5 * qtype)
        x = dev((rng.standard_normal((m, k)) * 2.0).astype(np.float32))
        gam = dev((1.0 + 0.1 * rng.standard_normal(k)).astype(np.float32))
        for norm in (False, True):
            xin = ctx.rms_norm(x, gam, 1e-5) if norm else x
            g, u = ctx.mul_mat_multi([wg, wu], xin, ACT_GGML)
            want = (g / (1.0 + torch.exp(-g))) * u
            got = ctx.ffn_gate_up(wg, wu, x, ACT_GGML, gamma=gam if norm else None, eps=1e-5 if norm else None)
            assert torch.allclose(got, want, rtol=2e-6, atol=1e-9), f"norm={norm} K={k}"
        xh = x.cpu().numpy()
        go, uo = orc.mul_mat(qtype, gate_b, k, xh, orc.ACT_GGML), orc.mul_mat(qtype, up_b, k, xh, orc.ACT_GGML)
        ref = (go / (1.0 + np.exp(-go.astype(np.float64)))).astype(np.float32) * uo
        close(ctx.ffn_gate_up(wg, wu, x, ACT_GGML).cpu().numpy(), ref, 5e-5)
        wg.free()
        wu.free()


def _planes_equal(ctx, a, b, kind, qtype, m, k):
    """Compares the planes of two activation buffers and ignores the alignment padding between them."""
    from magnitude_amd import ACT_GGML
    al = lambda v: (v + 255) // 256 * 256
    per256 = kind == ACT_GGML and qtype != Q8_0
    dblk = 256 if per256 else 32
    spans = [(0, m * k)]
    off_d = al(m * k)
    spans.append((off_d, off_d + m * (k // dblk) * 4))
    off_aux = off_d + al(m * (k // dblk) * 4)
    if per256:
        spans.append((off_aux, off_aux + m * (k // 16) * 2))
        off_ms = off_aux + al(m * (k // 16) * 2)
        spans.append((off_ms, off_ms + m * (k // 256) * 32))
    elif kind != ACT_GGML:
        spans.append((off_aux, off_aux + m * (k // 32) * 4))
        off_ms = off_aux + al(m * (k // 32) * 4)
        spans.append((off_ms, off_ms + m * (k // 256) * 32))
    return all(torch.equal(a[lo:hi], b[lo:hi]) for lo, hi in spans)


# ---------------------------------------------------------------- replayed from a HIP graph

def test_calls_replayed_from_a_hip_graph_give_the_eager_results(orc, moe):
    """Serving loops replay the projections from HIP graphs.  Once the context's workspace has its size the
    compute entry points only launch kernels, so a captured sequence must reproduce the eager results bit
    for bit on every replay - with other eager work and synchronizations of the same context in between,
    and with new activation values written into the same buffers.  Covered: the decode kernel (M = 1),
    quantizer + small-batch kernel with K cut into chunks and the chunk sum (M = 8, Q6_K, K = 14336), the
    tiled kernels with partial tiles added afterwards (M = 200, K = 14336), the MoE FFN with its grouping pass, and
    the launches whose two K parts add themselves to output rows the quantizer clears (M = 8 on the 14336 -> 4096
    Q6_K matrix, M = 192 on 4096 x 4096 Q4_K): the outputs hold NaN before every replay."""
    from magnitude_amd import Context, ACT_GGML, ACT_Q8X32, synth
    stream = torch.cuda.Stream()
    c = Context(0, stream=stream.cuda_stream)
    try:
        k, n = 4096, 256
        w4 = c.upload(Q4_K, k, n, make_weight(orc, Q4_K, n, k, seed=1500 + k + n))
        k6, n6 = 14336, 128
        w6 = c.upload(Q6_K, k6, n6, make_weight(orc, Q6_K, n6, k6, seed=1500 + k6 + n6))
        w4l = c.upload(Q4_K, k6, n6, make_weight(orc, Q4_K, n6, k6, seed=1500 + k6 + n6))
        w6big = c.upload_from_device(Q6_K, k6, 4096, synth.random_weight(Q6_K, 4096, k6, seed=31, device="cuda"))
        w4sq = c.upload_from_device(Q4_K, k, 4096, synth.random_weight(Q4_K, 4096, k, seed=32, device="cuda"))
        E, d_model, d_ff, top, B = moe["E"], moe["d_model"], moe["d_ff"], 8, 8
        g = c.upload(Q4_K, d_model, d_ff, moe["gate"], n_expert=E)
        u = c.upload(Q4_K, d_model, d_ff, moe["up"], n_expert=E)
        d = c.upload(Q4_K, d_ff, d_model, moe["down"], n_expert=E)
        rng = np.random.default_rng(77)
        ids, wts = routing(rng, B, top, E)
        ids_d, wts_d = dev(ids), dev(wts)
        xs = {"dec": torch.empty((1, k), device="cuda"), "small": torch.empty((8, k6), device="cuda"),
              "tiled": torch.empty((200, k6), device="cuda"), "moe": torch.empty((B, d_model), device="cuda"),
              "mid": torch.empty((192, k), device="cuda")}
        ys = {"dec": torch.empty((1, n), device="cuda"), "small": torch.empty((8, n6), device="cuda"),
              "tiled6": torch.empty((200, n6), device="cuda"), "tiled4": torch.empty((200, n6), device="cuda"),
              "per32": torch.empty((200, n6), device="cuda"), "moe": torch.empty((B, d_model), device="cuda"),
              "small_add": torch.empty((8, 4096), device="cuda"), "tiled_add": torch.empty((192, 4096), device="cuda"),
              "small_noalloc": torch.empty((8, n6), device="cuda"), "tiled_noalloc": torch.empty((200, n6), device="cuda")}

        def fill(seed):
            gen = torch.Generator(device="cuda").manual_seed(seed)
            for t in xs.values():
                t.copy_(torch.randn(t.shape, device="cuda", generator=gen))
            torch.cuda.synchronize()

        def calls():
            c.mul_mat(w4, xs["dec"], ACT_GGML, out=ys["dec"], sync=False)
            c.mul_mat(w6, xs["small"], ACT_GGML, out=ys["small"], sync=False)
            c.mul_mat(w6, xs["tiled"], ACT_GGML, out=ys["tiled6"], sync=False)
            c.mul_mat(w4l, xs["tiled"], ACT_GGML, out=ys["tiled4"], sync=False)
            c.mul_mat(w4l, xs["tiled"], ACT_Q8X32, out=ys["per32"], sync=False)
            c.moe_ffn(g, u, d, xs["moe"], ids_d, wts_d, ACT_GGML, out=ys["moe"], sync=False)
            c.mul_mat(w6big, xs["small"], ACT_GGML, out=ys["small_add"], sync=False)
            c.mul_mat(w4sq, xs["mid"], ACT_GGML, out=ys["tiled_add"], sync=False)
            # the allocation-free entry point is what a caller under capture is meant to use: chunks of K and partial
            # tiles in the library's fixed buffer
            c.mul_mat_multi([w6], xs["small"], ACT_GGML, outs=[ys["small_noalloc"]], sync=False, noalloc=True)
            c.mul_mat_multi([w4l], xs["tiled"], ACT_GGML, outs=[ys["tiled_noalloc"]], sync=False, noalloc=True)

        def eager(seed):
            fill(seed)
            calls()
            c.sync()
            return {name: t.clone() for name, t in ys.items()}

        eager(1)                                   # sizes the workspace: nothing allocates during capture
        graph = torch.cuda.CUDAGraph()
        fill(2)
        with torch.cuda.graph(graph, stream=stream):
            calls()
        for seed in (3, 4, 5):
            want = eager(seed)                     # eager work of the same context between the replays
            for t in ys.values():
                t.fill_(float("nan"))
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            for name, t in ys.items():
                assert torch.equal(t, want[name]), f"replay with inputs {seed}: {name} differs from the eager call"
            assert float(ys["moe"].abs().sum()) > 0
            assert torch.equal(ys["small_noalloc"], ys["small"]) and torch.equal(ys["tiled_noalloc"], ys["tiled4"])
    finally:
        c.close()


# ---------------------------------------------------------------- seeded sweeps over random shapes

@pytest.mark.parametrize("seed", [11, 12, 13])
def test_mul_mat_random_shapes_sweep(ctx, orc, seed):
    """40 random (type, K, N, M, activation mode) cases a seed -- ragged row counts, K of one block up to 80
    super-blocks, M across every kernel regime, outlier channels -- against the oracle in the same mode."""
    from magnitude_amd import ACT_F32, ACT_GGML, ACT_Q8X32
    rng = np.random.default_rng(seed)
    for case in range(40):
        qt = TYPES[rng.integers(3)]
        if qt == Q8_0:
            k = int(rng.choice([32, 64, 96, 1056, 2048, 4096, 4128, 5120, 8192, 256 * rng.integers(1, 40)]))
        else:
            k = int(256 * rng.choice([1, 2, 3, 5, 8, 16, 17, 32, 40, 56, 64, 80]))
        n = int(rng.choice([1, 2, 3, 31, 32, 33, 63, 100, 255, 256, 257, 1000, 4097, rng.integers(1, 9000)]))
        m = int(rng.choice([1, 1, 1, 2, 2, 3, 4, 5, 8, 9, 15, 16, 17, 31, 33, 48, 64, 65, 100, 128, 129, 200, 257]))
        m = max(1, min(m, int(1.5e9 / (k * n))))
        mode = ACT_GGML if rng.random() < 0.7 else (ACT_F32 if rng.random() < 0.5 else ACT_Q8X32)
        if mode == ACT_Q8X32 and (qt != Q4_K or k % 256):
            mode = ACT_GGML
        blocks = encode(qt, (rng.standard_normal((n, k)) * 0.02).astype(np.float32))
        x = rng.standard_normal((m, k)).astype(np.float32)
        if rng.random() < 0.2:
            x[:, rng.integers(0, k, max(1, k // 100))] *= 20
        w = ctx.upload(qt, k, n, blocks)
        got = ctx.mul_mat(w, dev(x), mode).cpu().numpy()
        want = orc.mul_mat(qt, blocks, k, x, {ACT_GGML: orc.ACT_GGML, ACT_F32: orc.ACT_F64, ACT_Q8X32: orc.ACT_Q8X32}[mode])
        try:
            close(got, want, 1e-4 if mode == ACT_F32 else 5e-5)
        except AssertionError as e:
            raise AssertionError(f"seed {seed} case {case}: type {qt} K {k} N {n} M {m} mode {mode}: {e}")
        w.free()


@pytest.mark.parametrize("seed", [21, 22])
def test_mul_mat_id_random_shapes_sweep(ctx, orc, seed):
    """20 random (type, experts, top-k, tokens, K, N, broadcast or per-slot rows) cases a seed against the oracle."""
    from magnitude_amd import ACT_GGML
    rng = np.random.default_rng(seed)
    for case in range(20):
        qt = TYPES[rng.integers(3)]
        E = int(rng.choice([1, 2, 4, 8, 16, 60, 128]))
        top = int(min(E, rng.choice([1, 2, 4, 8])))
        B = int(rng.choice([1, 2, 3, 5, 8, 17, 64, 100]))
        k = int(256 * rng.choice([1, 2, 3, 8, 16]))
        n = int(rng.choice([32, 96, 100, 256, 768, 1000]))
        nb1 = 1 if rng.random() < 0.5 else top
        wb = encode(qt, (rng.standard_normal((E * n, k)) * 0.02).astype(np.float32))
        ids = np.stack([rng.permutation(E)[:top] for _ in range(B)]).astype(np.int32)
        x = rng.standard_normal((B, nb1, k)).astype(np.float32)
        w = ctx.upload(qt, k, n, wb, n_expert=E)
        got = ctx.mul_mat_id(w, dev(x), dev(ids), ACT_GGML).cpu().numpy()
        want = orc.mul_mat_id(qt, wb, k, n, E, x, ids, orc.ACT_GGML)
        try:
            close(got, want, 5e-5)
        except AssertionError as e:
            raise AssertionError(f"seed {seed} case {case}: type {qt} E {E} top {top} B {B} K {k} N {n} nb1 {nb1}: {e}")
        w.free()


# ---------------------------------------------------------------- full benchmark sizes

@pytest.mark.parametrize("qtype,k,n", [(Q4_K, 4096, 14336), (Q6_K, 14336, 4096), (Q8_0, 4096, 4096)])
def test_full_size_against_device_fp64_of_proven_parts(ctx, qtype, k, n):
    """At the benchmark's full shapes the oracle is too slow, so the projection is checked against
    an fp64 matmul (torch) of two things already proven bit-exact above: the dequantized weights
    and the dequantized quantized activations.  In exact arithmetic that product IS the integer
    dot-product formula, so agreement to 2e-5 checks every row of the full-size kernel."""
    from magnitude_amd import ACT_F32, ACT_GGML, synth
    blocks = synth.random_weight(qtype, n, k, seed=qtype, device="cuda")
    w = ctx.upload_from_device(qtype, k, n, blocks)
    wd = ctx.dequantize(w).double()
    g = torch.Generator(device="cuda").manual_seed(1)
    for m in (1, 4, 16, 192, 1024):   # 192 and 1024: the 32- and the 64-token tiles of the Q6_K prefill kernel
        x = torch.randn((m, k), generator=g, device="cuda", dtype=torch.float32)
        y = ctx.mul_mat(w, x, ACT_GGML)
        a = ctx.quantize_activations(x, ACT_GGML, qtype)
        blk = 32 if qtype == Q8_0 else 256
        xq = (a["qs"].double().view(m, k // blk, blk) * a["d"].double()[:, :, None]).view(m, k)
        ref = xq @ wd.T
        err = ((y.double() - ref).abs() / ref.abs().clamp(min=1.0)).max().item()
        assert err <= 2e-5, err
        yf = ctx.mul_mat(w, x, ACT_F32)
        reff = x.double() @ wd.T
        errf = ((yf.double() - reff).abs() / reff.abs().clamp(min=1.0)).max().item()
        assert errf <= 1e-4, errf
    # linearity at full size: doubling x doubles y exactly
    x = torch.randn((1, k), generator=g, device="cuda", dtype=torch.float32)
    assert torch.equal(ctx.mul_mat(w, 2 * x, ACT_GGML), 2 * ctx.mul_mat(w, x, ACT_GGML))


@pytest.mark.parametrize("ns", [(28677,), (4096, 1024, 1024), (14336, 14336), (9001, 5003), (12289, 1)])
@pytest.mark.parametrize("m", [1, 2])
def test_decode_row_dealing_at_full_grids(ctx, ns, m):
    """Row counts that give the decode kernel's waves several rows each, dealt to pairs of waves in uneven
    parts (8 + 6, 8 + 7, 2 + 1, a last pair cut short by the end of the tensor), one to three tensors a launch:
    every row of every tensor against the fp64 product of the dequantized weights and the dequantized
    quantized activations (both proven bit-exact above), and against the launch of each tensor alone."""
    from magnitude_amd import ACT_GGML, synth
    k = 4096
    ws = [ctx.upload_from_device(Q4_K, k, n, synth.random_weight(Q4_K, n, k, seed=600 + i, device="cuda"))
          for i, n in enumerate(ns)]
    g = torch.Generator(device="cuda").manual_seed(sum(ns) + m)
    x = torch.randn((m, k), generator=g, device="cuda", dtype=torch.float32)
    a = ctx.quantize_activations(x, ACT_GGML, Q4_K)
    xq = (a["qs"].double().view(m, k // 256, 256) * a["d"].double()[:, :, None]).view(m, k)
    ys = ctx.mul_mat_multi(ws, x, ACT_GGML)
    for w, y in zip(ws, ys):
        ref = xq @ ctx.dequantize(w).double().T
        err = ((y.double() - ref).abs() / ref.abs().clamp(min=1.0)).max().item()
        assert err <= 2e-5, (w.N, err)
        assert torch.equal(y, ctx.mul_mat(w, x, ACT_GGML))
    for w in ws:
        w.free()


def test_full_size_prefill_gemm_against_device_fp64(ctx):
    from magnitude_amd import ACT_Q8X32, synth
    k, n, m = 4096, 4096, 512
    blocks = synth.random_weight(Q4_K, n, k, seed=3, device="cuda")
    w = ctx.upload_from_device(Q4_K, k, n, blocks)
    wd = ctx.dequantize(w).double()
    g = torch.Generator(device="cuda").manual_seed(2)
    x = torch.randn((m, k), generator=g, device="cuda", dtype=torch.float32)
    x[:, torch.randperm(k, generator=g, device="cuda")[: k // 100]] *= 20.0
    y = ctx.mul_mat(w, x, ACT_Q8X32)
    a = ctx.quantize_activations(x, ACT_Q8X32, Q4_K)
    xq = (a["qs"].double().view(m, k // 32, 32) * a["d"].double()[:, :, None]).view(m, k)
    ref = xq @ wd.T
    err = ((y.double() - ref).abs() / ref.abs().clamp(min=1.0)).max().item()
    assert err <= 5e-5, err

@pytest.mark.parametrize("m", [64, 130, 512])
def test_q6k_prefill_extreme_codes_and_scales(ctx, orc, m):
    """The Q6_K prefill kernels carry sc * (q - 32) as two int8 operands, 256 * hi + lo with hi in [-16, 16] and lo
    a signed byte, and add each over a whole super-block in int32: |I_lo| <= 256 * 128 * 127 < 2^23,
    |I_hi| <= 256 * 16 * 127 < 2^20, (I_hi << 8) + I_lo < 2^28 -- the exact integer ggml's vec_dot forms, no
    rounding anywhere before the one fp32 scaling per super-block.  Rows built to sit on those bounds: every code
    0 or 63 (q - 32 = -32 or 31), every scale -128 or 127 or a mix with small ones, activations that quantize to
    +-127 throughout, beside ordinary rows; d = 1 so nothing hides behind a small scale.  Against the oracle, both
    the 64-token and the 128-token kernel (M = 512 takes the latter with K cut in stretches)."""
    from magnitude_amd import ACT_GGML
    rng = np.random.default_rng(600 + m)
    k, n = 3072, 160
    nb = k // 256
    blocks = encode(Q6_K, (rng.standard_normal((n, k)) * 0.02).astype(np.float32)).reshape(n, nb, 210).copy()
    one = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    pat = [(0x00, 0x00, 0x80), (0xff, 0xff, 0x7f), (0x00, 0x00, 0x7f), (0xff, 0xff, 0x80), (0xff, 0x00, 0x80), (0x0f, 0xff, 0x7f)]
    for r in range(96):
        ql, qh, sc = pat[r % len(pat)]
        blocks[r, :, 0:128] = ql
        blocks[r, :, 128:192] = qh
        blocks[r, :, 192:208] = sc
        if r % 12 >= 6:     # alternating extreme scales inside a super-block, and small ones between
            blocks[r, :, 192:208] = np.array([0x80, 0x7f, 0x01, 0xff] * 4, np.uint8)
        blocks[r, :, 208:210] = one
    blocks = blocks.reshape(n, -1)
    x = rng.standard_normal((m, k)).astype(np.float32)
    x[0] = 1.0                                  # every code -127
    x[1] = -3.0                                 # every code -127 with d > 0 ... and its mirror image
    x[2] = np.where(np.arange(k) % 2 == 0, 2.0, -2.0)
    x[3, :] = 0.0
    x[3, 5::256] = 9.0                          # one non-zero code per super-block
    w = ctx.upload(Q6_K, k, n, blocks)
    got = ctx.mul_mat(w, dev(x), ACT_GGML).cpu().numpy()
    want = orc.mul_mat(Q6_K, blocks, k, x, orc.ACT_GGML)
    assert np.abs(want[:4, :96]).max() > 1e7    # the extreme rows do reach the large sums
    close(got[:, 96:], want[:, 96:], 2e-5)      # ordinary rows: the usual bar against the oracle
    # Extreme rows: with d = 1 the dequantized weights are the integers sc * (q - 32), so the exact result is
    # sum_sb dx[m, sb] * I[m, n, sb] with I an exact integer.  Random activations make those twelve terms of ~1e5
    # cancel to a few tens, so "relative to the result" measures the fp32 order of summation (the oracle's eight
    # interleaved lanes against one sum per super-block here), not the arithmetic.  The bar is relative to the
    # mass of the terms instead: (float)I, the scale product and one fma per super-block each round once.
    wi = orc.dequantize(Q6_K, blocks[:96], k).astype(np.float64)
    assert np.array_equal(wi, np.rint(wi)) and np.abs(wi).max() == 4096
    raw = orc.quantize_q8_K(x).reshape(m, nb, 292)
    dx = raw[:, :, 0:4].copy().view(np.float32)[:, :, 0].astype(np.float64)
    qa = raw[:, :, 4:260].view(np.int8).astype(np.float64)
    ints = np.einsum("msk,nsk->mns", qa, wi.reshape(96, nb, 256))          # exact: |I| < 2^28
    exact = (ints * dx[:, None, :]).sum(-1)
    mass = np.abs(ints * dx[:, None, :]).sum(-1)
    assert np.all(np.abs(got[:, :96] - exact) <= 1e-6 * mass + 1e-30)
    assert np.all(np.abs(want[:, :96] - exact) <= 1e-6 * mass + 1e-30)     # the oracle meets the same bar
    w.free()

@pytest.mark.parametrize("down_type", [Q4_K, Q6_K, Q8_0])
@pytest.mark.parametrize("m", [1, 2, 5, 20, 40, 150])
def test_ffn_equals_the_chain_and_the_oracle(ctx, orc, down_type, m):
    """qproj_ffn = norm -> gate/up -> swiglu -> down: bit for bit what qproj_(rms_norm_)ffn_gate_up followed by
    qproj_mul_mat gives, with and without the norm, on calls in a row; against the CPU restatement at the
    re-quantized-intermediate bar of the MoE feed-forward (2e-4).  Beyond two rows the swiglu is formed inside the
    down projection's quantizer (5: small-batch kernel; 20, 40, 150: tiled kernels, with the min-term plane for
    Q4_K, from the plain quantizer and from the one that takes a workgroup per row)."""
    from magnitude_amd import ACT_GGML
    for d_model, d_ff in ((512, 768), (4096, 2048)):
        rng = np.random.default_rng(7000 + d_model + d_ff + m + down_type)
        gate_b = make_weight(orc, Q4_K, d_ff, d_model, seed=7100 + d_ff)
        up_b = make_weight(orc, Q4_K, d_ff, d_model, seed=7200 + d_ff)
        down_b = make_weight(orc, down_type, d_model, d_ff, seed=7300 + d_ff + down_type)
        wg, wu, wd = ctx.upload(Q4_K, d_model, d_ff, gate_b), ctx.upload(Q4_K, d_model, d_ff, up_b), ctx.upload(down_type, d_ff, d_model, down_b)
        gam = dev((1.0 + 0.1 * rng.standard_normal(d_model)).astype(np.float32))
        xs = [dev(rng.standard_normal((m, d_model)).astype(np.float32)) for _ in range(3)]
        for norm in (False, True):
            kw = dict(gamma=gam, eps=1e-5) if norm else {}
            outs = [torch.full((m, d_model), float("nan"), device="cuda") for _ in xs]
            for x, y in zip(xs, outs):
                ctx.ffn(wg, wu, wd, x, ACT_GGML, out=y, sync=False, **kw)
            ctx.sync()
            for x, y in zip(xs, outs):
                h = ctx.ffn_gate_up(wg, wu, x, ACT_GGML, **kw)
                want = ctx.mul_mat(wd, h, ACT_GGML)
                assert torch.equal(y.view(torch.int32), want.view(torch.int32)), f"norm={norm}"
        xh = xs[0].cpu().numpy()
        go, uo = orc.mul_mat(Q4_K, gate_b, d_model, xh, orc.ACT_GGML), orc.mul_mat(Q4_K, up_b, d_model, xh, orc.ACT_GGML)
        hh = (go / (1.0 + np.exp(-go.astype(np.float64)))).astype(np.float32) * uo
        ref = orc.mul_mat(down_type, down_b, d_ff, hh, orc.ACT_GGML)
        got = ctx.ffn(wg, wu, wd, xs[0], ACT_GGML).cpu().numpy()
        # The intermediate rows differ from the oracle's in the last bits (fp32 association of gate / up), so now and then
        # a code of their re-quantization flips: one step of one code is d_x * w, up to 5e-3 of an output of this size.
        # A few rows rarely hold one (the 2e-4 bar of the MoE feed-forward); 150 rows x 2048 values hold a few, and a
        # Q8_0 block (a scale per 32) steps coarser.  There the two halves are held to the oracle one by one instead:
        # the intermediate rows at 5e-5, and the result against the oracle's down projection of THOSE rows at 5e-5
        # (the call itself is bitwise the chain, shown above).
        if m <= 5 and down_type != Q8_0:
            close(got, ref, 2e-4)
            gate(got, ref)
        else:
            h_gpu = ctx.ffn_gate_up(wg, wu, xs[0], ACT_GGML).cpu().numpy()
            close(h_gpu, hh, 5e-5)
            close(got, orc.mul_mat(down_type, down_b, d_ff, h_gpu, orc.ACT_GGML), 5e-5)
        for w in (wg, wu, wd):
            w.free()

@pytest.mark.parametrize("m", [1, 3, 40, 150])
def test_ffn_in_the_per32_format_equals_the_chain(ctx, orc, m):
    """qproj_ffn with per-32 int8 activations (Q4_K tensors): bit for bit qproj_ffn_gate_up followed by qproj_mul_mat
    in the same format, with and without the norm - the swiglu inside the quantizer writes the planes the
    elementwise pass followed by the plain quantizer writes."""
    from magnitude_amd import ACT_Q8X32
    d_model, d_ff = 512, 768
    rng = np.random.default_rng(7700 + m)
    wg = ctx.upload(Q4_K, d_model, d_ff, make_weight(orc, Q4_K, d_ff, d_model, seed=7701))
    wu = ctx.upload(Q4_K, d_model, d_ff, make_weight(orc, Q4_K, d_ff, d_model, seed=7702))
    wd = ctx.upload(Q4_K, d_ff, d_model, make_weight(orc, Q4_K, d_model, d_ff, seed=7703))
    gam = dev((1.0 + 0.1 * rng.standard_normal(d_model)).astype(np.float32))
    x = dev(rng.standard_normal((m, d_model)).astype(np.float32))
    for norm in (False, True):
        kw = dict(gamma=gam, eps=1e-5) if norm else {}
        y = ctx.ffn(wg, wu, wd, x, ACT_Q8X32, **kw)
        want = ctx.mul_mat(wd, ctx.ffn_gate_up(wg, wu, x, ACT_Q8X32, **kw), ACT_Q8X32)
        assert torch.equal(y.view(torch.int32), want.view(torch.int32)), f"norm={norm}"
        assert float(y.abs().sum()) > 0
    for w in (wg, wu, wd):
        w.free()


@pytest.mark.parametrize("act_name", ["ggml", "q8x32"])
@pytest.mark.parametrize("m", [64, 200])
def test_tiled_q4k_products_over_a_wide_range_of_activation_scales(ctx, orc, m, act_name):
    """The tiled Q4_K kernels carry the min term as fp16 high / low pairs of d * (block sum) / 16 and of dmin * min.
    The pairs are normalised by the row (a power of two under the row's largest block scale), so whole rows scaled by
    powers of two from 2^-40 to 2^40 must come out like the oracle's, which is exactly scale-invariant for powers of
    two (the decode and small-batch kernels are too): no precision lost to fp16 subnormals at the small end, no
    overflow at the large end.  One row carries a block 2^20 below the row's largest."""
    from magnitude_amd import ACT_GGML, ACT_Q8X32
    act, oact = (ACT_GGML, orc.ACT_GGML) if act_name == "ggml" else (ACT_Q8X32, orc.ACT_Q8X32)
    k, n = 2048, 192
    rng = np.random.default_rng(900 + m)
    blocks = make_weight(orc, Q4_K, n, k, seed=9100)
    w = ctx.upload(Q4_K, k, n, blocks)
    x = rng.standard_normal((m, k)).astype(np.float32)
    exps = [-40, -24, -12, -4, 0, 8, 16, 24, 40]
    x[5, 256:512] *= np.float32(2.0 ** -20)     # a block far below the row's largest: its bits no longer matter to the row
    for i in range(m):
        x[i] *= np.float32(2.0 ** exps[i % len(exps)])
    got = ctx.mul_mat(w, dev(x), act).cpu().numpy()
    want = orc.mul_mat(Q4_K, blocks, k, x, oact)
    scale = np.float32(2.0) ** np.array([exps[i % len(exps)] for i in range(m)], np.float32)[:, None]
    close(got / scale, want / scale, 5e-5)      # compared at the scale of an N(0, 1) row
    w.free()


BENCHED_PREFILL = (   # every (mode, type, K, N) x M the benchmark's prefill leg times (config 4 and the layer's other formats)
    [("q8x32", Q4_K, k, n) for (k, n) in ((4096, 14336), (14336, 4096), (4096, 4096))] +
    [("ggml", Q4_K, k, n) for (k, n) in ((4096, 14336), (14336, 4096), (4096, 4096))] +
    [("ggml", Q6_K, 14336, 4096), ("ggml", Q8_0, 4096, 4096)] +
    # shapes of other model sizes whose grids take other cuts of K (three stretches at 512 tokens)
    [("ggml", Q4_K, 11008, 4096), ("ggml", Q6_K, 13824, 5120)])


@pytest.mark.parametrize("m", [512, 2048, 4096])
@pytest.mark.parametrize("mode,qtype,k,n", BENCHED_PREFILL)
def test_every_benchmarked_prefill_shape_against_device_fp64(ctx, mode, qtype, k, n, m):
    """Config 4's whole grid (M in {512, 2048, 4096} x the three K x N shapes, per-32 and ggml activation formats)
    plus the Q6_K down projection and the Q8_0 matrix at the same M, on the dispatch path the benchmark times
    (quantize, then qproj_mul_mat_quantized: wide tiles, 64-token tiles, K cut into stretches where the grid is
    small).  Reference: fp64 product, on the device, of the dequantized weights and the dequantized quantized
    activations, both of which are proven bit-exact against the oracle at small sizes; outlier channels as in
    config 4."""
    from magnitude_amd import ACT_GGML, ACT_Q8X32, synth
    act = ACT_Q8X32 if mode == "q8x32" else ACT_GGML
    blocks = synth.random_weight(qtype, n, k, seed=77 + n + qtype, device="cuda")
    w = ctx.upload_from_device(qtype, k, n, blocks)
    del blocks
    g = torch.Generator(device="cuda").manual_seed(m + k + n)
    x = torch.randn((m, k), generator=g, device="cuda", dtype=torch.float32)
    x[:, torch.randperm(k, generator=g, device="cuda")[: k // 100]] *= 20.0
    print(f"prefill parity {mode} type {qtype} M {m} K {k} N {n}", flush=True)
    qb = ctx.quantize_activations_raw(x, act, qtype)
    y = torch.empty((m, n), device="cuda")
    ctx.mul_mat_quantized([w], qb, act, m, [y])
    a = ctx.quantize_activations(x, act, qtype)
    blk = 256 if (mode == "ggml" and qtype != Q8_0) else 32
    xq = (a["qs"].double().view(m, k // blk, blk) * a["d"].double()[:, :, None]).view(m, k)
    del a, qb, x
    wd = ctx.dequantize(w).double()
    worst = 0.0
    for m0 in range(0, m, 1024):                    # the fp64 reference 1024 tokens at a time
        ref = xq[m0:m0 + 1024] @ wd.T
        worst = max(worst, ((y[m0:m0 + 1024].double() - ref).abs() / ref.abs().clamp(min=1.0)).max().item())
        del ref
    w.free()
    del wd, xq
    torch.cuda.empty_cache()
    # 5e-5 as at the small sizes, except the per-32 kernel over K = 14336: 3584 sub-block terms a row are added in
    # fp32, the x20 outlier channels make the partial sums several times the result, and that kernel's min term is
    # carried as fp16 high / low pairs (22 bits): 6.5e-5 measured, held to 1e-4 -- a tenth of the 1e-3 gate.
    tol = 1e-4 if (mode == "q8x32" and k > 8192) else 5e-5
    assert worst <= tol, worst


# ---------------------------------------------------------------- GGUF file -> library

def test_weights_read_from_a_gguf_file_give_the_same_products(ctx, orc, tmp_path):
    """Tensors located by the GGUF reader and uploaded from the mapped file behave exactly like
    the same blocks uploaded directly; an expert stack [K, N, E] keeps its expert-major rows."""
    from magnitude_amd import ACT_GGML, gguf
    k, n, E = 512, 96, 4
    q4 = make_weight(orc, Q4_K, n, k, seed=8101)
    q6 = make_weight(orc, Q6_K, n, k, seed=8102)
    q8 = make_weight(orc, Q8_0, n, k, seed=8103)
    ex = np.concatenate([make_weight(orc, Q4_K, n, k, seed=8110 + e).reshape(-1) for e in range(E)])
    path = str(tmp_path / "model.gguf")
    gguf.write(path, [("blk.0.attn_q.weight", (k, n), Q4_K, q4), ("blk.0.ffn_down.weight", (k, n), Q6_K, q6),
                      ("output.weight", (k, n), Q8_0, q8), ("blk.0.ffn_up_exps.weight", (k, n, E), Q4_K, ex),
                      ("blk.0.attn_norm.weight", (k,), 0, np.ones(k, np.float32))],
               {"general.architecture": "llama", "general.file_type": 15})
    x = dev(np.random.default_rng(3).standard_normal((3, k)).astype(np.float32))
    with gguf.GgufFile(path) as g:
        ws = g.upload_all(ctx)
        assert set(ws) == {"blk.0.attn_q.weight", "blk.0.ffn_down.weight", "output.weight", "blk.0.ffn_up_exps.weight"}
        with pytest.raises(gguf.GgufError):
            g.upload(ctx, "blk.0.attn_norm.weight")
    for name, qt, blk in (("blk.0.attn_q.weight", Q4_K, q4), ("blk.0.ffn_down.weight", Q6_K, q6), ("output.weight", Q8_0, q8)):
        direct = ctx.upload(qt, k, n, blk)
        assert torch.equal(ctx.mul_mat(ws[name], x, ACT_GGML), ctx.mul_mat(direct, x, ACT_GGML))
        assert np.array_equal(ctx.download(ws[name]), np.asarray(blk).reshape(-1))
    we = ws["blk.0.ffn_up_exps.weight"]
    assert (we.K, we.N, we.E) == (k, n, E)
    ids = dev(np.array([[2, 0]], dtype=np.int32))
    got = ctx.mul_mat_id(we, x[:1, None, :].contiguous(), ids, ACT_GGML).cpu().numpy()[0]
    for slot, e in enumerate((2, 0)):
        one = ctx.upload(Q4_K, k, n, ex.reshape(E, -1)[e])
        close(got[slot], ctx.mul_mat(one, x[:1], ACT_GGML).cpu().numpy()[0], 2e-5)
