"""Pins the CPU oracle before anything is compared against it.

The reference checkout holds no golden vector for this path (its arithmetic is
in an un-vendored llama.cpp submodule), so each oracle function is held by what
the format and the mathematics fix: exhaustive small domains, closed forms on
hand-built blocks, an independent numpy restatement in a different code shape,
and brute force in int64/fp64.  Each check is chosen so that a dropped term, a
wrong shift or a swapped nibble fails it.
"""
import ctypes as C
import os

import numpy as np
import pytest

import np_ref
from kquant_encoders import encode

Q8_0, Q4_K, Q6_K = 8, 12, 14


# ---------------------------------------------------------------- sizes / fp16

def test_block_sizes(orc):
    L = orc.lib()
    assert L.orc_sizeof_block(Q8_0) == 34
    assert L.orc_sizeof_block(Q4_K) == 144
    assert L.orc_sizeof_block(Q6_K) == 210
    assert L.orc_sizeof_block(3) == 0
    assert L.orc_row_bytes(Q4_K, 4096) == 2304
    assert L.orc_row_bytes(Q6_K, 14336) == 56 * 210
    assert L.orc_row_bytes(Q8_0, 4096) == 128 * 34
    assert L.orc_row_bytes(Q4_K, 100) == 0  # not a multiple of the block


def test_fp16_to_fp32_exhaustive(orc):
    L = orc.lib()
    halves = np.arange(65536, dtype=np.uint16)
    want = halves.view(np.float16).astype(np.float32)
    got_sw = np.array([L.orc_fp16_to_fp32(int(h)) for h in halves], dtype=np.float32)
    got_hw = np.array([L.orc_fp16_to_fp32_f16c(int(h)) for h in halves], dtype=np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got_sw), nan) and np.array_equal(np.isnan(got_hw), nan)
    assert np.array_equal(got_sw[~nan].view(np.uint32), want[~nan].view(np.uint32))
    assert np.array_equal(got_hw[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_fp32_to_fp16_round_nearest_even(orc):
    L = orc.lib()
    rng = np.random.default_rng(11)
    vals = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * np.float32(0.02),
        rng.standard_normal(5000).astype(np.float32) * np.float32(1e-6),   # subnormal halves
        rng.standard_normal(5000).astype(np.float32) * np.float32(3e4),    # near overflow
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e-8, 5.9604645e-8, 2.98e-8, 2.99e-8,
                  6.1035156e-5, 6.0975552e-5, 1.0009766, 1.0004883, 1.0014648], dtype=np.float32),
    ])
    # exact ties between two halves: half + half-ulp, both parities
    h = rng.integers(0x0001, 0x7bff, 4000).astype(np.uint16)
    lo = h.view(np.float16).astype(np.float64)
    hi = (h + 1).astype(np.uint16).view(np.float16).astype(np.float64)
    vals = np.concatenate([vals, ((lo + hi) / 2).astype(np.float32)])
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    got = np.array([L.orc_fp32_to_fp16(float(v)) for v in vals], dtype=np.uint16)
    got_hw = np.array([L.orc_fp32_to_fp16_f16c(float(v)) for v in vals], dtype=np.uint16)
    assert np.array_equal(got, want)
    assert np.array_equal(got_hw, want)


# ---------------------------------------------------------------- 6-bit scale field

def test_scale_min_pack_unpack_exhaustive(orc):
    """All 64x64 (scale, min) values at each of the 8 positions, other positions random:
    pack -> C unpack == numpy unpack == the values packed."""
    L = orc.lib()
    rng = np.random.default_rng(5)
    out = (C.c_uint8 * 12)()
    sc_o, mn_o = C.c_uint8(), C.c_uint8()
    for j in range(8):
        for s in range(64):
            sc = rng.integers(0, 64, 8).astype(np.uint8)
            for m in (0, 1, 15, 16, 31, 32, 47, 48, 62, 63, (s * 7 + j) % 64):
                mn = rng.integers(0, 64, 8).astype(np.uint8)
                sc[j], mn[j] = s, m
                L.orc_pack_scale_min_k4(sc.ctypes.data, mn.ctypes.data, out)
                packed = np.frombuffer(out, dtype=np.uint8).copy()
                usc, umn = np_ref.unpack_scales_k4(packed[None, :])
                assert np.array_equal(usc[0], sc) and np.array_equal(umn[0], mn)
                for jj in range(8):
                    L.orc_get_scale_min_k4(jj, packed.ctypes.data, C.byref(sc_o), C.byref(mn_o))
                    assert (sc_o.value, mn_o.value) == (sc[jj], mn[jj])


def test_scale_field_known_bytes(orc):
    """Hand-computed: bytes 0..11 = 0xC1 0x42 0x83 0x04 | 0x45 0x86 0xC7 0x08 | 0x21 0x43 0x65 0x87."""
    L = orc.lib()
    q = np.array([0xC1, 0x42, 0x83, 0x04, 0x45, 0x86, 0xC7, 0x08, 0x21, 0x43, 0x65, 0x87], np.uint8)
    want_sc = [1, 2, 3, 4, 0x1 | (3 << 4), 0x3 | (1 << 4), 0x5 | (2 << 4), 0x7 | (0 << 4)]
    want_mn = [5, 6, 7, 8, 0x2 | (1 << 4), 0x4 | (2 << 4), 0x6 | (3 << 4), 0x8 | (0 << 4)]
    sc_o, mn_o = C.c_uint8(), C.c_uint8()
    for j in range(8):
        L.orc_get_scale_min_k4(j, q.ctypes.data, C.byref(sc_o), C.byref(mn_o))
        assert (sc_o.value, mn_o.value) == (want_sc[j], want_mn[j])


# ---------------------------------------------------------------- dequantize

def _half_bytes(v):
    return np.array([v], dtype="<f2").view(np.uint8)


def test_dequant_q8_0_closed_form(orc):
    blk = np.zeros(34, np.uint8)
    blk[0:2] = _half_bytes(1.0)
    blk[2:] = np.arange(-16, 16, dtype=np.int8).view(np.uint8)
    y = orc.dequantize(Q8_0, blk, 32)[0]
    assert np.array_equal(y, np.arange(-16, 16, dtype=np.float32))
    blk[0:2] = _half_bytes(-0.5)
    y = orc.dequantize(Q8_0, blk, 32)[0]
    assert np.array_equal(y, -0.5 * np.arange(-16, 16, dtype=np.float32))


def test_dequant_q4_K_closed_form(orc):
    """d=1, dmin=1, scale_j = j+1, min_j = 2j: weight l of sub-block j is (j+1)*q - 2j, with the
    nibble order 'chunk c = sub-blocks 2c (low nibbles) and 2c+1 (high nibbles)'."""
    L = orc.lib()
    blk = np.zeros(144, np.uint8)
    blk[0:2] = _half_bytes(1.0)
    blk[2:4] = _half_bytes(1.0)
    sc = np.arange(1, 9, dtype=np.uint8)
    mn = (2 * np.arange(8)).astype(np.uint8)
    packed = (C.c_uint8 * 12)()
    L.orc_pack_scale_min_k4(sc.ctypes.data, mn.ctypes.data, packed)
    blk[4:16] = np.frombuffer(packed, np.uint8)
    qv = (np.arange(256) * 7 % 16).astype(np.uint8)  # value of weight index i
    for c in range(4):
        lo = qv[64 * c: 64 * c + 32]
        hi = qv[64 * c + 32: 64 * c + 64]
        blk[16 + 32 * c: 16 + 32 * c + 32] = lo | (hi << 4)
    y = orc.dequantize(Q4_K, blk, 256)[0]
    j = np.arange(256) // 32
    want = ((j + 1) * qv.astype(np.int32) - 2 * j).astype(np.float32)
    assert np.array_equal(y, want)
    # all-zero block -> +0 everywhere (0*q - 0)
    z = orc.dequantize(Q4_K, np.zeros(144, np.uint8), 256)[0]
    assert np.array_equal(z.view(np.uint32), np.zeros(256, np.uint32))


def test_dequant_q6_K_closed_form(orc):
    """d=1, scale_s = s+1: weight i is (i//16 + 1) * (q_i - 32) with q laid out per the
    128-halves / four 32-groups / 2-bit high planes description."""
    qv = ((np.arange(256) * 37 + 11) % 64).astype(np.uint8)  # 6-bit value of weight i
    blk = np.zeros(210, np.uint8)
    for h in range(2):
        g = qv[128 * h: 128 * h + 128].reshape(4, 32)
        blk[64 * h: 64 * h + 32] = (g[0] & 0xF) | ((g[2] & 0xF) << 4)
        blk[64 * h + 32: 64 * h + 64] = (g[1] & 0xF) | ((g[3] & 0xF) << 4)
        blk[128 + 32 * h: 128 + 32 * h + 32] = (g[0] >> 4) | ((g[1] >> 4) << 2) | ((g[2] >> 4) << 4) | ((g[3] >> 4) << 6)
    blk[192:208] = np.arange(1, 17, dtype=np.int8).view(np.uint8)
    blk[208:210] = _half_bytes(1.0)
    y = orc.dequantize(Q6_K, blk, 256)[0]
    want = ((np.arange(256) // 16 + 1) * (qv.astype(np.int32) - 32)).astype(np.float32)
    assert np.array_equal(y, want)
    blk[192:208] = (-np.arange(1, 17)).astype(np.int8).view(np.uint8)  # negative scales
    y = orc.dequantize(Q6_K, blk, 256)[0]
    assert np.array_equal(y, -want)


def _random_blocks(rng, qtype, nb):
    """Random byte patterns (not quantizer outputs) with finite fp16 scales."""
    size = {Q8_0: 34, Q4_K: 144, Q6_K: 210}[qtype]
    b = rng.integers(0, 256, (nb, size), dtype=np.uint8)
    def fin(n):
        h = rng.integers(0, 65536, n).astype(np.uint16)
        bad = (h & 0x7c00) == 0x7c00
        h[bad] &= 0xbfff
        return h.view(np.uint8).reshape(n, 2)
    if qtype == Q8_0:
        b[:, 0:2] = fin(nb)
    elif qtype == Q4_K:
        b[:, 0:2] = fin(nb)
        b[:, 2:4] = fin(nb)
    else:
        b[:, 208:210] = fin(nb)
    return b


@pytest.mark.parametrize("qtype,fn", [(Q8_0, np_ref.deq_q8_0), (Q4_K, np_ref.deq_q4_K), (Q6_K, np_ref.deq_q6_K)])
def test_dequant_matches_numpy_restatement_bitwise(orc, qtype, fn):
    rng = np.random.default_rng(100 + qtype)
    nb = 4096
    blocks = _random_blocks(rng, qtype, nb)
    k = nb * orc.BLOCK_ELEMS[qtype]
    with np.errstate(over="ignore", invalid="ignore"):
        want = fn(blocks)
    got = orc.dequantize(qtype, blocks.reshape(1, -1), k)[0]
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


# ---------------------------------------------------------------- quantizers

def test_quantize_q8_0_matches_spec(orc):
    """Config 1 defines the quantizer completely: d = max|w|/127 (fp16), q = round(w/d)."""
    rng = np.random.default_rng(7)
    w = (rng.standard_normal((64, 4096)) * 0.02).astype(np.float32)
    w[3, 32:64] = 0.0                      # an all-zero block
    w[5, 0:32] = np.float32(0.02)          # constant block
    got = encode(Q8_0, w)
    want = np_ref.quant_q8_0(w).reshape(64, -1)
    assert np.array_equal(got, want)
    deq = orc.dequantize(Q8_0, got, 4096)
    d = np.repeat(np_ref.f16(got.reshape(-1, 34)[:, 0:2]), 32).reshape(64, 4096)
    # rounding to the nearest level of the unrounded scale, plus the fp16 rounding of d
    assert np.all(np.abs(deq - w) <= np.abs(d) * (0.5 + 127 * 2.0 ** -11) + 1e-12)
    assert np.array_equal(deq[3, 32:64], np.zeros(32, np.float32))


@pytest.mark.parametrize("qtype,rmse_max", [(Q4_K, 0.002), (Q6_K, 0.002), (Q8_0, 0.002)])
def test_encoder_round_trip_quality(orc, qtype, rmse_max):
    """The tests' weight encoders (kquant_encoders.c; Q8_0: the oracle's quantizer) against the bound ggml's own
    test-quantize-fns uses (recalled): array_rmse <= 0.002 on 0.1 + 2cos(i).  A quality check of test inputs,
    decoded by the oracle's pinned dequantizer -- not a parity pin."""
    i = np.arange(4096, dtype=np.float32)
    x = (0.1 + 2.0 * np.cos(i + 0.0)).astype(np.float32)[None, :]
    blocks = encode(qtype, x)
    y = orc.dequantize(qtype, blocks, 4096)
    # upstream array_rmse is sqrt(sum of squared differences) / n, threshold 0.002
    err = np.sqrt(np.sum((x.astype(np.float64) - y) ** 2)) / x.size
    assert err <= rmse_max, err
    assert err > 0 or qtype == Q8_0


@pytest.mark.parametrize("qtype", [Q4_K, Q6_K])
def test_encoder_outputs_are_valid_and_close(orc, qtype):
    rng = np.random.default_rng(21)
    w = (rng.standard_normal((32, 2048)) * 0.02).astype(np.float32)
    blocks = encode(qtype, w)
    y = orc.dequantize(qtype, blocks, 2048)
    rel = np.linalg.norm(y - w) / np.linalg.norm(w)
    assert rel < (0.08 if qtype == Q4_K else 0.02), rel
    # all-zero input -> all-zero output
    z = encode(qtype, np.zeros((1, 256), np.float32))
    assert np.array_equal(orc.dequantize(qtype, z, 256), np.zeros((1, 256), np.float32))


def test_the_oracle_makes_no_k_quant_weights(orc):
    """Q4_K / Q6_K weight blocks are inputs of the path; nothing under oracle/ claims to restate ggml's offline
    quantizer for them."""
    with pytest.raises(ValueError):
        orc.quantize(Q4_K, np.zeros((1, 256), np.float32))
    with pytest.raises(ValueError):
        orc.quantize(Q6_K, np.zeros((1, 256), np.float32))
    src = open(os.path.join(os.path.dirname(orc.__file__), "qproj_oracle.c")).read()
    assert "orc_quantize_row_q4_K" not in src and "orc_quantize_row_q6_K" not in src and "make_qkx2" not in src


def _q8_K(orc, x):
    raw = orc.quantize_q8_K(np.asarray(x, np.float32))[0].reshape(-1, 292)
    d = raw[:, 0:4].copy().view(np.float32)[:, 0]
    qs = raw[:, 4:260].view(np.int8).astype(np.int32)
    bs = raw[:, 260:292].copy().view(np.int16).astype(np.int32)
    return d, qs, bs


def test_quantize_q8_K_properties(orc):
    """Per-256 int8 with fp32 scale: the largest-|x| element maps to -127 (d takes its sign,
    negated), every quant is nearest(x/d) within [-127, 127], bsums are the 16-wide sums."""
    rng = np.random.default_rng(3)
    x = rng.standard_normal(1024).astype(np.float32)
    x[256:512] = 0.0
    d, qs, bs = _q8_K(orc, x)
    assert d[1] == 0 and not qs[1].any() and not bs[1].any()
    for b in (0, 2, 3):
        xb = x[256 * b: 256 * b + 256]
        imax = int(np.argmax(np.abs(xb)))
        assert qs[b, imax] == -127
        assert np.isclose(d[b], -xb[imax] / 127.0, rtol=1e-6)
        assert np.all(np.abs(qs[b] - xb / d[b]) <= 0.5 + 1e-4)
        assert np.array_equal(bs[b], qs[b].reshape(16, 16).sum(axis=1))


def test_quantize_q8_K_ties_round_half_to_even(orc):
    """Hand-computed from the published algorithm (quantize_row_q8_K: iscale = -127/max, q = nearest_int(iscale*x),
    nearest_int = round half to even through the 2^23 + 2^22 addend).  With max = 127 the inverse scale is exactly
    -1, so the codes are the negated inputs rounded: +-0.5 -> 0, +-1.5 -> -+2, +-2.5 -> -+2, +-3.5 -> -+4.
    roundf (half away from zero) would give -+1, -+2, -+3, -+4 and fails here."""
    x = np.zeros(256, np.float32)
    x[0] = 127.0
    ties = [0.5, -0.5, 1.5, -1.5, 2.5, -2.5, 3.5, -3.5, 126.5, -126.5, 0.49999997, 0.50000006]
    want = [0, 0, -2, 2, -2, 2, -4, 4, -126, 126, 0, -1]
    x[16:16 + len(ties)] = ties
    d, qs, bs = _q8_K(orc, x)
    assert d[0].view(np.uint32) == np.float32(-1.0).view(np.uint32)          # d = 1/iscale = 1/(-1)
    assert qs[0, 0] == -127
    assert qs[0, 16:16 + len(ties)].tolist() == want
    assert bs[0, 0] == -127 and bs[0, 1] == sum(want) and not bs[0, 2:].any()


def test_quantize_q8_K_first_largest_magnitude_sets_the_sign(orc):
    """`if (ax > amax)` is strict: of several elements of the same largest magnitude the FIRST one is `max`.
    x[3] = -8, x[10] = +8: max = -8, iscale = -127/-8 = 15.875, d = 1/15.875, q[3] = -127, q[10] = +127.
    A last-wins (or positive-wins) rule gives iscale = -15.875, d < 0 and the two codes swapped."""
    x = np.zeros(256, np.float32)
    x[3], x[10], x[200] = -8.0, 8.0, 4.0
    d, qs, _ = _q8_K(orc, x)
    assert d[0].view(np.uint32) == (np.float32(1.0) / np.float32(15.875)).view(np.uint32) and d[0] > 0
    assert qs[0, 3] == -127 and qs[0, 10] == 127 and qs[0, 200] == 64        # 63.5 -> 64: half to even
    x[3], x[10] = 8.0, -8.0
    d, qs, _ = _q8_K(orc, x)
    assert d[0] < 0 and qs[0, 3] == -127 and qs[0, 10] == 127 and qs[0, 200] == -64


def test_quantize_q8_K_constant_is_127_and_d_is_the_reciprocal_of_iscale(orc):
    """The pinned revision scales by -127/max (older ones by -128/max) and stores d = 1/iscale, two roundings,
    which is not always the one rounding of -max/127: both are told apart bit for bit."""
    m127 = np.float32(-127.0)
    differ = 0
    for mx in np.float32([3.0, 0.7, 1.6625982522964478, 60.667510986328125, 2.841683864593506, 12.437085151672363,
                          1e-3, 123.456, 7e4, 13.518299102783203]):
        x = np.zeros(256, np.float32)
        x[77] = mx
        x[5] = -mx * np.float32(0.5)
        d, qs, _ = _q8_K(orc, x)
        iscale = m127 / mx                                   # fp32 division, as in the C source
        want_d = np.float32(1.0) / iscale
        assert d[0].view(np.uint32) == want_d.view(np.uint32), mx
        assert qs[0, 77] == -127                              # -128 with the older constant
        # the half-size element: iscale * x is computed in fp32, then rounded half to even
        prod = np.float32(iscale * x[5])
        assert qs[0, 5] == int(np.rint(prod)) and abs(int(qs[0, 5]) - 63.5) <= 0.5
        differ += want_d.view(np.uint32) != (-mx / np.float32(127.0)).view(np.uint32)
    assert differ >= 5          # the vectors do separate 1/iscale from -max/127


def test_quantize_q8_K_clamps_at_127(orc):
    """`MIN(127, v)`: an element of the opposite sign and (almost) the same magnitude lands on +127, never 128.
    max = x[0] = -1 (iscale = 127): x[1] = 0.99999994 -> 126.99999 -> 127; x[2] = +1 cannot be `max` (not strictly
    larger) and gives exactly 127."""
    x = np.zeros(256, np.float32)
    x[0], x[1], x[2] = -1.0, np.float32(0.99999994), 1.0
    d, qs, _ = _q8_K(orc, x)
    assert qs[0, :3].tolist() == [-127, 127, 127] and qs.max() == 127 and qs.min() == -127
    assert d[0].view(np.uint32) == (np.float32(1.0) / np.float32(127.0)).view(np.uint32)


def test_quantize_q8_0_ties_round_half_away_from_zero(orc):
    """quantize_row_q8_0_ref: d = amax/127, id = 1/d, q = roundf(x*id).  With amax = 127 both are exactly 1, so the
    codes are the inputs rounded half AWAY from zero (+-0.5 -> +-1, +-2.5 -> +-3), where the K-quant activation
    quantizer's nearest_int would give 0 and +-2; d is stored as fp16 1.0 = 0x3C00.  Same vector through the
    activation-side entry point, which is the same function."""
    x = np.zeros((1, 64), np.float32)
    x[0, 0] = -127.0
    ties = [0.5, -0.5, 1.5, -1.5, 2.5, -2.5, 126.5, -126.5, 0.49999997]
    want = [1, -1, 2, -2, 3, -3, 127, -127, 0]
    x[0, 1:1 + len(ties)] = ties
    for raw in (orc.quantize(Q8_0, x), orc.quantize_q8_0_act(x[0])):
        blk = raw.reshape(2, 34)
        assert blk[0, 0:2].copy().view(np.uint16)[0] == 0x3C00
        q = blk[0, 2:].view(np.int8)
        assert q[0] == -127 and q[1:1 + len(ties)].tolist() == want and not q[1 + len(ties):].any()
        assert not blk[1].any()                               # the all-zero block: d = 0, id = 0, codes 0
    # d is rounded to fp16 but the codes use the unrounded fp32 scale: amax = 1 -> d = 1/127, id = 1/d
    y = np.zeros((1, 32), np.float32)
    y[0, 0], y[0, 1], y[0, 2] = 1.0, np.float32(0.5), np.float32(63.5 / 127)
    d32 = np.float32(1.0) / np.float32(127.0)
    idv = np.float32(1.0) / d32
    blk = orc.quantize(Q8_0, y).reshape(34)
    assert blk[0:2].copy().view(np.uint16)[0] == np.float16(d32).view(np.uint16)
    for j in range(3):
        v = np.float32(y[0, j] * idv)
        assert blk[2:].view(np.int8)[j] == int(np.sign(v) * np.floor(np.abs(v) + np.float32(0.5)))


def test_quantize_q8x32_properties(orc):
    rng = np.random.default_rng(4)
    x = rng.standard_normal(512).astype(np.float32)
    x[64:96] = 0
    raw = orc.quantize_q8x32(x)[0].reshape(16, 40)
    d = raw[:, 0:4].copy().view(np.float32)[:, 0]
    isum = raw[:, 4:8].copy().view(np.int32)[:, 0]
    qs = raw[:, 8:].view(np.int8).astype(np.int32)
    xb = x.reshape(16, 32)
    assert np.array_equal(d, (np.abs(xb).max(axis=1) / np.float32(127)).astype(np.float32))
    assert np.array_equal(isum, qs.sum(axis=1))
    assert d[2] == 0 and not qs[2].any()
    nz = d != 0
    assert np.all(np.abs(qs[nz] - xb[nz] / d[nz, None]) <= 0.5 + 1e-4)
    assert np.abs(qs).max() == 127


# ---------------------------------------------------------------- dot products

def _act_q8_K_parts(raw, k):
    r = raw.reshape(-1, 292)
    d = r[:, 0:4].copy().view(np.float32)[:, 0].astype(np.float64)
    qs = r[:, 4:260].view(np.int8).astype(np.int64)
    return d, qs


@pytest.mark.parametrize("k", [256, 512, 4096])
def test_vec_dot_q4_K_q8_K_brute_force(orc, k):
    """Exact value from independently unpacked integers, in int64/fp64:
    sum_b d_b*dx_b*sum_j sc_j*(q.a)_j - dmin_b*dx_b*sum_j m_j*sum(a_j)."""
    rng = np.random.default_rng(k)
    w = (rng.standard_normal((1, k)) * 0.02).astype(np.float32)
    x = rng.standard_normal(k).astype(np.float32)
    wb = encode(Q4_K, w)
    q, sc, mn, d, dmin = np_ref.q4_K_ints(wb)
    ax = orc.quantize_q8_K(x)[0]
    dx, a = _act_q8_K_parts(ax, k)
    qa = (q.astype(np.int64) * a).reshape(-1, 8, 32).sum(axis=2)
    asum = a.reshape(-1, 8, 32).sum(axis=2)
    want = np.sum(d.astype(np.float64) * dx * (sc.astype(np.int64) * qa).sum(axis=1)
                  - dmin.astype(np.float64) * dx * (mn.astype(np.int64) * asum).sum(axis=1))
    got = orc.lib().orc_vec_dot_q4_K_q8_K(k, wb.ctypes.data, ax.ctypes.data)
    assert abs(got - want) <= 2e-6 * max(1.0, abs(want)) + 1e-6
    # and the same through mul_mat
    y = orc.mul_mat(Q4_K, wb, k, x[None, :], orc.ACT_GGML)
    assert y[0, 0] == np.float32(got)


@pytest.mark.parametrize("k", [256, 1024, 14336])
def test_vec_dot_q6_K_q8_K_brute_force(orc, k):
    rng = np.random.default_rng(k + 1)
    w = (rng.standard_normal((1, k)) * 0.02).astype(np.float32)
    x = rng.standard_normal(k).astype(np.float32)
    wb = encode(Q6_K, w)
    q, sc, d = np_ref.q6_K_ints(wb)
    ax = orc.quantize_q8_K(x)[0]
    dx, a = _act_q8_K_parts(ax, k)
    qa = (q.astype(np.int64) * a).reshape(-1, 16, 16).sum(axis=2)
    want = np.sum(d.astype(np.float64) * dx * (sc.astype(np.int64) * qa).sum(axis=1))
    got = orc.lib().orc_vec_dot_q6_K_q8_K(k, wb.ctypes.data, ax.ctypes.data)
    assert abs(got - want) <= 2e-6 * max(1.0, abs(want)) + 1e-6


@pytest.mark.parametrize("k", [32, 4096])
def test_vec_dot_q8_0_q8_0_brute_force(orc, k):
    rng = np.random.default_rng(k + 2)
    w = (rng.standard_normal((1, k)) * 0.02).astype(np.float32)
    x = rng.standard_normal(k).astype(np.float32)
    wb = encode(Q8_0, w)
    ab = orc.quantize_q8_0_act(x)[0]
    W = wb.reshape(-1, 34)
    A = ab.reshape(-1, 34)
    dw = np_ref.f16(W[:, 0:2]).astype(np.float64)
    da = np_ref.f16(A[:, 0:2]).astype(np.float64)
    s = (W[:, 2:].view(np.int8).astype(np.int64) * A[:, 2:].view(np.int8).astype(np.int64)).sum(axis=1)
    want = np.sum(dw * da * s)
    got = orc.lib().orc_vec_dot_q8_0_q8_0(k, wb.ctypes.data, ab.ctypes.data)
    assert abs(got - want) <= 2e-6 * max(1.0, abs(want)) + 1e-7


@pytest.mark.parametrize("qtype", [Q8_0, Q4_K, Q6_K])
def test_vec_dot_q8x32_brute_force(orc, qtype):
    """Prefill-path dot == fp64 dot of dequantized weights with dequantized per-32 activations."""
    k = 1024
    rng = np.random.default_rng(qtype)
    w = (rng.standard_normal((3, k)) * 0.02).astype(np.float32)
    x = rng.standard_normal((2, k)).astype(np.float32)
    x[:, 5] *= 20
    wb = encode(qtype, w)
    wd = orc.dequantize(qtype, wb, k).astype(np.float64)
    raw = orc.quantize_q8x32(x).reshape(2, k // 32, 40)
    d = raw[:, :, 0:4].copy().view(np.float32)[:, :, 0].astype(np.float64)
    qs = raw[:, :, 8:].view(np.int8).astype(np.float64)
    xd = (qs * d[:, :, None]).reshape(2, k)
    want = xd @ wd.T
    got = orc.mul_mat(qtype, wb, k, x, orc.ACT_Q8X32)
    assert np.allclose(got, want, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("qtype", [Q8_0, Q4_K, Q6_K])
def test_mul_mat_one_hot_selects_dequantized_weight(orc, qtype):
    """x = v*e_k: the quantized activation is exactly {-127 * (-v/127)} at k, so y[n] ~= v*W[n,k].
    Ties the dot products to the dequantizer, index for index."""
    k = 512
    rng = np.random.default_rng(9)
    w = (rng.standard_normal((8, k)) * 0.02).astype(np.float32)
    wb = encode(qtype, w)
    wd = orc.dequantize(qtype, wb, k)
    for kk in (0, 15, 16, 31, 32, 63, 64, 100, 255, 256, 300, 511):
        x = np.zeros((1, k), np.float32)
        x[0, kk] = 2.0
        y = orc.mul_mat(qtype, wb, k, x, orc.ACT_GGML)[0]
        assert np.allclose(y, 2.0 * wd[:, kk], rtol=2e-3, atol=1e-7), kk
        y64 = orc.mul_mat_f64(qtype, wb, k, x)[0]
        assert np.array_equal(y64, 2.0 * wd[:, kk].astype(np.float64))


@pytest.mark.parametrize("qtype", [Q8_0, Q4_K, Q6_K])
def test_mul_mat_linearity_and_zero(orc, qtype):
    """Scaling x by a power of two scales the quantized-activation result exactly
    (the int8 codes are unchanged, only the fp32 scale doubles); zero in, zero out."""
    k = 1024
    rng = np.random.default_rng(10)
    w = (rng.standard_normal((16, k)) * 0.02).astype(np.float32)
    x = rng.standard_normal((1, k)).astype(np.float32)
    wb = encode(qtype, w)
    y1 = orc.mul_mat(qtype, wb, k, x, orc.ACT_GGML)
    y4 = orc.mul_mat(qtype, wb, k, 4 * x, orc.ACT_GGML)
    assert np.array_equal(4 * y1, y4)
    y0 = orc.mul_mat(qtype, wb, k, 0 * x, orc.ACT_GGML)
    assert not y0.any()
    # fp64 ground truth vs numpy matmul of dequantized weights
    wd = orc.dequantize(qtype, wb, k).astype(np.float64)
    y64 = orc.mul_mat_f64(qtype, wb, k, x)
    assert np.allclose(y64, x.astype(np.float64) @ wd.T, rtol=1e-12, atol=1e-12)


def test_ggml_activation_noise_is_what_the_design_notes_say(orc):
    """Quantifies why the quantized-activation path and the exact dot are gated separately:
    at K=4096 the Q8_K activation rounding alone moves outputs by ~1e-2 relative."""
    k, n = 4096, 256
    rng = np.random.default_rng(12)
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    x = rng.standard_normal((1, k)).astype(np.float32)
    wb = encode(Q4_K, w)
    yq = orc.mul_mat(Q4_K, wb, k, x, orc.ACT_GGML)[0]
    ye = orc.mul_mat_f64(Q4_K, wb, k, x)[0]
    big = np.abs(ye) >= 1
    rel = np.abs(yq[big] - ye[big]) / np.abs(ye[big])
    assert 1e-4 < rel.max() < 0.1


# ---------------------------------------------------------------- mul_mat_id / MoE

def test_mul_mat_id_equals_loop_of_dense(orc):
    k, n, E, B, top = 512, 24, 6, 5, 3
    rng = np.random.default_rng(13)
    w = (rng.standard_normal((E * n, k)) * 0.02).astype(np.float32)
    wb = encode(Q4_K, w).reshape(E, n, -1)
    ids = np.stack([rng.permutation(E)[:top] for _ in range(B)]).astype(np.int32)
    x1 = rng.standard_normal((B, 1, k)).astype(np.float32)
    xt = rng.standard_normal((B, top, k)).astype(np.float32)
    y1 = orc.mul_mat_id(Q4_K, wb, k, n, E, x1, ids)
    yt = orc.mul_mat_id(Q4_K, wb, k, n, E, xt, ids)
    for b in range(B):
        for j in range(top):
            e = ids[b, j]
            assert np.array_equal(y1[b, j], orc.mul_mat(Q4_K, wb[e], k, x1[b, 0:1])[0])
            assert np.array_equal(yt[b, j], orc.mul_mat(Q4_K, wb[e], k, xt[b, j:j + 1])[0])
    bad = ids.copy()
    bad[0, 0] = E
    with pytest.raises(RuntimeError):
        orc.mul_mat_id(Q4_K, wb, k, n, E, x1, bad)


def test_moe_ffn_equals_explicit_numpy(orc):
    d_model, d_ff, E, B, top = 512, 256, 8, 4, 3
    rng = np.random.default_rng(14)
    q = lambda rows, cols: encode(Q4_K, (rng.standard_normal((E * rows, cols)) * 0.02).astype(np.float32)).reshape(E, rows, -1)
    gate, up, down = q(d_ff, d_model), q(d_ff, d_model), q(d_model, d_ff)
    ids = np.stack([rng.permutation(E)[:top] for _ in range(B)]).astype(np.int32)
    logits = rng.standard_normal((B, top)).astype(np.float32)
    wts = (np.exp(logits) / np.exp(logits).sum(axis=1, keepdims=True)).astype(np.float32)
    x = rng.standard_normal((B, d_model)).astype(np.float32)
    y = orc.moe_ffn(Q4_K, Q4_K, gate, up, down, d_model, d_ff, E, x, ids, wts, orc.ACT_F64)
    want = np.zeros((B, d_model))
    for b in range(B):
        for j in range(top):
            e = ids[b, j]
            g = orc.dequantize(Q4_K, gate[e], d_model).astype(np.float64) @ x[b]
            u = orc.dequantize(Q4_K, up[e], d_model).astype(np.float64) @ x[b]
            h = (g / (1 + np.exp(-g)) * u).astype(np.float32)
            want[b] += wts[b, j] * (orc.dequantize(Q4_K, down[e], d_ff).astype(np.float64) @ h)
    assert np.allclose(y, want, rtol=2e-4, atol=2e-6)
    # slot order does not matter beyond fp32 rounding of the final sum
    perm = np.array([2, 0, 1])
    y2 = orc.moe_ffn(Q4_K, Q4_K, gate, up, down, d_model, d_ff, E, x, ids[:, perm].copy(), wts[:, perm].copy(), orc.ACT_F64)
    assert np.allclose(y, y2, rtol=1e-5, atol=1e-7)


# ---------------------------------------------------------------- rms_norm (+ weight multiply)

def test_rms_norm_closed_forms(orc):
    """Rows whose norm is known exactly: a mistake in where eps goes (outside the root, added to the sum
    instead of the mean), a mean over K-1, or a missing weight multiply fails one of them."""
    k = 64
    # constant row 1, eps = 3: mean = 1, 1/sqrt(1 + 3) = 0.5 exactly
    y = orc.rms_norm(np.ones((1, k), np.float32), None, 3.0)
    assert np.array_equal(y, np.full((1, k), 0.5, np.float32))
    # one-hot row a*e_j, eps = 0: mean = a^2/K, y_j = sqrt(K) * sign(a) (K = 64: exactly 8), zeros elsewhere
    x = np.zeros((2, k), np.float32)
    x[0, 5], x[1, 63] = 3.0, -0.25
    y = orc.rms_norm(x, None, 0.0)
    want = np.zeros_like(x)
    want[0, 5], want[1, 63] = 8.0, -8.0
    assert np.array_equal(y, want)
    # the weights multiply the normalised value element by element; rows are independent
    g = np.arange(1, k + 1, dtype=np.float32)
    y = orc.rms_norm(np.ones((3, k), np.float32), g, 3.0)
    assert np.array_equal(y, np.tile(0.5 * g, (3, 1)))
    # eps is added to the mean, not to the sum: constant row 2 over K = 64 with eps = 12 -> 2/sqrt(4 + 12) = 0.5
    y = orc.rms_norm(np.full((1, k), 2.0, np.float32), None, 12.0)
    assert np.array_equal(y, np.full((1, k), 0.5, np.float32))


def test_rms_norm_against_fp64_and_scale_invariance(orc):
    rng = np.random.default_rng(21)
    for k in (32, 288, 4096, 14336):
        x = (rng.standard_normal((4, k)) * rng.uniform(0.01, 30.0, (4, 1))).astype(np.float32)
        g = rng.standard_normal(k).astype(np.float32)
        eps = 1e-5
        y = orc.rms_norm(x, g, eps)
        x64 = x.astype(np.float64)
        ref = x64 / np.sqrt((x64 ** 2).mean(axis=1, keepdims=True) + eps) * g
        # float roundings of the mean, the root, the reciprocal and the two products: a few ulp of the fp64 value
        assert np.all(np.abs(y - ref) <= 4.0 * np.spacing(np.abs(ref).astype(np.float32)) + 1e-30)
        # a power-of-two rescaling of the row changes nothing when eps = 0 (every step scales exactly)
        y0 = orc.rms_norm(x, g, 0.0)
        assert np.array_equal(orc.rms_norm(x * np.float32(8.0), g, 0.0), y0)
        assert np.array_equal(orc.rms_norm(x, None, 0.0) * g, y0)


@pytest.mark.parametrize("qtype,k", [(Q8_0, 4096), (Q4_K, 4096), (Q6_K, 14336), (Q4_K, 256), (Q6_K, 512), (Q8_0, 96)])
def test_avx2_baseline_dots_agree_with_the_generic_ones(orc, qtype, k):
    """The CPU baseline is timed on AVX2 forms of the dot products (the shape of ggml's x86 path).  They form the
    same integers as the generic functions the parity tests use and add the floats in another order."""
    if not orc.has_avx2():
        pytest.skip("oracle built without AVX2")
    rng = np.random.default_rng(k + qtype)
    w = (rng.standard_normal((37, k)) * 0.02).astype(np.float32)
    x = rng.standard_normal((3, k)).astype(np.float32)
    x[1] *= 30.0
    blocks = encode(qtype, w)
    want = orc.mul_mat(qtype, blocks, k, x, orc.ACT_GGML)
    got = orc.mul_mat_avx2(qtype, blocks, k, x)
    assert np.max(np.abs(got - want) / np.maximum(1.0, np.abs(want))) <= 5e-5   # eight float lanes against one running sum
    # random byte patterns (every scale / min / code value), finite fp16 scales kept small
    nblk = k // (32 if qtype == Q8_0 else 256)
    size = {Q8_0: 34, Q4_K: 144, Q6_K: 210}[qtype]
    raw = rng.integers(0, 256, (5 * nblk, size), dtype=np.uint8)
    one = np.frombuffer(np.float16(0.01).tobytes(), np.uint8)
    if qtype == Q8_0:
        raw[:, 0:2] = one
    elif qtype == Q4_K:
        raw[:, 0:2] = one
        raw[:, 2:4] = one
    else:
        raw[:, 208:210] = one
    raw = raw.reshape(5, -1)
    want = orc.mul_mat(qtype, raw, k, x, orc.ACT_GGML)
    got = orc.mul_mat_avx2(qtype, raw, k, x)
    # random codes and scales: terms far larger than their sum, so the order of the float additions shows more
    assert np.max(np.abs(got - want) / np.maximum(1.0, np.abs(want))) <= 5e-5
