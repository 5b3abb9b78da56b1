"""Pins the CPU oracle (oracle/gq_oracle.py and oracle/gq_oracle.c).

What pins what:
* field order / offset / scale indexing / padded K: hand-derived words, and the numpy
  formulation the reference's own test uses (tests/python/quantization/
  test_group_quantization.py:54-81 builds the expected dequantized matrix by repeat + indices;
  `_dequant_by_repeat` below follows that formulation, which differs from the oracle's gather);
* packing: exhaustive field enumeration, inverse of unpack, zero padding, top bits of int3;
* scale and codes: closed-form groups whose exact answer is known without running any
  quantizer, constructed ties, invariants, and the reference test's own loose check
  (test_group_quantization.py:20-51, 84-108) on its shapes;
* the C restatement must agree bit for bit with the numpy one;
* routing: the worked example in the reference docstring (op/moe_misc.py:399-427) and brute force;
* golden fixtures freeze all of it.
"""

import numpy as np
import pytest

from oracle import c_oracle
from oracle import gq_oracle as o

import exact_fp

Q4, Q3 = o.SCHEMES["q4f16_1"], o.SCHEMES["q3f16_1"]
REF_SHAPES = [("q3f16_1", (2, 13)), ("q3f16_1", (16, 120)), ("q4f16_1", (2, 13)), ("q4f16_1", (16, 128))]


def test_scheme_constants():
    # group_quantization.py:57-61 for the two registry entries (quantization.py:58-68, 80-90)
    assert (Q4.elem_per_storage, Q4.storage_per_group, Q4.max_int) == (8, 4, 7)
    assert (Q3.elem_per_storage, Q3.storage_per_group, Q3.max_int) == (10, 4, 3)
    assert (Q4.num_group(4096), Q4.num_storage(4096)) == (128, 512)
    assert (Q4.num_group(14336), Q4.num_storage(14336)) == (448, 1792)
    assert (Q3.num_group(4096), Q3.num_storage(4096)) == (103, 412)
    assert (Q3.num_group(11008), Q3.num_storage(11008)) == (276, 1104)
    assert (Q3.num_group(13), Q3.num_storage(13)) == (1, 4)


def test_unpack_known_words():
    # nibble r of 0x76543210 is r; LSB first
    qw = np.array([[0x76543210, 0xFEDCBA98, 0, 0]], np.uint32)
    assert o.unpack(qw, Q4, 16).tolist() == [list(range(16))]
    # int3: field r sits at bit 3r, 10 fields, bits 30-31 unused
    word = sum((r % 8) << (3 * r) for r in range(10))
    qw3 = np.array([[word, 0xFFFFFFFF, 0, 0]], np.uint32)
    assert o.unpack(qw3, Q3, 20).tolist() == [[0, 1, 2, 3, 4, 5, 6, 7, 0, 1] + [7] * 10]


def test_dequantize_known_values():
    # (q - 7) * s and (q - 3) * s with s exactly representable
    qw = np.array([[0x76543210, 0xFEDCBA98, 0, 0]], np.uint32)
    d = o.dequantize(qw, np.array([[0.5]], np.float16), Q4, 32)
    assert d[0, :16].tolist() == [(q - 7) * 0.5 for q in range(16)]
    assert (d[0, 16:] == -3.5).all()
    word = sum((r % 8) << (3 * r) for r in range(10))
    d3 = o.dequantize(np.array([[word, 0, 0, 0]], np.uint32), np.array([[2.0]], np.float16), Q3, 13)
    assert d3[0].tolist() == [(q - 3) * 2.0 for q in [0, 1, 2, 3, 4, 5, 6, 7, 0, 1, 0, 0, 0]]


def test_dequantize_rounds_product_to_fp16():
    # 7 * s needs more than 11 significant bits for s = 1 + 2^-10: fp16 product must round
    s = np.float16(1 + 2**-10)
    qw = np.array([[14, 0, 0, 0]], np.uint32)  # q = 14 -> (14 - 7) = 7
    d = o.dequantize(qw, np.array([[s]], np.float16), Q4, 1)
    exact = 7 * float(s)
    assert float(d[0, 0]) == float(np.float16(exact)) and float(d[0, 0]) != exact


def _dequant_by_repeat(s, weight, scale, out_shape):
    """The formulation of the reference test's expected value (repeat words and scales)."""
    mask = (1 << s.bits) - 1
    wr = np.repeat(weight, s.elem_per_storage, axis=-1)
    sr = np.repeat(scale, s.group_size, axis=-1)
    j = np.indices(wr.shape)[1]
    wb = (wr >> ((j % s.elem_per_storage) * s.bits).astype(np.uint32)) & np.uint32(mask)
    assert wb.shape[1] <= sr.shape[1]
    return ((wb.astype(np.float32) - s.max_int) * sr[..., : wb.shape[1]].astype(np.float32))[
        : out_shape[0], : out_shape[1]]


@pytest.mark.parametrize("name,shape", REF_SHAPES)
def test_dequantize_matches_reference_test_formulation(name, shape):
    # test_group_quantization.py:111-146: random full-range words, random scales, rtol/atol 1e-3
    s = o.SCHEMES[name]
    rng = np.random.default_rng(7)
    n, k = shape
    qw = rng.integers(0, 2**32, (n, s.num_storage(k)), dtype=np.uint64).astype(np.uint32)
    qs = rng.random((n, s.num_group(k))).astype(np.float16)
    got = o.dequantize(qw, qs, s, k).astype(np.float32)
    want = _dequant_by_repeat(s, qw, qs, shape)
    np.testing.assert_allclose(got, want, rtol=1e-3, atol=1e-3)
    # and exactly: the fp32 product of two halves rounded once to half
    assert (got == want.astype(np.float16).astype(np.float32)).all()


@pytest.mark.parametrize("s", [Q4, Q3])
def test_pack_unpack_exhaustive_fields(s):
    e, b = s.elem_per_storage, s.bits
    for pos in range(e):
        for val in range(1 << b):
            q = np.zeros((1, s.group_size), np.uint32)
            q[0, pos] = val
            packed = o.pack(q, s)
            assert packed.shape == (1, 4)
            assert int(packed[0, 0]) == val << (pos * b) and not packed[0, 1:].any()
            assert (o.unpack(packed, s, s.group_size) == q).all()
    rng = np.random.default_rng(1)
    q = rng.integers(0, 1 << b, (5, 3 * s.group_size - 7)).astype(np.uint32)
    packed = o.pack(q, s)
    assert (o.unpack(packed, s, q.shape[1]) == q).all()
    # zero padding beyond K, and bits 30-31 of int3 words stay clear
    full = o.unpack(packed, s, packed.shape[1] * e)
    assert not full[:, q.shape[1]:].any()
    if b == 3:
        assert not (packed >> np.uint32(30)).any()


@pytest.mark.parametrize("s", [Q4, Q3])
def test_quantize_closed_form_group(s):
    # w = (q - m) * 2^-6 with the extremes present: scale is exactly 2^-6 and q comes back exactly,
    # whatever the tie rule
    m, g = s.max_int, s.group_size
    rng = np.random.default_rng(3)
    q = rng.integers(0, 2 * m + 1, (4, 2 * g)).astype(np.int64)
    q[:, 0] = 2 * m
    q[:, g] = 0
    w = ((q - m) * 2.0**-6).astype(np.float16)
    for mode in ("half_away", "half_even"):
        qw, qs = o.quantize(w, s, mode)
        assert (qs == np.float16(2.0**-6)).all()
        assert (o.unpack(qw, s, 2 * g) == q).all()
        assert (o.dequantize(qw, qs, s, 2 * g) == w).all()


@pytest.mark.parametrize("s", [Q4, Q3])
def test_quantize_ties_follow_round_mode(s):
    m, g = s.max_int, s.group_size
    w = np.zeros((1, g), np.float16)
    w[0, 0] = m * 2.0**-6  # fixes scale = 2^-6
    w[0, 1] = 0.5 * 2.0**-6  # t = m + 0.5
    w[0, 2] = 1.5 * 2.0**-6  # t = m + 1.5
    w[0, 3] = -0.5 * 2.0**-6  # t = m - 0.5
    away = o.unpack(o.quantize(w, s, "half_away")[0], s, g)[0]
    even = o.unpack(o.quantize(w, s, "half_even")[0], s, g)[0]
    assert away[:4].tolist() == [2 * m, m + 1, m + 2, m]
    exp_even = [2 * m] + [int(np.rint(v)) for v in (m + 0.5, m + 1.5, m - 0.5)]
    assert even[:4].tolist() == exp_even
    assert away[:4].tolist() != even[:4].tolist()


@pytest.mark.parametrize("s", [Q4, Q3])
def test_quantize_invariants_and_zero_group(s):
    rng = np.random.default_rng(5)
    k = 5 * s.group_size - 11
    w = (rng.standard_normal((32, k)) * 0.02).astype(np.float16)
    w[3, : s.group_size] = 0
    qw, qs = o.quantize(w, s)
    q = o.unpack(qw, s, k).astype(np.int64)
    assert q.min() >= 0 and q.max() <= 2 * s.max_int
    assert not q[3, : s.group_size].any() and qs[3, 0] == 0  # 0/0 -> NaN -> 0
    # scale is the correctly rounded fp16 quotient max|w| / m
    g = s.group_size
    for n in (0, 7):
        for gi in range(qs.shape[1]):
            grp = w[n, gi * g: (gi + 1) * g]
            mx = np.abs(grp).max()
            assert qs[n, gi] == np.float16(np.float32(mx) / np.float32(s.max_int))
            # the element of largest magnitude lands on an end of the range
            j = int(np.abs(grp.astype(np.float32)).argmax())
            assert q[n, gi * g + j] in (0, 2 * s.max_int) or mx == 0
            # monotone in w inside a group
            order = np.argsort(grp.astype(np.float32), kind="stable")
            assert (np.diff(q[n, gi * g: gi * g + len(grp)][order]) >= 0).all()
    # reconstruction error is at most half a step (plus fp16 rounding of the quotient)
    d = o.dequantize(qw, qs, s, k).astype(np.float32)
    step = np.repeat(qs.astype(np.float32), g, axis=1)[:, :k]
    assert (np.abs(d - w.astype(np.float32)) <= 0.5 * step * 1.04 + 1e-6).all()


def _quantize_np_float64(s, w):
    """The loose numpy check of the reference test (test_group_quantization.py:20-51)."""
    g, m = s.group_size, s.max_int
    n, k = w.shape
    wp = np.pad(w.astype(np.float64), ((0, 0), (0, (-k) % g)))
    wr = wp.reshape(n, -1, g)
    mx = np.maximum(np.abs(wr).max(-1), 1e-4)
    scale = mx / m
    q = np.clip(np.round(wr / scale[..., None]) + m, 0, 2 * m)
    return q.reshape(n, -1)[:, :k], scale


@pytest.mark.parametrize("name,shape", REF_SHAPES)
def test_quantize_within_reference_test_tolerance(name, shape):
    # test_group_quantization.py:84-108: uniform[0,1) weights; scales rtol/atol 1e-3; dequantized
    # values atol 0.2 (int4) / 0.4 (int3)
    s = o.SCHEMES[name]
    w = np.random.default_rng(11).random(shape).astype(np.float16)
    qw, qs = o.quantize(w, s)
    q_ref, scale_ref = _quantize_np_float64(s, w)
    np.testing.assert_allclose(qs.astype(np.float64), scale_ref, rtol=1e-3, atol=1e-3)
    got = o.dequantize(qw, qs, s, shape[1]).astype(np.float64)
    want = (q_ref - s.max_int) * np.repeat(scale_ref, s.group_size, axis=1)[:, : shape[1]]
    np.testing.assert_allclose(got, want, rtol=1e-2 if s.bits == 3 else 1e-3,
                               atol=0.4 if s.bits == 3 else 0.2)


# --------------------------------------------------------------------------- the two roundings of _quantize
#
# group_quantization.py:274-287 rounds twice in the model dtype before `round`: the quotient w / scale, then
# its sum with max_int.  The checks below pin both rounding points with arithmetic that shares nothing with
# numpy's float16 operators or with the oracle (tests/exact_fp.py: exact rationals, and long division in
# int64), so that a quantizer which divides and adds in float32 and rounds once does not pass.


def _config1_weights(rows, k):
    """Rows of the baseline's first configuration: seed 0, N(0, 0.02), float16 [4096, 4096]."""
    w = (np.random.default_rng(0).standard_normal((4096, 4096)) * 0.02).astype(np.float16)
    return np.ascontiguousarray(w[:rows, :k])


def _single_rounding_float32(w, s, mode="half_away"):
    """The plausible mistake: float32 divide and add, no rounding to the model dtype in between."""
    _, scale = o.quantize_values(w, s, mode)
    sf = np.repeat(scale.astype(np.float32), s.group_size, axis=-1)[..., : w.shape[-1]]
    t = w.astype(np.float32) / sf + np.float32(s.max_int)
    return np.clip(o._round(t, mode), 0, 2 * s.max_int).astype(np.uint32)


@pytest.mark.parametrize("s", [Q4, Q3])
@pytest.mark.parametrize("mode", ["half_away", "half_even"])
def test_quantize_equals_exact_rational_arithmetic(s, mode):
    # every code of 8 rows (32 768 values) against fractions.Fraction with an explicit round-to-nearest-even
    # to binary16 after the divide and again after the add; scales as well
    k = 4096 if s.bits == 4 else 4080
    w = _config1_weights(8, k)
    q, scale = o.quantize_values(w, s, mode)
    for r in range(w.shape[0]):
        for g in range(k // s.group_size):
            sl = slice(g * s.group_size, (g + 1) * s.group_size)
            codes, sc = exact_fp.quantize_group_fraction(exact_fp.to_fraction(w[r, sl]), s.max_int, "float16", mode)
            assert codes == q[r, sl].tolist(), (r, g)
            assert float(sc) == float(scale[r, g])


@pytest.mark.parametrize("s", [Q4, Q3])
def test_quantize_equals_exact_integer_arithmetic_on_a_million_values(s):
    # the same two roundings by long division in int64, on 256 rows of the configuration-1 matrix (1 048 576
    # values for q4; 1 044 480 for q3 with K = 102 whole groups of 40), both tie modes
    k = 4096 if s.bits == 4 else 4080
    w = _config1_weights(256, k)
    for mode in ("half_away", "half_even"):
        q, _ = o.quantize_values(w, s, mode)
        exact = exact_fp.quantize_codes_int(w.view(np.uint16), s.group_size, s.max_int, "float16", mode)
        assert np.array_equal(q, exact), int((q != exact).sum())
        cw, _ = c_oracle.quantize(w, s.bits, s.group_size, 0 if mode == "half_away" else 1)  # the C twin, directly
        assert np.array_equal(o.unpack(cw, s, k), exact)
    # the check cannot go vacuous: on this data the one-rounding variants differ from the reference's order,
    # the float32 one on more than 0.1 % of the values (0.30 % q4, 0.11 % q3), and the integer checker tells
    # one rounding from two as well
    q, _ = o.quantize_values(w, s)
    wrong = _single_rounding_float32(w, s)
    assert (wrong != q).mean() > 1e-3
    once = exact_fp.quantize_codes_int(w.view(np.uint16), s.group_size, s.max_int, "float16", roundings=1)
    assert (once != q).mean() > 2e-4
    # and the integer form of "one rounding" is the rational one (so the integer checker is itself pinned)
    for g in range(0, 8 * s.group_size, s.group_size):
        c1, _ = exact_fp.quantize_group_fraction(exact_fp.to_fraction(w[0, g: g + s.group_size]), s.max_int, "float16",
                                                 roundings=1)
        assert c1 == once[0, g: g + s.group_size].tolist()


def test_exact_rounding_helper_known_values():
    # the checker's own rounding against values that can be read off the binary16 grid by hand
    F = exact_fp.Fraction
    rne = lambda x: exact_fp.rne(F(x), "float16")
    assert rne(F(1) + F(1, 2048)) == 1  # tie between 1 and 1 + 2^-10: even significand
    assert rne(F(1) + F(3, 2048)) == F(1) + F(2, 1024)  # tie between 1+2^-10 (odd) and 1+2^-9 (even)
    assert rne(F(1, 3)) == F(1365, 4096)  # 0.333..: grid 2^-12 in [0.25, 0.5): 1365.33 -> 1365
    assert rne(F(2) ** -25) == 0 and rne(F(3, 2) * F(2) ** -25) == F(2) ** -24  # subnormal ties / rounding
    assert rne(F(65519)) == 65504 and rne(F(65520)) == exact_fp.INF  # overflow threshold
    assert rne(F(-7) * F(1025, 1024)) == F(-1794, 256)
    # and against numpy's conversion on random doubles (float64 -> float16 is one correctly rounded step)
    rng = np.random.default_rng(23)
    xs = rng.standard_normal(3000) * 10.0 ** rng.integers(-8, 5, 3000)
    with np.errstate(over="ignore"):
        want = xs.astype(np.float16)
    for x, h in zip(xs, want):
        got = exact_fp.rne(F(float(x)), "float16")
        assert (got == exact_fp.INF and np.isinf(h) and h > 0) or (got == -exact_fp.INF and np.isinf(h) and h < 0) \
            or got == F(float(h))
    b = lambda x: exact_fp.rne(F(x), "bfloat16")
    assert b(F(1) + F(1, 256)) == 1 and b(F(1) + F(3, 256)) == F(1) + F(2, 128)  # bf16 ties (8-bit significand)


def _codes(values, s, mode="half_away"):
    w = np.zeros((1, s.group_size), np.float16)
    w[0, : len(values)] = values
    return o.unpack(o.quantize(w, s, mode)[0], s, s.group_size)[0, : len(values)].tolist()


def test_quantize_hand_derived_double_rounding_vectors():
    # (1) the ADD rounds.  q4, group maximum 7 -> scale = 7 / 7 = 1 exactly.  w = 0.5 - 2^-12 = 0.499755859375
    # (binary16 0x37FF).  Quotient = w, exact.  w + 7 = 7.499755859375 lies in [4, 8), where binary16 steps by
    # 2^-8: the neighbours are 7.49609375 (distance 0.00366) and 7.5 (distance 0.00024) -> 7.5, and round() of
    # 7.5 is 8 (both tie rules: 8 is even).  Rounding once, 7.4997... goes to 7.
    assert _codes([7.0, 0.499755859375], Q4) == [14, 8]
    assert _codes([7.0, 0.499755859375], Q4, "half_even") == [14, 8]
    assert _single_rounding_float32(np.array([[7.0, 0.499755859375] + [0] * 30], np.float16), Q4)[0, 1] == 7
    # the mirror image: w = -(0.5 + 2^-11), quotient exact, 7 - 0.50048828125 = 6.49951171875 -> neighbours
    # 6.49609375 / 6.5 -> 6.5 -> half away: 7, half even: 6; rounding once gives 6 under either rule
    assert _codes([7.0, -0.50048828125], Q4) == [14, 7]
    assert _codes([7.0, -0.50048828125], Q4, "half_even") == [14, 6]
    # q3: maximum 3 -> scale 1; 3 + 0.499755859375 = 3.499755859375 in [2, 4), step 2^-9: neighbours 3.498046875
    # (0.0017) and 3.5 (0.00024) -> 3.5 -> 4 (even too); rounding once: 3
    assert _codes([3.0, 0.499755859375], Q3) == [6, 4]
    assert _codes([3.0, 0.499755859375], Q3, "half_even") == [6, 4]
    # (2) the DIVIDE rounds, with a scale that is not a power of two.  q4, maximum 7.0078125 = 1794 / 256:
    # 7.0078125 / 7 = 1.0011160..., binary16 steps by 2^-10 in [1, 2): 1025.14 / 1024 -> scale = 1025 / 1024.
    # w = -6.5078125 = -1666 / 256.  w / scale = -1666 * 4 / 1025 = -6664 / 1025 = -6.501463..., step 2^-8 in
    # [4, 8): -1664.37 / 256 -> -1664 / 256 = -6.5 exactly.  -6.5 + 7 = 0.5 (exact) -> half away: 1, half even: 0.
    # Rounding once: 7 - 6.501463... = 0.498536... -> 0 under either rule.
    assert _codes([7.0078125, -6.5078125], Q4) == [14, 1]
    assert _codes([7.0078125, -6.5078125], Q4, "half_even") == [14, 0]
    assert _single_rounding_float32(np.array([[7.0078125, -6.5078125] + [0] * 30], np.float16), Q4)[0, 1] == 0
    # q3, maximum 3.0078125 = 1540 / 512: / 3 = 1.0026041..., * 1024 = 1026.67 -> scale = 1027 / 1024.
    # w = -2.5078125 = -1284 / 512.  w / scale = -1284 * 2 / 1027 = -2568 / 1027 = -2.500486..., step 2^-9 in
    # [2, 4): -1280.25 / 512 -> -1280 / 512 = -2.5.  -2.5 + 3 = 0.5 -> half away: 1, half even: 0; once: 0.
    assert _codes([3.0078125, -2.5078125], Q3) == [6, 1]
    assert _codes([3.0078125, -2.5078125], Q3, "half_even") == [6, 0]
    assert _single_rounding_float32(np.array([[3.0078125, -2.5078125] + [0] * 38], np.float16), Q3)[0, 1] == 0
    # (3) a scale that was rounded DOWN makes the most negative weight overshoot: maximum 7.01953125 = 1797 / 256,
    # / 7 = 1.00279..., * 1024 = 1026.86 -> scale = 1027 / 1024 (rounded up, no overshoot); maximum 7.0078125 above
    # has scale 1025 / 1024 < 7.0078125 / 7, so -7.0078125 / scale = -7.00097 -> -7.0 after the divide's rounding
    # (step 2^-8) and the sum is 0, never negative; code 0.  Its positive twin: 7.0 + 7 = 14.
    assert _codes([7.0078125, -7.0078125], Q4) == [14, 0]


@pytest.mark.parametrize("md", ["bfloat16", "float16"])
@pytest.mark.parametrize("s", [Q4, Q3])
def test_quantize_dt_equals_exact_arithmetic(md, s):
    # the generic-dtype quantizer (float32 carrier arrays rounded to the model dtype after each operation)
    # against the same exact checkers: rationals on 4 rows, int64 on 128 rows (half a million values)
    import torch

    k = 4096 if s.bits == 4 else 4080
    w16 = _config1_weights(128, k)
    if md == "bfloat16":
        wf = torch.from_numpy(w16.astype(np.float32)).bfloat16().float().numpy()
        bits = (wf.view(np.uint32) >> 16).astype(np.uint16)
    else:
        wf = w16.astype(np.float32)
        bits = w16.view(np.uint16)
    for mode in ("half_away", "half_even"):
        qw, scale = o.quantize_dt(wf, s, md, mode)
        q = o.unpack(qw, s, k)
        exact = exact_fp.quantize_codes_int(bits, s.group_size, s.max_int, md, mode)
        assert np.array_equal(q, exact), int((q != exact).sum())
    qw, scale = o.quantize_dt(wf, s, md)
    q = o.unpack(qw, s, k)
    for r in range(4):
        for g in range(k // s.group_size):
            sl = slice(g * s.group_size, (g + 1) * s.group_size)
            codes, sc = exact_fp.quantize_group_fraction(exact_fp.to_fraction(wf[r, sl]), s.max_int, md)
            assert codes == q[r, sl].tolist() and float(sc) == float(scale[r, g])
    once = exact_fp.quantize_codes_int(bits, s.group_size, s.max_int, md, roundings=1)
    assert (once != q).mean() > 2e-4  # bf16: 0.54 % (q4), 0.20 % (q3)


def test_quantize_dt_float32_equals_exact_rational_arithmetic():
    # q4f32_1: every operation is an IEEE single operation; 2 rows of 4096 against rationals rounded to binary32
    w = _config1_weights(2, 4096).astype(np.float32) * np.float32(1.0009766)  # off the binary16 grid
    qw, scale = o.quantize_dt(w, Q4, "float32")
    q = o.unpack(qw, Q4, 4096)
    for r in range(2):
        for g in range(128):
            sl = slice(g * 32, g * 32 + 32)
            codes, sc = exact_fp.quantize_group_fraction(exact_fp.to_fraction(w[r, sl]), 7, "float32")
            assert codes == q[r, sl].tolist() and float(sc) == float(scale[r, g])


@pytest.mark.parametrize("s", [Q4, Q3])
def test_c_oracle_matches_numpy_oracle(s):
    rng = np.random.default_rng(13)
    for shape in [(2, 13), (16, 4 * s.group_size), (9, 1000)]:
        w = (rng.standard_normal(shape) * 0.02).astype(np.float16)
        w[0, : min(shape[1], s.group_size)] = 0
        for mode, name in ((0, "half_away"), (1, "half_even")):
            qw, qs = o.quantize(w, s, name)
            cw, cs = c_oracle.quantize(w, s.bits, s.group_size, mode)
            assert (qw == cw).all() and (qs.view(np.uint16) == cs.view(np.uint16)).all()
        d = o.dequantize(qw, qs, s, shape[1])
        cd = c_oracle.dequantize(qw, qs, shape[1], s.bits, s.group_size)
        assert (d.view(np.uint16) == cd.view(np.uint16)).all()
        x = rng.standard_normal((3, shape[1])).astype(np.float16)
        err, bound, rel = o.check_linear(c_oracle.linear(x, qw, qs, s.bits, s.group_size),
                                         o.linear_fp32(x, qw, qs, s), x, shape[1])
        assert err <= bound and rel <= 1e-5


def test_c_oracle_half_conversion_exhaustive():
    lib = c_oracle.lib()
    allh = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    f = allh.view(np.float16).astype(np.float32)
    for h in range(0, 65536, 5):
        v = lib.gqo_h2f(h)
        assert v == f[h] or (np.isnan(v) and np.isnan(f[h]))
    rng = np.random.default_rng(17)
    xs = rng.standard_normal(20000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, 20000)
    xs = np.concatenate([xs, np.array([65519.99, 65520, 65504, 6e-8, 2.9802322e-8, 2.9802326e-8,
                                       0.0, -0.0, 1.00048828125, 1.00146484375], np.float32)])
    with np.errstate(over="ignore"):
        want = xs.astype(np.float16).view(np.uint16)
    for v, w_ in zip(xs, want):
        assert lib.gqo_f2h(float(v)) == w_


def test_linear_special_cases():
    # scale 1: the quantized matmul is an integer matmul; identity activations return the matrix
    rng = np.random.default_rng(19)
    for s in (Q4, Q3):
        k = 2 * s.group_size
        q = rng.integers(0, 2 * s.max_int + 1, (6, k)).astype(np.uint32)
        qw = o.pack(q, s)
        qs = np.ones((6, 2), np.float16)
        x = rng.integers(-4, 5, (3, k)).astype(np.float16)
        want = x.astype(np.int64) @ (q.astype(np.int64) - s.max_int).T
        assert (o.linear_fp32(x, qw, qs, s) == want).all()
        eye = np.eye(k, dtype=np.float16)
        assert (o.linear_fp32(eye, qw, qs, s).T == o.dequantize(qw, qs, s, k)).all()


def test_moe_cumsum_docstring_example():
    # op/moe_misc.py:399-427 of the reference
    ids = np.array([[0, 1], [1, 2], [3, 4], [2, 5]], np.int32)
    want = np.array([[1, 1, 1, 1], [2, 3, 3, 3], [3, 4, 4, 5], [5, 5, 6, 6], [6, 6, 7, 7], [7, 7, 7, 8]])
    cs = o.moe_cumsum(ids, 6)
    assert (cs.reshape(6, 4) == want).all()
    assert o.get_indptr(cs, 6, 4, False).tolist() == [0, 1, 3, 5, 6, 7, 8]
    assert o.get_indptr(cs, 6, 4, True).tolist() == [1, 3, 5, 6, 7, 8]
    rev, tok = o.get_indices(cs, ids)
    # slots ordered by (expert, token): e0:{t0} e1:{t0,t1} e2:{t1,t3} e3:{t2} e4:{t2} e5:{t3}
    assert tok.tolist() == [0, 0, 1, 1, 3, 2, 2, 3]
    assert rev.tolist() == [0, 1, 2, 3, 6, 4, 5, 7]


def test_routing_brute_force_properties():
    rng = np.random.default_rng(23)
    t, ne, k = 37, 8, 2
    logits = rng.standard_normal((t, ne)).astype(np.float16)
    logits[4, :] = 0.25  # full tie: lowest indices, in order
    w, ids = o.gating_softmax_topk(logits, k)
    assert ids[4].tolist() == [0, 1]
    for r in range(t):
        order = sorted(range(ne), key=lambda e: (-float(logits[r, e]), e))[:k]
        assert ids[r].tolist() == order
        v = logits[r, order].astype(np.float64)
        p = np.exp(v - v.max())
        np.testing.assert_allclose(w[r].astype(np.float64), p / p.sum(), atol=6e-4)
    cs = o.moe_cumsum(ids, ne)
    rev, tok = o.get_indices(cs, ids)
    indptr = o.get_indptr(cs, ne, t, False)
    assert indptr[0] == 0 and indptr[-1] == t * k and (np.diff(indptr) >= 0).all()
    assert sorted(rev.tolist()) == list(range(t * k))  # a permutation
    for e in range(ne):
        seg = tok[indptr[e]: indptr[e + 1]]
        assert (np.diff(seg) > 0).all()  # stable by token inside an expert
        assert all(e in ids[b] for b in seg)
    x = rng.standard_normal((t * k, 5)).astype(np.float16)
    flat = np.repeat(np.arange(t), k)
    assert (flat[rev] == tok).all()
    assert (o.scatter_output(x[rev], rev) == x).all()  # scatter undoes the gather


def test_group_gemm_and_moe_gemv_against_dense():
    rng = np.random.default_rng(29)
    s = Q4
    ne, n, k = 3, 10, 64
    w = (rng.standard_normal((ne, n, k)) * 0.05).astype(np.float16)
    qw, qs = o.quantize(w, s)
    x = rng.standard_normal((7, k)).astype(np.float16)
    indptr = np.array([0, 3, 3, 7], np.int32)
    y = o.dequantize_group_gemm_fp32(x, qw, qs, indptr, s)
    wd = o.dequantize(qw, qs, s, k).astype(np.float64)
    assert np.allclose(y[:3], x[:3].astype(np.float64) @ wd[0].T)
    assert np.allclose(y[3:], x[3:].astype(np.float64) @ wd[2].T)
    yc = c_oracle.group_gemm(x, qw, qs, indptr, s.bits, s.group_size)
    assert np.allclose(yc, y, atol=1e-4)
    ids = np.array([[2, 0]], np.int32)
    g = o.moe_dequantize_gemv_fp32(x[:1], qw, qs, ids, s)
    assert np.allclose(g[0], wd[2] @ x[0].astype(np.float64)) and np.allclose(g[1], wd[0] @ x[0].astype(np.float64))
    g2 = o.moe_dequantize_gemv_fp32(x[:2], qw, qs, ids, s)
    assert np.allclose(g2[1], wd[0] @ x[1].astype(np.float64))


def test_golden_fixtures_reproduce(golden):
    import glob
    import os

    from conftest import GOLDEN

    names = sorted(os.path.basename(p)[:-4] for p in glob.glob(os.path.join(GOLDEN, "*.npz")))
    assert len(names) >= 20
    for name in names:
        z = golden(name)
        if name.startswith("quant_"):
            s = o.SCHEMES[name.split("_")[1] + "_1"]
            for mode in ("half_away", "half_even"):
                qw, qs = o.quantize(z["w"], s, mode)
                assert (qw == z[f"q_weight_{mode}"]).all()
                assert (qs.view(np.uint16) == z[f"q_scale_{mode}"].view(np.uint16)).all()
            k = z["w"].shape[1]
            d = o.dequantize(z["q_weight_half_away"], z["q_scale_half_away"], s, k)
            assert (d.view(np.uint16) == z["dequant"].view(np.uint16)).all()
            assert np.array_equal(o.linear_fp32(z["x"], z["q_weight_half_away"], z["q_scale_half_away"], s), z["y"])
        elif name.startswith("dtype_"):
            md = name.split("_")[1]
            s = o.SCHEMES["q4f16_1"]
            k = z["w"].shape[1]
            for mode in ("half_away", "half_even"):
                qw, qs = o.quantize_dt(z["w"], s, md, mode)
                assert (qw == z[f"q_weight_{mode}"]).all() and np.array_equal(qs, z[f"q_scale_{mode}"])
            d = o.dequantize_dt(z["q_weight_half_away"], z["q_scale_half_away"], s, k, md)
            assert np.array_equal(d, z["dequant"])
            assert np.array_equal(o.linear_dt_fp64(z["x"], z["q_weight_half_away"], z["q_scale_half_away"], s, md), z["y"])
        elif name.startswith("dequant_"):
            s = o.SCHEMES[name.split("_")[1] + "_1"]
            k = z["dequant"].shape[1]
            d = o.dequantize(z["q_weight"], z["q_scale"], s, k)
            assert (d.view(np.uint16) == z["dequant"].view(np.uint16)).all()
        elif name.startswith("routing_"):
            t, ne = z["logits"].shape
            k = z["ids"].shape[1]
            w, ids = o.gating_softmax_topk(z["logits"], k)
            assert (ids == z["ids"]).all() and (w.view(np.uint16) == z["weights"].view(np.uint16)).all()
            cs = o.moe_cumsum(ids, ne)
            assert (cs == z["cumsum"]).all()
            rev, tok = o.get_indices(cs, ids)
            assert (rev == z["reverse_indices"]).all() and (tok == z["token_indices"]).all()
            assert (o.get_indptr(cs, ne, t, False) == z["indptr"]).all()
        elif name.startswith("moe_"):
            y = o.mixtral_moe(z["x"], z["logits"], z["q13"], z["s13"], z["q2"], z["s2"], Q4, 2)
            assert (y.view(np.uint16) == z["y"].view(np.uint16)).all()


# --------------------------------------------------------------------------- other model dtypes

def test_generic_dtype_oracle_reproduces_the_pinned_float16_one():
    # the float32 / bfloat16 restatement shares its code with a float16 instance; that instance must
    # be the float16 oracle pinned above, bit for bit (codes, scales, dequantised values)
    rng = np.random.default_rng(11)
    for name in ("q4f16_1", "q3f16_1"):
        s = o.SCHEMES[name]
        w = (rng.standard_normal((9, 203)) * 0.05).astype(np.float16)
        w[2, :80] = 0
        w[3, 5] = 60000.0
        for mode in ("half_away", "half_even"):
            qw, qs = o.quantize(w, s, mode)
            qw2, qs2 = o.quantize_dt(w.astype(np.float32), s, "float16", mode)
            assert np.array_equal(qw, qw2) and np.array_equal(qs.astype(np.float32), qs2)
        d = o.dequantize(qw, qs, s, 203)
        assert np.array_equal(d.astype(np.float32), o.dequantize_dt(qw, qs.astype(np.float32), s, 203, "float16"))


def test_bf16_rounding_known_values():
    x = np.array([1.0, 1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -8, 1.0 + 2.0 ** -8 + 2.0 ** -20, -2.5, 3.3895314e38, 3.4e38],
                 dtype=np.float32)
    want = np.array([1.0, 1.0, 1.015625, 1.0078125, -2.5, 3.3895314e38, np.inf], dtype=np.float32)
    assert np.array_equal(o.bf16_round(x), want)  # ties to even, overflow to infinity
    assert np.isnan(o.bf16_round(np.array([np.nan], dtype=np.float32))[0])
    # agrees with torch's conversion on random values
    import torch
    r = np.random.default_rng(3).standard_normal(20000).astype(np.float32) * 10
    assert np.array_equal(o.bf16_round(r), torch.from_numpy(r).bfloat16().float().numpy())


def test_float32_scheme_closed_forms():
    # float32 arithmetic: scale = max|w| / 7 exactly as numpy float32 divides; a weight equal to +-max
    # maps to 14 / 0; an all-zero group gives code 0 and scale 0; dequantize is (q - 7) * scale
    s = o.SCHEMES["q4f16_1"]
    rng = np.random.default_rng(5)
    w = rng.standard_normal((4, 96)).astype(np.float32)
    w[1, 32:64] = 0
    qw, qs = o.quantize_dt(w, s, "float32")
    q = o.unpack(qw, s, 96)
    assert np.array_equal(qs, (np.abs(w).reshape(4, 3, 32).max(-1) / np.float32(7)).astype(np.float32))
    g = np.abs(w).reshape(4, 3, 32)
    am = g.argmax(-1)
    for r in range(4):
        for gi in range(3):
            if r == 1 and gi == 1:
                assert (q[r, 32:64] == 0).all() and qs[r, gi] == 0
                continue
            k = gi * 32 + am[r, gi]
            assert q[r, k] == (14 if w[r, k] > 0 else 0)
    d = o.dequantize_dt(qw, qs, s, 96, "float32")
    assert np.array_equal(d, (q.astype(np.float32) - 7) * np.repeat(qs, 32, -1))
    assert np.abs(d - w).max() <= np.abs(qs).max() * 0.5000001


# --------------------------------------------------------------------------- silu * mul and the composed layer
#
# What fixes these without a run of the reference: silu(x) = x * sigmoid(x) is a closed form, so the fp32
# evaluation rounded once to the dtype is compared with torch's own silu (an independent implementation)
# and with float64 mathematics; the product of two halves is a single correctly rounded operation.  The
# composed layer is compared with a dense per-token form that has no gather, scatter, cumsum or indptr
# in it, over weights dequantised by the repeat-and-index formulation of the reference's own test.

def _ulp16_diff(a, b):
    """distance in fp16 representation steps (sign-magnitude to a monotone integer line)"""
    def line(v):
        u = np.asarray(v, np.float16).view(np.uint16).astype(np.int64)
        return np.where(u & 0x8000, -(u & 0x7FFF), u)
    return np.abs(line(a) - line(b))


def test_silu_mul_f16_against_closed_form_and_torch():
    import torch

    rng = np.random.default_rng(31)
    x1 = np.concatenate([rng.standard_normal(4000) * 3, np.linspace(-20, 20, 801),
                         np.array([0.0, -0.0, 1e-4, -1e-4, 30.0, -30.0, 65504.0, -65504.0, 6e-8])]).astype(np.float16)
    x3 = np.concatenate([rng.standard_normal(4000) * 2, rng.standard_normal(801),
                         np.array([5.0, 5.0, -3.0, 7.0, 2.0, 2.0, 1.0, 1.0, 1.0])]).astype(np.float16)
    got = o.silu_mul_f16(np.concatenate([x1, x3])[None, :])[0]
    # silu in float64 mathematics, rounded once to half, then the exact product rounded once to half
    x64 = x1.astype(np.float64)
    with np.errstate(over="ignore"):
        silu64 = x64 / (1.0 + np.exp(-x64))
    silu16 = silu64.astype(np.float16)
    with np.errstate(over="ignore", invalid="ignore"):
        want = (silu16.astype(np.float64) * x3.astype(np.float64)).astype(np.float16)
    # the oracle evaluates silu in fp32 before the rounding to half: it may land on the other side of a rounding
    # boundary of the float64 value in rare cases, never further
    ok = ~(np.isnan(want.astype(np.float32)) | np.isinf(want.astype(np.float32)))
    assert _ulp16_diff(got[ok], want[ok]).max() <= 1
    assert (got[ok].view(np.uint16) == want[ok].view(np.uint16)).mean() > 0.995
    # torch's silu on float32 (an independent implementation), rounded once, times x3 in half
    t_silu = torch.nn.functional.silu(torch.from_numpy(x1.astype(np.float32))).half()
    t_out = (t_silu * torch.from_numpy(x3)).numpy()
    assert _ulp16_diff(got[ok], t_out[ok]).max() <= 1
    # fixed points: silu(0) = 0 (either sign of zero gives a zero), silu(x) -> x for large x, -> -0 for large -x
    z = o.silu_mul_f16(np.array([[0.0, -0.0, 30.0, -30.0, 5.0, 5.0, 2.0, 2.0]], np.float16))[0]
    assert z[0] == 0 and z[1] == 0 and float(z[2]) == 60.0 and abs(float(z[3])) < 1e-6
    # the halves are not interchangeable: silu applies to the FIRST half (mixtral_model.py:66-68)
    a = o.silu_mul_f16(np.array([[4.0, 0.5]], np.float16))[0, 0]
    b = o.silu_mul_f16(np.array([[0.5, 4.0]], np.float16))[0, 0]
    assert float(a) == float(np.float16(np.float16(4.0 / (1 + np.exp(-4.0))) * np.float16(0.5)))
    assert float(a) != float(b)


@pytest.mark.parametrize("md", ["float32", "bfloat16", "float16"])
def test_silu_mul_dt_against_closed_form(md):
    rng = np.random.default_rng(37)
    x1 = o.round_to(np.concatenate([rng.standard_normal(3000) * 3, np.linspace(-15, 15, 301)]).astype(np.float32), md)
    x3 = o.round_to((rng.standard_normal(3301) * 2).astype(np.float32), md)
    got = o.silu_mul_dt(np.concatenate([x1, x3])[None, :], md)[0]
    x64 = x1.astype(np.float64)
    silu = o.round_to((x64 / (1.0 + np.exp(-x64))).astype(np.float32), md)
    want = o.round_to((silu.astype(np.float64) * x3.astype(np.float64)).astype(np.float32), md)
    # one unit of the dtype at most (fp32 evaluation against float64 before the rounding)
    # (float32: the fp32 exp, add and divide each round, a few units of the last place in all)
    eps = {"float32": 2.0 ** -20, "bfloat16": 2.0 ** -7, "float16": 2.0 ** -10}[md]
    assert (np.abs(got - want) <= eps * np.abs(want) + 1e-30).all()
    if md != "float32":
        assert (got == want).mean() > 0.99
    if md == "float16":  # the generic form is the float16 form
        h = o.silu_mul_f16(np.concatenate([x1, x3]).astype(np.float16)[None, :])[0]
        assert np.array_equal(h.astype(np.float32), got)


def _dense_moe_bruteforce(x, logits, q13, s13, q2, s2, s, top_k):
    """MixtralMoE.forward (mixtral_model.py:64-117) token by token, with no gather / scatter / cumsum / indptr:
    out[t] = sum_j w[t, j] * e2_id(silu(e1_id x) * e3_id x), fp16 wherever the reference stores fp16."""
    t, h = x.shape
    ne, n13, _ = q13.shape
    inter = n13 // 2
    w13 = np.stack([_dequant_by_repeat(s, q13[e], s13[e], (n13, h)) for e in range(ne)]).astype(np.float16)
    w2 = np.stack([_dequant_by_repeat(s, q2[e], s2[e], (h, inter)) for e in range(ne)]).astype(np.float16)
    out = np.zeros((t, h), np.float16)
    for ti in range(t):
        lg = logits[ti].astype(np.float64)
        order = sorted(range(ne), key=lambda e: (-lg[e], e))[:top_k]
        p = np.exp(lg[order] - lg[order].max())
        wts = (p / p.sum()).astype(np.float16)
        acc = None
        for j, e in enumerate(order):
            y13 = (w13[e].astype(np.float64) @ x[ti].astype(np.float64)).astype(np.float16)
            g64 = y13[:inter].astype(np.float64)
            act = (g64 / (1.0 + np.exp(-g64))).astype(np.float16)
            a = (act.astype(np.float64) * y13[inter:].astype(np.float64)).astype(np.float16)
            y2 = (w2[e].astype(np.float64) @ a.astype(np.float64)).astype(np.float16)
            term = (wts[j].astype(np.float64) * y2.astype(np.float64)).astype(np.float16)
            acc = term if acc is None else (acc.astype(np.float64) + term.astype(np.float64)).astype(np.float16)
        out[ti] = acc
    return out


@pytest.mark.parametrize("t", [1, 2, 3, 9, 40])
def test_mixtral_moe_against_dense_bruteforce(t):
    rng = np.random.default_rng(41 + t)
    ne, h, inter, top_k = 8, 64, 96, 2
    w13 = (rng.standard_normal((ne, 2 * inter, h)) * 0.2).astype(np.float16)
    w2 = (rng.standard_normal((ne, h, inter)) * 0.2).astype(np.float16)
    q13, s13 = o.quantize(w13, Q4)
    q2, s2 = o.quantize(w2, Q4)
    x = rng.standard_normal((t, h)).astype(np.float16)
    logits = rng.standard_normal((t, ne)).astype(np.float16)
    if t >= 3:
        logits[1] = logits[0]  # two tokens with the same experts, in order
        logits[2, :] = 0.5     # a full tie: experts 0 and 1
    got = o.mixtral_moe(x, logits, q13, s13, q2, s2, Q4, top_k)
    want = _dense_moe_bruteforce(x, logits, q13, s13, q2, s2, Q4, top_k)
    # rounding points are the same; the fp32 softmax / silu of the oracle may differ from float64 by a unit in
    # rare places, which the second matmul spreads: a few units at most, nothing like a wrong index or order
    d = _ulp16_diff(got, want)
    scale = np.abs(want.astype(np.float64)).max()
    assert np.abs(got.astype(np.float64) - want.astype(np.float64)).max() <= 4e-3 * scale
    assert (d <= 1).mean() > 0.98
    # the same check must reject a swapped weight order and a shifted scatter
    ids = o.gating_softmax_topk(logits, top_k)[1]
    if t > 1 and len(np.unique(ids)) > 2:
        wrong = o.mixtral_moe(x[::-1].copy(), logits, q13, s13, q2, s2, Q4, top_k)
        assert np.abs(wrong.astype(np.float64) - want.astype(np.float64)).max() > 0.05 * scale


@pytest.mark.parametrize("md", ["float32", "bfloat16"])
def test_mixtral_moe_dt_against_dense_bruteforce(md):
    rng = np.random.default_rng(43)
    ne, h, inter, top_k = 4, 64, 64, 2
    for t in (1, 7):
        w13 = o.round_to((rng.standard_normal((ne, 2 * inter, h)) * 0.2).astype(np.float32), md)
        w2 = o.round_to((rng.standard_normal((ne, h, inter)) * 0.2).astype(np.float32), md)
        q13, s13 = o.quantize_dt(w13, Q4, md)
        q2, s2 = o.quantize_dt(w2, Q4, md)
        x = o.round_to(rng.standard_normal((t, h)).astype(np.float32), md)
        logits = o.round_to(rng.standard_normal((t, ne)).astype(np.float32), md)
        got = o.mixtral_moe_dt(x, logits, q13, s13, q2, s2, Q4, md, top_k)
        r = lambda a: o.round_to(np.asarray(a, np.float64).astype(np.float32), md).astype(np.float64)
        d13 = np.stack([r((o.unpack(q13[e], Q4, h).astype(np.float64) - 7) * np.repeat(s13[e].astype(np.float64), 32, -1))
                        for e in range(ne)])
        d2 = np.stack([r((o.unpack(q2[e], Q4, inter).astype(np.float64) - 7) * np.repeat(s2[e].astype(np.float64), 32, -1))
                       for e in range(ne)])
        want = np.zeros((t, h))
        for ti in range(t):
            lg = logits[ti].astype(np.float64)
            order = sorted(range(ne), key=lambda e: (-lg[e], e))[:top_k]
            p = np.exp(lg[order] - lg[order].max())
            wts = r(p / p.sum())
            acc = None
            for j, e in enumerate(order):
                y13 = r(d13[e] @ x[ti].astype(np.float64))
                a = r(r(y13[:inter] / (1.0 + np.exp(-y13[:inter]))) * y13[inter:])
                term = r(wts[j] * r(d2[e] @ a))
                acc = term if acc is None else r(acc + term)
            want[ti] = acc
        scale = np.abs(want).max()
        tol = {"float32": 2e-5, "bfloat16": 3e-2}[md]
        assert np.abs(got.astype(np.float64) - want).max() <= tol * scale


def test_gating_topk_and_full_softmax_branch_brute_force():
    # moe_misc.py:63-132 and :234-235 (norm_topk_prob=False): softmax over all experts in fp32, cast to the
    # model dtype, then top-k of the ROUNDED scores with ties to the lower index
    rng = np.random.default_rng(47)
    t, ne, k = 64, 8, 2
    logits = rng.standard_normal((t, ne)).astype(np.float16)
    logits[5, :] = 1.0                      # all equal: scores all 1/8, experts 0, 1
    logits[6, [2, 6]] = 3.0                 # an exact tie at the top: 2 before 6
    logits[7] = np.array([0, 0, 0, 0, 0, 0, 0, 9], np.float16)
    w, ids = o.gating_softmax_topk_full(logits, k)
    assert ids[5].tolist() == [0, 1] and float(w[5, 0]) == 0.125 and float(w[5, 1]) == 0.125
    assert ids[6].tolist() == [2, 6] and w[6, 0] == w[6, 1]
    assert ids[7, 0] == 7
    p = np.exp(logits.astype(np.float64) - logits.astype(np.float64).max(-1, keepdims=True))
    p = p / p.sum(-1, keepdims=True)
    p16 = p.astype(np.float16)
    assert _ulp16_diff(o.softmax_fp32(logits.astype(np.float32)).astype(np.float16), p16).max() <= 1
    for r in range(t):
        s16 = o.softmax_fp32(logits[r: r + 1].astype(np.float32)).astype(np.float16)[0]
        order = sorted(range(ne), key=lambda e: (-float(s16[e]), e))[:k]
        assert ids[r].tolist() == order            # top-k of the rounded scores, ties to the lower index
        assert (w[r] == s16[order]).all()          # and the scores are returned as they are (no renormalisation)
        assert abs(float(w[r].astype(np.float64).sum())) <= 1.0 + 1e-3
    # unlike the norm_topk_prob=True branch the weights do not sum to one
    w_norm, ids_norm = o.gating_softmax_topk(logits, k)
    assert (ids_norm[8:] == ids[8:]).mean() > 0.95  # same experts away from rounding ties
    assert (w.astype(np.float32).sum(-1)[8:] < w_norm.astype(np.float32).sum(-1)[8:] - 0.05).all()
    # gating_topk alone: scores pass through unchanged
    sc = rng.random((5, 6)).astype(np.float16)
    v, i = o.gating_topk(sc, 3)
    for r in range(5):
        order = sorted(range(6), key=lambda e: (-float(sc[r, e]), e))[:3]
        assert i[r].tolist() == order and (v[r] == sc[r, order]).all()
