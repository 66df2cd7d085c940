"""The oracle's quantizer, embedding and packed layouts against vectors written from the reference's own numpy
modules, plus the invariants the reference's self-tests assert (sim/mx_int8.py:194-209, e2e/sc_format.py:114-127)."""
import hashlib

import numpy as np
import pytest

from oracle import family, layout, quantizer as Q

SMALL = ("lognormal_cols", "llm_outlier_cols", "wide_exponents_zeros", "midpoints")


def sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def test_round_e2m1_golden(golden):
    out = Q.round_e2m1(golden["e2m1_in"])
    assert np.array_equal(out, golden["e2m1_out"])
    assert np.array_equal(np.signbit(out), np.signbit(golden["e2m1_out"]))


def test_round_e2m1_closed_form():
    # every midpoint goes to the lower level; one ulp above goes up; saturation at 6
    for lo, hi in zip(Q.LEVELS[:-1], Q.LEVELS[1:]):
        mid = (lo + hi) / 2
        assert Q.round_e2m1(mid) == lo and Q.round_e2m1(-mid) == -lo
        assert Q.round_e2m1(np.nextafter(mid, 10)) == hi
        assert Q.round_e2m1(np.nextafter(mid, -10)) == lo
    assert Q.round_e2m1(1e9) == 6 and Q.round_e2m1(-1e9) == -6
    # brute force: nearest level by exhaustive distance, ties down
    x = np.linspace(-7, 7, 5001)
    d = np.abs(np.abs(np.minimum(np.abs(x), 6.0))[:, None] - Q.LEVELS[None])
    assert np.array_equal(np.abs(Q.round_e2m1(x)), Q.LEVELS[d.argmin(1)])


@pytest.mark.parametrize("name", SMALL)
def test_exponents_golden(golden, name):
    w = golden[f"w/{name}"]
    for rule in ("spec", "search"):
        assert np.array_equal(Q.block_exponents(w, rule), golden[f"e_{rule}/{name}"]), rule
    e = Q.constrain_spread(Q.block_exponents(w, "search"))
    assert np.array_equal(e, golden[f"e_sc/{name}"])
    v, wdq = Q.e2m1_values(w, e)
    assert np.array_equal(v, golden[f"v/{name}"]) and np.array_equal(wdq, golden[f"wdq/{name}"])
    q, shift, e_lo, scale = Q.embed_int8(v, e)
    assert np.array_equal(q, golden[f"q/{name}"])
    assert np.array_equal(scale, golden[f"sc/{name}"][:, 0])


@pytest.mark.parametrize("name", SMALL)
def test_pack_golden(golden, name):
    w = golden[f"w/{name}"]
    packed, shifts, wscale, qw = Q.pack(w)
    assert np.array_equal(packed, golden[f"packed/{name}"])
    assert np.array_equal(shifts, golden[f"shifts/{name}"])
    assert np.array_equal(wscale, golden[f"wscale/{name}"]) and wscale.dtype == np.float32
    assert np.array_equal(qw, golden[f"qw/{name}"])
    # pack from (values, exponents) with no requantization gives the same bytes (e2e/gptq_pack.py:29-47)
    again = Q.pack_from_values(golden[f"v/{name}"], golden[f"e_sc/{name}"])
    assert all(np.array_equal(a, b) for a, b in zip(again, (packed, shifts, wscale, qw)))
    codes, bc, ws, q2 = layout.quantize(w)
    assert np.array_equal(codes, golden[f"codes/{name}"]) and np.array_equal(bc, golden[f"bcodes/{name}"])
    assert np.array_equal(layout.decode(codes, bc, *w.shape), qw)


BIG = {
    "selftest_mx_int8": lambda: (lambda r: r.standard_normal((64, 1024)) * r.lognormal(0, 1.0, (1, 1024)))(
        np.random.default_rng(0)),
    "selftest_sc_format": lambda: (lambda r: r.standard_normal((64, 512)) * 0.02 * r.lognormal(0, 0.3, (1, 512)))(
        np.random.default_rng(0)),
    "test_sc_kernels_384x2048": lambda: (lambda r: r.standard_normal((384, 2048)) * 0.02
                                         * r.lognormal(0, 0.3, (1, 2048)))(np.random.default_rng(0)),
}


def _config0_like():
    rng = np.random.default_rng(7)
    w = rng.standard_normal((256, 2048)) * 0.02
    w[:, rng.choice(2048, 10, replace=False)] *= 8
    return w


BIG["config0_like_256x2048"] = _config0_like


@pytest.mark.parametrize("name", sorted(BIG))
def test_pack_digests(golden, name):
    got = [sha(a) for a in Q.pack(BIG[name]())]
    assert got == list(golden[f"sha/{name}"])


def test_reference_selftest_invariants():
    """sim/mx_int8.py:194-209: spread <= 3, q * scale == dequantized weights, and the INT8 GEMM times the row
    scale equals x @ Wq^T exactly."""
    rng = np.random.default_rng(0)
    w = rng.standard_normal((64, 1024)) * rng.lognormal(0, 1.0, (1, 1024))
    e = Q.constrain_spread(Q.block_exponents(w, "search"))
    assert Q.exponent_spread(e).max() <= 3
    v, wdq = Q.e2m1_values(w, e)
    q, shift, e_lo, scale = Q.embed_int8(v, e)
    assert np.abs(q).max() <= 96 and shift.max() <= 3
    assert np.array_equal(q * scale[:, None], wdq)
    x = rng.integers(-127, 128, (8, 1024)).astype(np.float64)
    assert np.array_equal((x @ q.astype(np.float64).T) * scale[None], x @ wdq.T)


def test_embed_rejects_wide_rows():
    v = np.ones((1, 2, 32))
    with pytest.raises(ValueError):
        Q.embed_int8(v, np.array([[0.0, 4.0]]))


def test_block16_runs_same_procedure():
    rng = np.random.default_rng(5)
    w = rng.standard_normal((32, 256)) * 0.02
    w[:, 3] *= 8
    fmt = layout.Format(block=16)
    codes, bc, ws, q = layout.quantize(w, fmt)
    assert np.array_equal(layout.decode(codes, bc, 32, 256, fmt), q)
    assert np.all(np.log2(ws) == np.rint(np.log2(ws)))          # power-of-two row scale
    # finer blocks never lose accuracy against 32-blocks on the same data
    _, _, ws32, q32 = layout.quantize(w)
    e16 = ((q * ws[:, None].astype(np.float64) - w) ** 2).sum()
    e32 = ((q32 * ws32[:, None].astype(np.float64) - w) ** 2).sum()
    assert e16 <= e32 * 1.05


@pytest.mark.parametrize("i", range(5))
def test_layout_random_codes_golden(golden, i):
    kw = [dict(), dict(block=16), dict(block=32, mult=(1, 2, 3, 4)),
          dict(block=16, mult=(1, 2, 3, 4, 5, 6, 8, 10), bc_bits=4),
          dict(block=32, code_mag=(0, 1, 2, 3, 4, 5, 6, 7), mult=(1, 3, 9, 15))][i]
    f = layout.Format(**kw)
    c4, b = golden[f"fmt{i}/c4"], golden[f"fmt{i}/b"]
    codes, bc, ws = layout.pack_rows(c4, b, golden[f"fmt{i}/ws"], f)
    assert np.array_equal(codes, golden[f"fmt{i}/codes"]) and codes.dtype == np.uint32
    assert np.array_equal(bc, golden[f"fmt{i}/bc"])
    q = layout.decode(codes, bc, 8, 256, f)
    assert np.array_equal(q, golden[f"fmt{i}/q"])
    # the decode formula, element by element (e2e/sc_format.py:8)
    mag = np.array(f.code_mag)[c4 & 7] * np.repeat(np.array(f.mult)[b], f.block, axis=1)
    assert np.array_equal(q, np.where(c4 & 8, -mag, mag))
    c4b, bb = layout.unpack_fields(codes, bc, 8, 256, f)
    assert np.array_equal(c4b, c4) and np.array_equal(bb, b)


def test_format_invariants():
    for bad in (dict(block=12), dict(bc_bits=3), dict(mult=(1, 2, 4, 8, 16)), dict(mult=(1, 16))):
        with pytest.raises(ValueError):
            layout.Format(**bad)
    assert abs(layout.DEFAULT.bits_per_weight(4096) - 4.0703125) < 1e-12


def test_mxfp4_view_closed_form(golden):
    """E8M0 = log2(wscale) + 1 + shift + 127 and the value is e2m1 * 2^(E8M0 - 127) (e2e/fused_qwen38.py:319-334)."""
    w = golden["w/llm_outlier_cols"]
    codes, bc, ws, q = layout.quantize(w)
    n, k = w.shape
    nib, e8 = layout.to_mxfp4(codes, bc, ws, n, k)
    c = np.stack([nib & 0xF, nib >> 4], -1).reshape(n, k)
    val = np.where(c & 8, -1.0, 1.0) * Q.LEVELS[c & 7] * np.exp2(np.repeat(e8.astype(np.float64), 32, 1) - 127)
    assert np.array_equal(val, q.astype(np.float64) * ws[:, None].astype(np.float64))
    assert np.array_equal(val, golden["wdq/llm_outlier_cols"])
    c2, b2, w2 = layout.from_mxfp4(nib, e8)
    assert np.array_equal(c2, codes) and np.array_equal(b2, bc) and np.array_equal(w2, ws)
    e8[0, 0] += 5
    with pytest.raises(ValueError):
        layout.from_mxfp4(nib, e8)


@pytest.mark.parametrize("name", ["e2m1/B16/pow2", "e2m1/B16/M1..10", "e2m1/B32/M1..8", "int4/B16/M1..16"])
def test_family_quantizer_golden(golden, name):
    key = name.replace("/", "_")
    fam = family.member(name)
    wq, qi, base, scales = family.quantize(golden["fam/w"], fam)
    assert np.array_equal(qi, golden[f"fam/{key}/qi"])
    assert np.array_equal(base, golden[f"fam/{key}/base"])
    assert np.array_equal(scales, golden[f"fam/{key}/scales"])
    assert np.array_equal(wq, golden[f"fam/{key}/wq"])
    sf = fam.storage()
    spec = golden[f"fam/{key}/fmt"]
    assert [sf.block, sf.bc_bits, len(sf.mult)] + list(sf.code_mag) + list(sf.mult) == list(spec)
    codes, bc, ws = family.pack_parts(qi, base, scales, sf)
    assert np.array_equal(codes, golden[f"fam/{key}/codes"]) and np.array_equal(bc, golden[f"fam/{key}/bc"])
    assert np.array_equal(ws, golden[f"fam/{key}/ws"])
    # sim/formats.py:136-148: stored form reproduces the weights
    assert np.array_equal(qi.astype(np.float32) * base[:, None], wq)
