"""Pins for the oracle's RMSNorm family (`linear.row_sumsq`, `rmsnorm`, `rmsnorm_quant`, `res_norm_quant`,
`swiglu_quant`, `headnorm`, `fullnorm`) against what the reference's kernel text fixes and an independent bf16
implementation can check (torch CPU bfloat16 ops): which product is rounded to bf16 and in which order
(`w * T(x * inv)`, e2e/sc_kernels.py:139), where `eps` sits (`rsqrt(ss / K + eps)`, :133), which slice of the row a
head's statistics cover and which weight vector it takes (:359-380), the whole-width statistics of :388-423, the
head-major output order, and that the fused kernels are the composition of their parts (:177-189, :279-315).
Every structural check is paired with a deliberately wrong variant that must differ on the same data, so that the
check cannot pass for an oracle with that mistake.

What stays open: the summation ORDER inside the sum of squares (MLX's 32-lane simd_sum tree against this build's
64-lane butterfly) and metal::precise::rsqrt against IEEE 1/sqrt.  MLX is not installable here, so no vector can
settle those; they move `inv` by a few FP32 ulps at most, which `test_row_sumsq_*` bounds."""
import math

import numpy as np
import pytest
import torch

from oracle import bf16, linear

F32 = np.float32
EPS = 1e-6


def tb(bits):
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).view(torch.bfloat16)


def tbits(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def acts(rng, m, k):
    return bf16.to_bits((rng.standard_normal((m, k)) * rng.lognormal(0, 1, (1, k))).astype(F32))


def gains(rng, k):
    return bf16.to_bits(rng.lognormal(0, 0.3, k).astype(F32))


def oracle_inv(x_bits, eps=EPS):
    x = bf16.from_bits(x_bits)
    return (F32(1) / np.sqrt(linear.row_sumsq(x) / F32(x.shape[1]) + F32(eps))).astype(F32)


def torch_norm(x_bits, w_bits, inv):
    """w * bf16(float(x) * inv) with torch's bf16 arithmetic, the FP32 `inv` handed in."""
    xn = (tb(x_bits).float() * torch.from_numpy(inv)[:, None]).to(torch.bfloat16)
    return tbits(tb(w_bits)[None, :] * xn)


# ---- (a) rounding structure of rmsnorm -----------------------------------------------------------------------------

@pytest.mark.parametrize("k", [128, 512, 2048, 6144])
def test_rmsnorm_rounding_structure_against_torch(k):
    rng = np.random.default_rng(k)
    x, w = acts(rng, 9, k), gains(rng, k)
    inv = oracle_inv(x)
    got = linear.rmsnorm(x, w, EPS)
    assert np.array_equal(got, torch_norm(x, w, inv))
    # the wrong orders: one rounding of the triple product, and the weight applied before the statistic's scale
    one_rounding = tbits((tb(w).float()[None, :] * tb(x).float() * torch.from_numpy(inv)[:, None]).to(torch.bfloat16))
    weight_first = tbits(((tb(w)[None, :] * tb(x)).float() * torch.from_numpy(inv)[:, None]).to(torch.bfloat16))
    assert (got != one_rounding).any() and (got != weight_first).any()
    # and it is an RMSNorm: within two bf16 roundings of the float64 value, element by element
    xf, wf = bf16.from_bits(x).astype(np.float64), bf16.from_bits(w).astype(np.float64)
    ref = wf * xf / np.sqrt((xf ** 2).mean(1, keepdims=True) + EPS)
    assert np.all(np.abs(bf16.from_bits(got) - ref) <= 2.0 ** -7 * np.abs(ref) + 1e-30)


def test_rmsnorm_uses_the_row_mean_not_the_row_sum():
    """ss / K inside the root: a row of equal values c normalises to +-1 whatever K is."""
    for k in (64, 256, 1024):
        x = bf16.to_bits(np.full((1, k), 3.0, F32))
        x[0, ::2] ^= 0x8000
        w = bf16.to_bits(np.ones(k, F32))
        y = bf16.from_bits(linear.rmsnorm(x, w, 0.0))
        assert np.array_equal(np.abs(y), np.ones((1, k), F32))
        assert np.array_equal(np.signbit(y), np.signbit(bf16.from_bits(x)))


# ---- (b) the sum of squares and eps --------------------------------------------------------------------------------

@pytest.mark.parametrize("k", [4, 64, 100, 256, 260, 2048, 6144, 16384])
def test_row_sumsq_within_ulps_of_exact(k):
    rng = np.random.default_rng(k)
    x = bf16.from_bits(acts(rng, 6, k))
    got = linear.row_sumsq(x)
    for r in range(x.shape[0]):
        exact = math.fsum(float(v) * float(v) for v in x[r])
        # a tree of FP32 adds over K terms: error below (log2(K) + 4) half-ulps of the total
        assert abs(float(got[r]) - exact) <= (math.log2(k) + 4) * 2.0 ** -24 * exact


def test_row_sumsq_counts_every_element_once():
    """Basis rows: a single 1 at any column sums to exactly 1; a single column doubled adds exactly 3."""
    k = 772                                           # 193 virtual threads: three full waves and a ragged fourth
    assert np.array_equal(linear.row_sumsq(np.eye(k, dtype=F32)), np.ones(k, F32))
    base = np.ones((k, k), F32)
    bumped = base + np.eye(k, dtype=F32)
    assert np.array_equal(linear.row_sumsq(bumped) - linear.row_sumsq(base), np.full(k, 3, F32))


def test_eps_sits_inside_the_square_root():
    k = 256
    zero = np.zeros((1, k), np.uint16)
    w = bf16.to_bits(np.ones(k, F32))
    assert not linear.rmsnorm(zero, w, EPS).any()
    assert oracle_inv(zero, EPS)[0] == F32(1) / np.sqrt(F32(EPS))
    # a row whose mean square equals eps: inv = 1/sqrt(2 eps), not 1/(sqrt(eps) + eps) or 1/sqrt(eps)
    c = F32(2.0 ** -10)
    x = bf16.to_bits(np.full((1, k), c, F32))
    eps = float(c) ** 2
    assert oracle_inv(x, eps)[0] == F32(1) / np.sqrt(F32(2 * eps))
    y = bf16.from_bits(linear.rmsnorm(x, w, eps))
    assert np.array_equal(y, np.full((1, k), bf16.rnd(np.array(c * (F32(1) / np.sqrt(F32(2 * eps))), F32)), F32))


# ---- (c) per-head norm ---------------------------------------------------------------------------------------------

@pytest.mark.parametrize("d", [64, 128, 256])
def test_headnorm_is_rmsnorm_per_head_slice(d):
    rng = np.random.default_rng(d)
    hq, hk, length, mp = 4, 2, 11, 16
    y = acts(rng, mp, (hq + 2 * hk) * d)
    qn, kn = gains(rng, d), gains(rng, d)
    q, k, v = linear.headnorm(y, qn, kn, EPS, length, hq, hk, d)
    assert q.shape == (hq, length, d) and k.shape == (hk, length, d) and v.shape == (hk, length, d)
    heads = y[:length].reshape(length, hq + 2 * hk, d)
    for h in range(hq + hk):
        sl = np.ascontiguousarray(heads[:, h])
        inv = oracle_inv(sl)
        want = torch_norm(sl, qn if h < hq else kn, inv)
        got = q[h] if h < hq else k[h - hq]
        assert np.array_equal(got, want), f"head {h}"
        # the statistic is the head's own: FP32-close to the float64 mean square of that slice only
        sf = bf16.from_bits(sl).astype(np.float64)
        assert np.allclose(inv, 1 / np.sqrt((sf ** 2).mean(1) + EPS), rtol=2e-6)
    # q heads use qn and k heads kn: with the weights swapped every head changes
    qs, ks, _ = linear.headnorm(y, kn, qn, EPS, length, hq, hk, d)
    assert all((qs[h] != q[h]).any() for h in range(hq)) and all((ks[h] != k[h]).any() for h in range(hk))
    # v passes through untouched, head-major
    assert np.array_equal(v, heads[:, hq + hk:].transpose(1, 0, 2))
    # rows past `length` are not read
    y2 = y.copy()
    y2[length:] ^= 0x1234
    assert all(np.array_equal(a, b) for a, b in zip(linear.headnorm(y2, qn, kn, EPS, length, hq, hk, d), (q, k, v)))


def test_headnorm_matches_reference_test_shapes_against_torch_rmsnorm():
    """The check of e2e/test_sc_kernels.py:95-108 with torch in MLX's place: q / k equal a float64-statistic RMSNorm
    of each head to within the bf16 rounding of `x * inv`, at the Qwen3-1.7B head layout."""
    rng = np.random.default_rng(5)
    hq, hk, d, length = 16, 8, 128, 40
    y = acts(rng, 48, (hq + 2 * hk) * d)
    qn, kn = gains(rng, d), gains(rng, d)
    q, k, v = linear.headnorm(y, qn, kn, EPS, length, hq, hk, d)
    lin = bf16.from_bits(y[:length]).astype(np.float64).reshape(length, hq + 2 * hk, d)
    for out, w, first in ((q, qn, 0), (k, kn, hq)):
        part = lin[:, first:first + out.shape[0]]
        ref = bf16.from_bits(w).astype(np.float64) * part / np.sqrt((part ** 2).mean(-1, keepdims=True) + EPS)
        got = bf16.from_bits(out).astype(np.float64).transpose(1, 0, 2)
        assert np.all(np.abs(got - ref) <= 2.0 ** -7 * np.abs(ref) + 1e-30)
    assert np.array_equal(bf16.from_bits(v).transpose(1, 0, 2), lin[:, hq + hk:].astype(F32))


# ---- (d) whole-width q / k norm ------------------------------------------------------------------------------------

def test_fullnorm_is_rmsnorm_over_all_heads():
    rng = np.random.default_rng(6)
    h, d, length, mp = 4, 64, 9, 16
    w = h * d
    y = acts(rng, mp, 3 * w)
    qn, kn = gains(rng, w), gains(rng, w)
    q, k, v = linear.fullnorm(y, qn, kn, EPS, length, h, d)
    assert q.shape == k.shape == v.shape == (h, length, d)
    for out, wt, c0 in ((q, qn, 0), (k, kn, w)):
        sl = np.ascontiguousarray(y[:length, c0:c0 + w])
        want = torch_norm(sl, wt, oracle_inv(sl)).reshape(length, h, d).transpose(1, 0, 2)
        assert np.array_equal(out, want)
    assert np.array_equal(v, y[:length, 2 * w:].reshape(length, h, d).transpose(1, 0, 2))
    # not a per-head norm: scaling one head's inputs changes the other heads' outputs
    y2 = y.copy()
    y2[:length, :d] = bf16.to_bits(bf16.from_bits(y[:length, :d]) * F32(8))
    q2, _, _ = linear.fullnorm(y2, qn, kn, EPS, length, h, d)
    assert (q2[1:] != q[1:]).any()
    qs, ks, _ = linear.fullnorm(y, kn, qn, EPS, length, h, d)
    assert (qs != q).any() and (ks != k).any()


# ---- (e) the fused kernels are compositions of pinned parts --------------------------------------------------------

def test_rmsnorm_quant_is_rmsnorm_then_act_quant():
    rng = np.random.default_rng(7)
    m, mp, k = 5, 8, 512
    x, w = acts(rng, m, k), gains(rng, k)
    xq, xs, xn = linear.rmsnorm_quant(x, w, EPS, mp)
    n = linear.rmsnorm(x, w, EPS)
    cq, cs = linear.act_quant(bf16.from_bits(n))
    assert np.array_equal(xn[:m], n) and np.array_equal(xq[:m], cq) and np.array_equal(xs[:m], cs)
    assert xq.shape == (mp, k) and not xq[m:].any() and not xs[m:].any() and not xn[m:].any()
    # the quantization sees the bf16-rounded normalised row (e2e/sc_kernels.py:139-141), not the FP32 product
    xf = bf16.from_bits(w)[None, :] * bf16.rnd(bf16.from_bits(x) * oracle_inv(x)[:, None])
    fq, _ = linear.act_quant(xf.astype(F32))
    assert (fq != cq).any()


def test_res_norm_quant_is_residual_epilogue_then_rmsnorm_quant():
    """e2e/sc_kernels.py:177-189 and the check of e2e/test_sc_kernels.py:66-76: h = res + bf16(acc xs ws) in bf16
    (torch bf16 add as the independent implementation), then rmsnorm_quant of h."""
    rng = np.random.default_rng(8)
    mp, k = 8, 256
    acc = rng.integers(-2 ** 20, 2 ** 20, (mp, k)).astype(np.int32)
    xs = (np.abs(rng.standard_normal(mp)) * 1e-3).astype(F32)
    ws = (np.abs(rng.standard_normal(k)) * 1e-3).astype(F32)
    res, w = acts(rng, mp, k), gains(rng, k)
    h, xq, xs2 = linear.res_norm_quant(acc, xs, ws, res, w, EPS)
    lin = ((torch.from_numpy(acc).float() * torch.from_numpy(xs)[:, None]) * torch.from_numpy(ws)[None, :])
    h_ref = tb(res) + lin.to(torch.bfloat16)
    assert np.array_equal(h, tbits(h_ref))
    cq, cs, _ = linear.rmsnorm_quant(h, w, EPS)
    assert np.array_equal(xq, cq) and np.array_equal(xs2, cs)
    assert np.array_equal(linear.res_epilogue(acc, xs, ws, res), h)


def test_swiglu_quant_is_scale_swiglu_act_quant():
    """e2e/sc_kernels.py:279-315: gate = columns [0, F), up = [F, 2F) of bf16(acc xs ws), not interleaved."""
    rng = np.random.default_rng(9)
    mp, f = 6, 128
    acc = rng.integers(-2 ** 18, 2 ** 18, (mp, 2 * f)).astype(np.int32)
    xs = (np.abs(rng.standard_normal(mp)) * 1e-4).astype(F32)
    ws = np.exp2(-rng.integers(3, 8, 2 * f)).astype(F32)
    xq, s = linear.swiglu_quant(acc, xs, ws)
    y = linear.scale_out(acc, xs, ws)
    a = linear.swiglu(y[:, :f], y[:, f:])
    cq, cs = linear.act_quant(bf16.from_bits(a))
    assert np.array_equal(xq, cq) and np.array_equal(s, cs)
    swapped, _ = linear.act_quant(bf16.from_bits(linear.swiglu(y[:, f:], y[:, :f])))
    assert (swapped != xq).any()
