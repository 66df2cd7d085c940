"""Pins for the oracle's post-packing arithmetic: golden vectors of the reference's linear-layer test case,
brute force on small inputs, and independent bf16 arithmetic (torch CPU) for the rounding structure."""
import numpy as np
import pytest
import torch

from oracle import bf16, layout, linear, moe

F32 = np.float32


def tbits(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def test_bf16_against_torch():
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.standard_normal(100000).astype(F32) * 10.0 ** rng.integers(-30, 30, 100000),
                        np.array([0.0, -0.0, 1.0, 1.00390625, 1.01171875, np.inf, -np.inf, 3.3895314e38, 1e-40],
                                 F32)]).astype(F32)
    assert np.array_equal(bf16.to_bits(x), tbits(torch.from_numpy(x).to(torch.bfloat16)))
    b = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    f = bf16.from_bits(b)
    ok = ~np.isnan(f)
    assert np.array_equal(bf16.to_bits(f)[ok], b[ok])


def test_layer_case_golden(golden):
    """sim/make_testcase.py:47-60 through the oracle: same packed bytes, xq, xscale and y_ref."""
    x = golden["layer/x"].astype(np.float64)
    xq, xscale = linear.act_quant_f64(x)
    assert np.array_equal(xq, golden["layer/xq"])
    assert np.array_equal(xscale.astype(F32), golden["layer/xscale"])
    y = linear.float_reference(x, golden["layer/wq"], golden["layer/wscale"])
    assert np.array_equal(y, golden["layer/y_ref"])
    codes, bc, ws = layout.from_shift_layout(golden["layer/codes"], golden["layer/shifts"], golden["layer/wscale"])
    assert np.array_equal(layout.decode(codes, bc, *golden["layer/wq"].shape), golden["layer/wq"])
    assert np.array_equal(bc, golden["layer/shifts2"])         # 2-bit block codes == make_testcase's shifts2


def test_act_quant_scalar_bruteforce():
    rng = np.random.default_rng(1)
    x = bf16.rnd((rng.standard_normal((9, 64)) * rng.lognormal(0, 1, (1, 64))).astype(F32))
    x[4] = 0
    xq, xs = linear.act_quant(x, 12)
    assert xq.shape == (12, 64) and not xq[9:].any() and not xs[9:].any()
    for m in range(9):
        amax = F32(0)
        for v in x[m]:
            amax = max(amax, abs(F32(v)))
        s = F32(amax / F32(127))
        qi = F32(1) / s if s > 0 else F32(0)
        ref = [int(min(127, max(-127, np.rint(F32(F32(v) * qi))))) for v in x[m]]
        assert xs[m] == s and list(xq[m]) == ref
        if s > 0:
            assert np.abs(xq[m]).max() == 127
    # the reference's numpy twin (e2e/test_sc_kernels.py:21-26) written out
    s = (np.abs(x).max(1) / F32(127)).astype(F32)
    qi = np.where(s > 0, F32(1) / np.where(s > 0, s, 1), 0).astype(F32)
    assert np.array_equal(xq[:9], np.clip(np.rint(x * qi[:, None]), -127, 127).astype(np.int8))


def test_int_gemm_bruteforce():
    rng = np.random.default_rng(2)
    xq = rng.integers(-127, 128, (5, 96)).astype(np.int8)
    xq[0] = 127
    wq = rng.integers(-96, 97, (7, 96)).astype(np.int8)
    wq[0] = -96
    ref = np.array([[sum(int(a) * int(b) for a, b in zip(xr, wr)) for wr in wq] for xr in xq])
    assert np.array_equal(linear.int_gemm(xq, wq), ref)
    assert np.array_equal(linear.int_gemm(xq, wq), xq.astype(np.int64) @ wq.astype(np.int64).T)
    # worst case stays inside INT32: 127 * 96 * 6144
    assert 127 * 96 * 6144 < 2 ** 31


def test_epilogues_against_torch_bf16():
    rng = np.random.default_rng(3)
    m, n = 6, 16
    acc = rng.integers(-2 ** 26, 2 ** 26, (m, n)).astype(np.int32)
    acc[0, 0] = 2 ** 24 + 1            # int -> f32 conversion rounds (ties to even)
    xs = (np.abs(rng.standard_normal(m)) * 1e-3).astype(F32)
    ws = (np.abs(rng.standard_normal(n)) * 1e-4).astype(F32)
    res = bf16.to_bits(rng.standard_normal((m, n)).astype(F32))
    t = (torch.from_numpy(acc).to(torch.float32) * torch.from_numpy(xs)[:, None]) * torch.from_numpy(ws)[None]
    y_t = t.to(torch.bfloat16)
    assert np.array_equal(linear.epilogue(acc, xs, ws, 1), tbits(y_t))
    r_t = torch.from_numpy(res.view(np.int16)).view(torch.bfloat16)
    assert np.array_equal(linear.epilogue(acc, xs, ws, 2, res), tbits(r_t + y_t))
    # with a power-of-two weight scale the product is the exactly rounded float64 one
    ws2 = np.exp2(rng.integers(-12, -4, n)).astype(F32)
    exact = (acc.astype(np.float64) * xs.astype(np.float64)[:, None]).astype(F32) * ws2[None]
    assert np.array_equal(linear.epilogue(acc, xs, ws2, 1), bf16.to_bits(exact))


def test_exp_f32_all_bf16_inputs():
    b = np.arange(0x0000, 0x7F80, dtype=np.uint32).astype(np.uint16)       # every non-negative finite bf16
    a = bf16.from_bits(b)
    mine = linear.exp_f32(a)
    with np.errstate(over="ignore"):
        exact = np.exp(a.astype(np.float64))
    fin = exact < 3.3e38
    rel = np.abs(mine[fin].astype(np.float64) - exact[fin]) / exact[fin]
    assert rel.max() < 3e-7
    assert np.all(np.isinf(mine[exact > 3.5e38]))
    with np.errstate(over="ignore"):
        same = bf16.to_bits(mine) == bf16.to_bits(exact.astype(F32))
    assert same.all(), f"{(~same).sum()} bf16 inputs round differently from the exact exponential"


def test_swiglu_rounding_structure_against_torch():
    """Every op rounded to bf16, in the order of e2e/sc_kernels.py:319-328, for all 65536 gate patterns."""
    rng = np.random.default_rng(4)
    gb = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    gf = bf16.from_bits(gb)
    gb = np.where(np.isnan(gf) | np.isinf(gf), np.uint16(0), gb)
    ub = bf16.to_bits((rng.standard_normal(65536) * 3).astype(F32))
    g = torch.from_numpy(gb.view(np.int16)).view(torch.bfloat16)
    u = torch.from_numpy(ub.view(np.int16)).view(torch.bfloat16)
    e = torch.exp(g.abs().float()).to(torch.bfloat16)
    y = 1 / (1 + e)
    sig = torch.where(g < 0, y, 1 - y)
    ref = (g * sig) * u
    got = linear.swiglu(gb, ub)
    assert np.array_equal(got, tbits(ref))
    # and it is silu(g) * u to bf16 accuracy
    gf, uf = bf16.from_bits(gb).astype(np.float64), bf16.from_bits(ub).astype(np.float64)
    with np.errstate(over="ignore"):
        true = gf / (1 + np.exp(-gf)) * uf
    err = np.abs(bf16.from_bits(got).astype(np.float64) - true)
    inside = np.abs(true) < 3.3e38                      # beyond bf16 range the result is +-inf
    assert np.all(err[inside] <= 0.04 * np.abs(true[inside]) + 1e-30)


def test_epilogue_swiglu_column_pairing():
    rng = np.random.default_rng(5)
    m, f = 4, 8
    acc = rng.integers(-2 ** 20, 2 ** 20, (m, 2 * f)).astype(np.int32)        # rows [gate; up] -> columns here
    xs = np.full(m, 1e-4, F32)
    ws = np.exp2(-rng.integers(3, 8, 2 * f)).astype(F32)
    perm = linear.interleave_gate_up(f)
    assert list(perm[:8]) == [0, 1, f, f + 1, 2, 3, f + 2, f + 3]
    y = linear.scale_out(acc, xs, ws)
    ref = linear.swiglu(y[:, :f], y[:, f:])
    assert np.array_equal(linear.epilogue(acc[:, perm], xs, ws[perm], 3), ref)


def test_gemv_is_gemm_row():
    rng = np.random.default_rng(6)
    wq = rng.integers(-96, 97, (32, 256)).astype(np.int8)
    ws = np.exp2(-rng.integers(3, 8, 32)).astype(F32)
    xq = rng.integers(-127, 128, (3, 256)).astype(np.int8)
    xs = np.array([0.01, 0.02, 0.5], F32)
    full = linear.epilogue(linear.int_gemm(xq, wq), xs, ws, 1)
    assert np.array_equal(linear.gemv(xq, xs, wq, ws, 1), full)
    assert np.array_equal(linear.gemv(xq[1], xs[1], wq, ws, 1), full[1])


def test_rmsnorm_close_to_float64():
    rng = np.random.default_rng(7)
    x = bf16.to_bits((rng.standard_normal((5, 512)) * rng.lognormal(0, 1, (1, 512))).astype(F32))
    w = bf16.to_bits(rng.lognormal(0, 0.3, 512).astype(F32))
    got = bf16.from_bits(linear.rmsnorm(x, w, 1e-6)).astype(np.float64)
    xf, wf = bf16.from_bits(x).astype(np.float64), bf16.from_bits(w).astype(np.float64)
    ref = wf * xf / np.sqrt((xf ** 2).mean(1, keepdims=True) + 1e-6)
    assert linear.rel_fro(got, ref) < 5e-3
    ss = linear.row_sumsq(bf16.from_bits(x))
    assert np.allclose(ss, (xf ** 2).sum(1), rtol=1e-5)
    xq, xs, xn = linear.rmsnorm_quant(x, w, 1e-6, 8)
    assert xq.shape == (8, 512) and not xq[5:].any() and not xn[5:].any()


def test_route_sort_contract():
    rng = np.random.default_rng(8)
    m, topk, e, tm = 50, 4, 9, 16
    inds = np.stack([rng.permutation(e - 2)[:topk] for _ in range(m)])       # experts 7, 8 never chosen
    inds[inds == 3] = 2                                                       # expert 3 empty; duplicates allowed
    pos, tok, es, off, ts, mt = moe.route_sort(inds, e, tm)
    moe.check_route_sort(inds, e, tm, pos, tok, es, off, ts)
    assert mt == -(-m * topk // tm) + e and tok.shape == (m * topk + tm,)
    assert off[4] == off[3] and ts[4] == ts[3] and off[-1] == m * topk
    # brute force
    flat = inds.reshape(-1)
    rows = [i for ex in range(e) for i in range(len(flat)) if flat[i] == ex]
    assert [int(p) for p in np.argsort(pos)] == rows
    bad = pos.copy()
    bad[[0, 1]] = bad[[1, 0]]
    with pytest.raises(AssertionError):
        moe.check_route_sort(inds, e, tm, bad, tok, es, off, ts)


def test_combine_against_torch_bf16():
    """Sequential bf16 accumulation over the top-k axis then the residual (e2e/fused_olmoe.py:54-60), against torch
    bf16 scalar-order adds."""
    rng = np.random.default_rng(9)
    m, mp, topk, d = 7, 8, 4, 32
    ye = bf16.to_bits(rng.standard_normal((m, topk, d)).astype(F32))
    sc = bf16.to_bits(np.abs(rng.standard_normal((m, topk))).astype(F32))
    res = bf16.to_bits(rng.standard_normal((mp, d)).astype(F32))
    order = rng.permutation(m * topk)
    pos = np.empty(m * topk, np.int32)
    pos[order] = np.arange(m * topk)
    y_sorted = ye.reshape(m * topk, d)[order]
    h = moe.combine(y_sorted, pos, sc, res, m)
    tb = lambda a: torch.from_numpy(a.view(np.int16)).view(torch.bfloat16)
    acc = torch.zeros(m, d, dtype=torch.bfloat16)
    for j in range(topk):
        acc = (tb(ye)[:, j] * tb(sc)[:, j:j + 1]) + acc
    ref = tb(res).clone()
    ref[:m] = ref[:m] + acc
    assert np.array_equal(h, tbits(ref))


def test_moe_grouped_gemm_matches_per_expert():
    rng = np.random.default_rng(10)
    e, n, k, r = 4, 8, 64, 20
    wq = rng.integers(-96, 97, (e, n, k)).astype(np.int8)
    es = np.sort(rng.choice([0, 2, 3], r)).astype(np.int32)
    xq = rng.integers(-127, 128, (r, k)).astype(np.int8)
    acc = moe.moe_int_gemm(xq, es, wq)
    for i in range(r):
        assert np.array_equal(acc[i], wq[es[i]].astype(np.int64) @ xq[i].astype(np.int64))


def test_rot_blocks_is_a_scaled_hadamard_transform():
    """The butterfly order of rot_blocks (e2e/sc_kernels.py:231-256) is the Sylvester-ordered Walsh-Hadamard transform
    of each 32-block of x * signs, scaled by 1/sqrt(32): checked against the explicit matrix in float64; an
    orthonormal transform, so row norms are preserved; a constant block maps onto its first coefficient."""
    rng = np.random.default_rng(3)
    x = bf16.rnd(rng.standard_normal((6, 256)).astype(np.float32))
    signs = linear.rot_signs(256)
    assert set(np.unique(signs)) == {-1.0, 1.0} and np.array_equal(signs, linear.rot_signs(256))
    i = np.arange(32)
    h = (-1.0) ** np.array([[bin(a & b).count("1") for b in i] for a in i])
    want = ((x * signs).astype(np.float64).reshape(6, 8, 32) @ h.T / np.sqrt(32)).reshape(6, 256)
    got = linear.rot_blocks(x, signs).astype(np.float64)
    assert np.abs(got - want).max() <= 2.0 ** -8 * np.abs(want).max()          # one bf16 rounding
    assert np.allclose(np.linalg.norm(got, axis=1), np.linalg.norm(x, axis=1), rtol=5e-3)
    ones = linear.rot_blocks(np.ones((1, 32), np.float32), np.ones(32, np.float32))
    assert ones[0, 0] == bf16.rnd(np.float32(32) * linear.ROT_NORM) and not ones[0, 1:].any()
    xq, xs = linear.rot_quant(x, signs, 8)
    assert xq.shape == (8, 256) and not xq[6:].any() and xs[6] == 0 and np.abs(xq[:6]).max() == 127
