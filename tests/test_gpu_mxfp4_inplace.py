"""A standard MXFP4 tensor read in place (E2M1 nibble bytes + one E8M0 byte per 32-block, e2e/fused_qwen38.py:319-334;
`sc_format.MXFP4`): the GEMV, the dense GEMM and the grouped GEMM give, bit for bit, what the oracle gives for the
INT8 embedding of the same tensor (`oracle/layout.from_mxfp4` -> `decode`), and what the kernels give on the
converted 2-bit form."""
import numpy as np
import pytest
import torch

from oracle import bf16, layout, linear, moe
from tests.util import dev, host, llm_acts, llm_weights

pytestmark = pytest.mark.gpu
F32 = np.float32


@pytest.fixture(scope="module")
def F():
    from mxfp4_int8_m5_amd import sc_format
    return sc_format


@pytest.fixture(scope="module")
def G():
    from mxfp4_int8_m5_amd import sc_decode
    return sc_decode


@pytest.fixture(scope="module")
def S():
    from mxfp4_int8_m5_amd import sc_kernels
    return sc_kernels


def mxfp4_tensor(rng, n, k, base=None):
    """(nibbles, e8m0) of a quantized N(0, 0.02) matrix with outlier columns, its oracle embedding q and row scales.
    `base` moves every row's exponents (rows then differ in their lowest byte)."""
    codes, bc, ws, q = layout.quantize(llm_weights(rng, n, k))
    if base is not None:
        ws = (ws * np.exp2(base)).astype(F32)
    nib, e8 = layout.to_mxfp4(codes, bc, ws, n, k)
    c2, b2, w2 = layout.from_mxfp4(nib, e8)                 # the oracle's reading of the standard tensor
    assert np.array_equal(layout.decode(c2, b2, n, k), q) and np.array_equal(w2, ws)
    return nib, e8, q, ws


def on_device(F, nib, e8):
    dn, de = dev(nib), dev(e8)
    return F.mxfp4_codes(dn), de, F.mxfp4_row_scales(de)


def test_row_scales_and_rejections(F):
    rng = np.random.default_rng(0)
    n, k = 96, 512
    nib, e8, q, ws = mxfp4_tensor(rng, n, k, base=rng.integers(-20, 6, n))
    assert np.array_equal(host(F.mxfp4_row_scales(dev(e8))), ws)
    bad = e8.copy()
    bad[3, 0] = bad[3].min() + 4
    with pytest.raises(ValueError):
        F.mxfp4_row_scales(dev(bad))
    bad = e8.copy()
    bad[5] = 0
    with pytest.raises(ValueError):
        F.mxfp4_row_scales(dev(bad))
    with pytest.raises(ValueError):                          # the INT8 tensor needs the converted form
        from mxfp4_int8_m5_amd import sc_kernels
        sc_kernels.unpack_i8(F.mxfp4_codes(dev(nib)), dev(e8), n, k, lazy=False, fmt=F.MXFP4, wscale=dev(ws))


@pytest.mark.parametrize("n,k", [(256, 2048), (512, 6144), (64, 1024), (20, 128), (4096, 2048), (36864, 512)])
def test_gemv_batch1_every_epilogue_and_prologue(F, G, n, k):
    rng = np.random.default_rng(n + k)
    nib, e8, q, ws = mxfp4_tensor(rng, n, k, base=rng.integers(-12, 4, n))
    dc, de, dw = on_device(F, nib, e8)
    assert np.array_equal(host(dw), ws)
    xq = rng.integers(-127, 128, k).astype(np.int8)
    xq[:16] = 127
    xs = np.array([0.01], F32)
    ref1 = linear.gemv(xq, xs[0], q, ws, 1)
    assert np.array_equal(host(G.gemv(dev(xq), dc, de, dev(xs), dw, n, 1, fmt=F.MXFP4)), ref1)
    res = bf16.to_bits(rng.standard_normal(n).astype(F32))
    y2 = host(G.gemv(dev(xq), dc, de, dev(xs), dw, n, 2, res=dev(res), fmt=F.MXFP4))
    assert np.array_equal(y2, linear.gemv(xq, xs[0], q, ws, 2, res))
    perm = linear.interleave_gate_up(n // 2)
    dcp, dep, dwp = on_device(F, nib[perm], e8[perm])
    y3 = host(G.gemv(dev(xq), dcp, dep, dev(xs), dwp, n, 3, fmt=F.MXFP4))
    with np.errstate(all="ignore"):
        assert np.array_equal(y3, linear.swiglu(ref1[:n // 2], ref1[n // 2:]))
    xb, x = llm_acts(rng, 1, k)
    rq, rs = linear.act_quant(x)
    yp = host(G.gemv(dev(xb)[0], dc, de, None, dw, n, 1, pro=1, fmt=F.MXFP4))
    assert np.array_equal(yp, linear.gemv(rq[0], rs[0], q, ws, 1))
    nw = bf16.to_bits(rng.lognormal(0, 0.3, k).astype(F32))
    nq, ns, _ = linear.rmsnorm_quant(xb, nw, 1e-6)
    yn = host(G.gemv(dev(xb)[0], dc, de, None, dw, n, 1, pro=2, nw=dev(nw), eps=1e-6, fmt=F.MXFP4))
    assert np.array_equal(yn, linear.gemv(nq[0], ns[0], q, ws, 1))


@pytest.mark.parametrize("batch", [2, 4, 8])
@pytest.mark.parametrize("n,k", [(2048, 2048), (512, 6144), (33280, 1024), (100, 384)])
def test_gemv_batches(F, G, n, k, batch):
    """Wide layers (half-precision MFMA kernel), narrow ones (the same split over K) and shapes neither takes."""
    rng = np.random.default_rng(n + k + batch)
    nib, e8, q, ws = mxfp4_tensor(rng, n, k, base=rng.integers(-12, 4, n))
    dc, de, dw = on_device(F, nib, e8)
    xq = rng.integers(-127, 128, (batch, k)).astype(np.int8)
    xq[0, :32] = -127
    xs = (rng.random(batch) * 0.02 + 1e-3).astype(F32)
    ref = linear.gemv(xq, xs, q, ws, 1)
    assert np.array_equal(host(G.gemv(dev(xq), dc, de, dev(xs), dw, n, 1, fmt=F.MXFP4)), ref)
    res = bf16.to_bits(rng.standard_normal((batch, n)).astype(F32))
    assert np.array_equal(host(G.gemv(dev(xq), dc, de, dev(xs), dw, n, 2, res=dev(res), fmt=F.MXFP4)),
                          linear.gemv(xq, xs, q, ws, 2, res))
    xb, x = llm_acts(rng, batch, k)
    rq, rs = linear.act_quant(x)
    assert np.array_equal(host(G.gemv(dev(xb), dc, de, None, dw, n, 1, pro=1, fmt=F.MXFP4)), linear.gemv(rq, rs, q, ws, 1))


def test_gemv_expert_gather(F, G):
    """Decode of a mixture of experts on in-place MXFP4 expert weights: slot j multiplies row j with expert eidx[j]."""
    rng = np.random.default_rng(11)
    e, n, k, slots = 6, 128, 512, 4
    packs = [mxfp4_tensor(rng, n, k, base=rng.integers(-8, 2, n)) for _ in range(e)]
    nib, e8 = np.stack([p[0] for p in packs]), np.stack([p[1] for p in packs])
    dn, de = dev(nib), dev(e8)
    dw = F.mxfp4_row_scales(de.reshape(e * n, -1)).reshape(e, n)
    eidx = np.array([4, 0, 5, 0], np.int32)
    xq = rng.integers(-127, 128, (slots, k)).astype(np.int8)
    xs = (rng.random(slots) * 0.02 + 1e-3).astype(F32)
    y = host(G.gemv(dev(xq), F.mxfp4_codes(dn), de, dev(xs), dw, n, 1, eidx=dev(eidx), xstride=1, fmt=F.MXFP4))
    for j in range(slots):
        assert np.array_equal(y[j], linear.gemv(xq[j], xs[j], packs[eidx[j]][2], packs[eidx[j]][3], 1)), j


@pytest.mark.parametrize("m,n,k", [(2048, 2048, 2048), (512, 4096, 2048), (300, 260, 384), (64, 64, 128), (8192, 2048, 256),
                                   (1, 4, 128), (200, 1024, 1280), (131, 2048, 2048), (2048, 4096, 256)])
def test_dense_gemm(F, S, m, n, k):
    """Every tile configuration of the dense GEMM on the in-place form: INT32 accumulators and all epilogues."""
    rng = np.random.default_rng(m + n + k)
    nib, e8, q, ws = mxfp4_tensor(rng, n, k, base=rng.integers(-12, 4, n))
    dc, de, dw = on_device(F, nib, e8)
    wq = S.unpack_i8(dc, de, n, k, fmt=F.MXFP4, wscale=dw)
    xq = rng.integers(-127, 128, (m, k)).astype(np.int8)
    xs = (rng.random(m) * 0.02).astype(F32)
    acc = linear.int_gemm(xq, q)
    assert np.array_equal(host(S.mm_i8_i32(dev(xq), wq)), acc)
    assert np.array_equal(host(S.mm_epi(dev(xq), wq, dev(xs), dw, 1)), linear.epilogue(acc, xs, ws, 1))
    res = bf16.to_bits(rng.standard_normal((m, n)).astype(F32))
    assert np.array_equal(host(S.mm_epi(dev(xq), wq, dev(xs), dw, 2, res=dev(res))), linear.epilogue(acc, xs, ws, 2, res))
    if n % 8 == 0:
        with np.errstate(all="ignore"):
            assert np.array_equal(host(S.mm_epi(dev(xq), wq, dev(xs), dw, 3)), linear.epilogue(acc, xs, ws, 3))
    bits, x = llm_acts(rng, m, k)
    rq, rs = linear.act_quant(x)
    y = host(S.linear_w4a8(dev(bits), dc, de, dw, n, fmt=F.MXFP4))
    assert np.array_equal(y, linear.epilogue(linear.int_gemm(rq, q), rs, ws, 1))


def test_in_place_equals_converted_form_at_lm_head_width(F, G):
    """Config 2's wide layer at full size: the GEMV on the standard tensor and on its 2-bit conversion agree bit for
    bit (batch 1 and 4); a sample of rows against the oracle."""
    rng = np.random.default_rng(5)
    n, k = 151936, 2048
    g = torch.Generator(device="cuda").manual_seed(1)
    nib = torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, device="cuda", generator=g)
    e8 = (torch.randint(0, 4, (n, k // 32), dtype=torch.uint8, device="cuda", generator=g)
          + torch.randint(100, 125, (n, 1), dtype=torch.uint8, device="cuda", generator=g))
    e8[:, 0] = e8.min(dim=1).values                          # nothing else to keep: the span is at most 3 already
    dw = F.mxfp4_row_scales(e8)
    c2, b2, w2 = F.from_mxfp4(nib, e8)
    assert torch.equal(w2, dw)
    for batch in (1, 4):
        xb, x = llm_acts(rng, batch, k)
        dx = dev(xb) if batch > 1 else dev(xb)[0]
        ya = G.gemv(dx, F.mxfp4_codes(nib), e8, None, dw, n, 1, pro=1, fmt=F.MXFP4)
        yb = G.gemv(dx, c2, b2, None, w2, n, 1, pro=1)
        assert torch.equal(ya, yb), batch
        rows = rng.choice(n, 64, replace=False)
        cs, bs, wss = layout.from_mxfp4(host(nib[rows]), host(e8[rows]))
        qs = layout.decode(cs, bs, 64, k)
        rq, rs = linear.act_quant(x)
        want = linear.gemv(rq if batch > 1 else rq[0], rs if batch > 1 else rs[0], qs, wss, 1)
        assert np.array_equal(host(ya)[..., rows], want)


@pytest.mark.parametrize("tm", [64, 128, 256])
def test_grouped_gemm(F, tm):
    from mxfp4_int8_m5_amd import sc_moe as M
    rng = np.random.default_rng(tm)
    e, n, k, r = 5, 256, 512, 700
    ex = np.sort(rng.choice([0, 1, 2, 4], r, p=[0.5, 0.2, 0.2, 0.1])).astype(np.int32)          # expert 3 empty
    packs = [mxfp4_tensor(rng, n, k, base=rng.integers(-8, 2, n)) for _ in range(e)]
    nib, e8 = np.stack([p[0] for p in packs]), np.stack([p[1] for p in packs])
    wq, ws = np.stack([p[2] for p in packs]), np.stack([p[3] for p in packs])
    dn, de = dev(nib), dev(e8)
    dw = F.mxfp4_row_scales(de.reshape(e * n, -1)).reshape(e, n)
    xq = rng.integers(-127, 128, (r, k)).astype(np.int8)
    xs = (np.abs(rng.standard_normal(r)) * 1e-2).astype(F32)
    ref = moe.moe_int_gemm(xq, ex, wq)
    off, tstart, mt = M.segments(dev(ex), e, tm)
    dc = F.mxfp4_codes(dn)
    y1 = host(M.moe_mm(dev(xq), r, dc, de, dw, off, tstart, mt, n, 1, dev(xs), tile=(tm, 64, 4), fmt=F.MXFP4))
    assert np.array_equal(y1, moe.moe_epilogue(ref, xs, ws, ex, 1))
    with np.errstate(all="ignore"):
        y3 = host(M.moe_mm(dev(xq), r, dc, de, dw, off, tstart, mt, n, 3, dev(xs), tile=(tm, 64, 4), fmt=F.MXFP4))
        assert np.array_equal(y3, moe.moe_epilogue(ref, xs, ws, ex, 3))
