"""Decode GEMV parity on the GPU through the C ABI: equal to the INT32 GEMM row plus the prefill epilogue, bit for
bit, for every prologue / epilogue / batch / expert-gather form.  Mirrors e2e/sc_decode.py:241-309."""
import numpy as np
import pytest
import torch

from oracle import bf16, layout, linear
from tests.util import FORMATS, dev, host, llm_acts, product_format, random_packed

pytestmark = pytest.mark.gpu
F32 = np.float32


@pytest.fixture(scope="module")
def G():
    from mxfp4_int8_m5_amd import sc_decode
    return sc_decode


@pytest.fixture(scope="module")
def S():
    from mxfp4_int8_m5_amd import sc_kernels
    return sc_kernels


@pytest.mark.parametrize("n,k", [(256, 2048), (512, 6144), (64, 1024), (4096, 2048), (20, 128)])
def test_gemv_epilogues(G, S, n, k):
    rng = np.random.default_rng(n + k)
    w = rng.standard_normal((n, k)) * 0.02 * rng.lognormal(0, 0.5, (1, k))
    codes, bc, ws, qw = layout.quantize(w)
    xq = rng.integers(-127, 128, k).astype(np.int8)
    xq[:16] = 127
    xs = np.array([0.01], F32)
    dc, db, dw = dev(codes), dev(bc), dev(ws)
    y1 = host(G.gemv(dev(xq), dc, db, dev(xs), dw, n, 1))
    ref1 = linear.gemv(xq, xs[0], qw, ws, 1)
    assert np.array_equal(y1, ref1)
    # the prefill GEMM on the same row gives the same bits
    yg = host(S.mm_epi(dev(np.tile(xq, (4, 1))), S.unpack_i8(dc, db, n, k), dev(np.repeat(xs, 4)), dw, 1))
    assert np.array_equal(yg[0], y1)
    res = bf16.to_bits(rng.standard_normal(n).astype(F32))
    y2 = host(G.gemv(dev(xq), dc, db, dev(xs), dw, n, 2, res=dev(res)))
    assert np.array_equal(y2, linear.gemv(xq, xs[0], qw, ws, 2, res))
    perm = linear.interleave_gate_up(n // 2)
    cp = codes.reshape(n, -1)[perm].reshape(-1)
    y3 = host(G.gemv(dev(xq), dev(cp), dev(bc[perm]), dev(xs), dev(ws[perm]), n, 3))
    assert np.array_equal(y3, linear.swiglu(ref1[:n // 2], ref1[n // 2:]))


@pytest.mark.parametrize("i", range(len(FORMATS)))
def test_gemv_formats(G, i):
    fmt = FORMATS[i]
    rng = np.random.default_rng(60 + i)
    n, k = 256, 2048
    codes, bc, ws, q = random_packed(rng, n, k, fmt)
    xq = rng.integers(-127, 128, k).astype(np.int8)
    xs = np.array([1e-2], F32)
    y = host(G.gemv(dev(xq), dev(codes), dev(bc), dev(xs), dev(ws), n, 1, fmt=product_format(fmt)))
    assert np.array_equal(y, linear.gemv(xq, xs[0], q, ws, 1))


@pytest.mark.parametrize("n,k", [(512, 6144), (64, 1024), (20, 128), (1024, 2048)])
def test_gemv_block16_power_of_two_format(G, n, k):
    """The 16-element-block variant of the published format (its own conversion path in the kernel): saturated
    activations, every epilogue, rows that take several passes over K, and a fused act_quant prologue."""
    fmt = layout.Format(block=16)
    pf = product_format(fmt)
    rng = np.random.default_rng(n + k + 16)
    codes, bc, ws, q = random_packed(rng, n, k, fmt)
    xq = rng.integers(-127, 128, k).astype(np.int8)
    xq[:16] = 127
    xs = np.array([0.01], F32)
    dc, db, dw = dev(codes), dev(bc), dev(ws)
    ref1 = linear.gemv(xq, xs[0], q, ws, 1)
    assert np.array_equal(host(G.gemv(dev(xq), dc, db, dev(xs), dw, n, 1, fmt=pf)), ref1)
    res = bf16.to_bits(rng.standard_normal(n).astype(F32))
    y2 = host(G.gemv(dev(xq), dc, db, dev(xs), dw, n, 2, res=dev(res), fmt=pf))
    assert np.array_equal(y2, linear.gemv(xq, xs[0], q, ws, 2, res))
    perm = linear.interleave_gate_up(n // 2)
    cp = codes.reshape(n, -1)[perm].reshape(-1)
    y3 = host(G.gemv(dev(xq), dev(cp), dev(bc[perm]), dev(xs), dev(ws[perm]), n, 3, fmt=pf))
    assert np.array_equal(y3, linear.swiglu(ref1[:n // 2], ref1[n // 2:]))
    xb, x = llm_acts(rng, 1, k)
    rq, rs = linear.act_quant(x)
    yp = host(G.gemv(dev(xb), dc, db, None, dw, n, 1, pro=1, fmt=pf))
    assert np.array_equal(yp, linear.gemv(rq[0], rs[0], q, ws, 1))


@pytest.mark.parametrize("pro", [1, 2])
def test_gemv_fused_prologues(G, S, pro):
    """PRO 1 / 2 inside the GEMV equal the separate act_quant / rmsnorm_quant kernels (e2e/sc_decode.py:278-291)."""
    rng = np.random.default_rng(pro)
    n, k = 512, 2048
    codes, bc, ws, q = random_packed(rng, n, k)
    x = bf16.to_bits((rng.standard_normal((1, k)) * rng.lognormal(0, 1, k)).astype(F32))
    nw = bf16.to_bits(rng.lognormal(0, 0.3, k).astype(F32))
    dc, db, dw = dev(codes), dev(bc), dev(ws)
    if pro == 1:
        xq, xs = S.act_quant(dev(x), 1)
        rq, rs = linear.act_quant(bf16.from_bits(x))
    else:
        xq, xs = S.rmsnorm_quant(dev(x), dev(nw), 1e-6, 1)
        rq, rs, _ = linear.rmsnorm_quant(x, nw, 1e-6)
    assert np.array_equal(host(xq), rq) and np.array_equal(host(xs), rs)
    y0 = host(G.gemv(xq[0], dc, db, xs, dw, n, 1))
    y1 = host(G.gemv(dev(x)[0], dc, db, None, dw, n, 1, pro=pro, nw=dev(nw), eps=1e-6))
    assert np.array_equal(y0, y1)
    assert np.array_equal(y0, linear.gemv(rq[0], rs[0], q, ws, 1))


@pytest.mark.parametrize("batch", [2, 3, 4, 5, 7, 8, 9, 19])
def test_gemv_batch_equals_rows(G, batch):
    """B rows against one pass over the weights give the bits of B independent batch-1 GEMVs (3, 5, 6 and 7 rows run
    padded to 4 / 8 by the Python surface, more than 8 rows eight at a time)."""
    rng = np.random.default_rng(batch)
    n, k = 1024, 2048
    codes, bc, ws, q = random_packed(rng, n, k)
    xq = rng.integers(-127, 128, (batch, k)).astype(np.int8)
    xs = (np.abs(rng.standard_normal(batch)) * 1e-2).astype(F32)
    dc, db, dw = dev(codes), dev(bc), dev(ws)
    yb = host(G.gemv(dev(xq), dc, db, dev(xs), dw, n, 1))
    assert yb.shape == (batch, n)
    for b in range(batch):
        y1 = host(G.gemv(dev(xq[b]), dc, db, dev(xs[b:b + 1]), dw, n, 1))
        assert np.array_equal(yb[b], y1)
    assert np.array_equal(yb, linear.gemv(xq, xs, q, ws, 1))
    xb = bf16.to_bits(rng.standard_normal((batch, k)).astype(F32))
    yp = host(G.gemv(dev(xb), dc, db, None, dw, n, 1, pro=1))
    rq, rs = linear.act_quant(bf16.from_bits(xb))
    assert np.array_equal(yp, linear.gemv(rq, rs, q, ws, 1))


@pytest.mark.parametrize("batch,n,k", [(2, 512, 512), (4, 2048, 6144), (8, 256, 1536), (4, 1028, 1024), (4, 1022, 1024),
                                       (4, 512, 640)])
def test_gemv_batch_shapes_and_epilogues(G, batch, n, k):
    """Several rows per pass over K of one, several and fractional 2048-slices, N off the 4-row grain, K off the
    512 grain, with the residual and SwiGLU epilogues."""
    rng = np.random.default_rng(batch + n + k)
    codes, bc, ws, q = random_packed(rng, n, k)
    xq = rng.integers(-127, 128, (batch, k)).astype(np.int8)
    xq[0, :16] = 127
    xs = (np.abs(rng.standard_normal(batch)) * 1e-2 + 1e-3).astype(F32)
    dc, db, dw = dev(codes), dev(bc), dev(ws)
    ref1 = linear.gemv(xq, xs, q, ws, 1)
    assert np.array_equal(host(G.gemv(dev(xq), dc, db, dev(xs), dw, n, 1)), ref1)
    res = bf16.to_bits(rng.standard_normal((batch, n)).astype(F32))
    assert np.array_equal(host(G.gemv(dev(xq), dc, db, dev(xs), dw, n, 2, res=dev(res))), linear.gemv(xq, xs, q, ws, 2, res))
    if n % 4 == 0:
        perm = linear.interleave_gate_up(n // 2)
        cp = codes.reshape(n, -1)[perm].reshape(-1)
        y3 = host(G.gemv(dev(xq), dev(cp), dev(bc[perm]), dev(xs), dev(ws[perm]), n, 3))
        assert np.array_equal(y3, linear.swiglu(ref1[:, :n // 2], ref1[:, n // 2:]))


def test_gemv_expert_gather(G):
    """MoE: slot j uses expert eidx[j] and its own input row; `shared` appends one more slot
    (e2e/sc_decode.py:292-307, e2e/decode.py:126-143)."""
    rng = np.random.default_rng(5)
    e, n, k = 5, 256, 1024
    packs = [random_packed(rng, n, k) for _ in range(e)]
    codes = np.stack([p[0] for p in packs])
    bc = np.stack([p[1] for p in packs])
    ws = np.stack([p[2] for p in packs])
    dc, db, dw = dev(codes), dev(bc), dev(ws)
    xq = rng.integers(-127, 128, (3, k)).astype(np.int8)
    xs = np.array([0.01, 0.02, 0.03], F32)
    eidx = np.array([2, 0], np.int32)
    y = host(G.gemv(dev(xq[:2]), dc, db, dev(xs[:2]), dw, n, 1, eidx=dev(eidx), xstride=1))
    for j, ex in enumerate(eidx):
        assert np.array_equal(y[j], linear.gemv(xq[j], xs[j], packs[ex][3], ws[ex], 1))
    # one shared input row, routed experts + shared expert 4, SwiGLU epilogue
    y = host(G.gemv(dev(xq[0]), dc, db, dev(xs[:1]), dw, n, 3, eidx=dev(eidx), xstride=0, shared=4))
    assert y.shape == (3, n // 2)
    for j, ex in enumerate([2, 0, 4]):
        assert np.array_equal(y[j], linear.gemv(xq[0], xs[0], packs[ex][3], ws[ex], 3))
    # per-slot bf16 inputs quantized in the kernel (the down projection of e2e/decode.py:137)
    xb = bf16.to_bits(rng.standard_normal((3, k)).astype(F32))
    y = host(G.gemv(dev(xb), dc, db, None, dw, n, 1, eidx=dev(eidx), xstride=1, pro=1, shared=4))
    rq, rs = linear.act_quant(bf16.from_bits(xb))
    for j, ex in enumerate([2, 0, 4]):
        assert np.array_equal(y[j], linear.gemv(rq[j], rs[j], packs[ex][3], ws[ex], 1))


def test_config2_lm_head_full_size(G, S):
    """BASELINE config 2's widest layer, 151936 x 2048, batch 1 and 4: every output against the oracle."""
    rng = np.random.default_rng(2)
    n, k = 151936, 2048
    codes, bc, ws, q = random_packed(rng, n, k)
    xb = bf16.to_bits(rng.standard_normal((4, k)).astype(F32))
    rq, rs = linear.act_quant(bf16.from_bits(xb))
    dc, db, dw = dev(codes), dev(bc), dev(ws)
    ref = linear.gemv(rq, rs, q, ws, 1)
    y4 = host(G.gemv(dev(xb), dc, db, None, dw, n, 1, pro=1))
    assert np.array_equal(y4, ref)
    y1 = host(G.gemv(dev(xb)[0], dc, db, None, dw, n, 1, pro=1))
    assert np.array_equal(y1, ref[0])


@pytest.mark.parametrize("name,n,k", [("qkv", 4096, 2048), ("o_proj", 2048, 2048), ("gate_up", 12288, 2048),
                                      ("down", 2048, 6144)])
def test_config2_dense_shapes_full_size(G, name, n, k):
    """BASELINE config 2 on the four dense layer shapes exactly as benchmarked: weights N(0, 0.02) quantized by the
    oracle, a bf16 N(0, 1) token quantized in the kernel, batch 1 and batch 4; every output against the oracle."""
    rng = np.random.default_rng(200 + n + k)
    codes, bc, ws, q = layout.quantize(rng.standard_normal((n, k)) * 0.02)
    xb = bf16.to_bits(rng.standard_normal((4, k)).astype(F32))
    rq, rs = linear.act_quant(bf16.from_bits(xb))
    dc, db, dw = dev(codes), dev(bc), dev(ws)
    ref = linear.gemv(rq, rs, q, ws, 1)
    assert np.array_equal(host(G.gemv(dev(xb), dc, db, None, dw, n, 1, pro=1)), ref)
    assert np.array_equal(host(G.gemv(dev(xb)[0], dc, db, None, dw, n, 1, pro=1)), ref[0])
    assert linear.rel_fro(bf16.from_bits(ref[0]), linear.float_reference(bf16.from_bits(xb[:1]), q, ws)[0]) < 1e-2


@pytest.mark.parametrize("batch,n,k,pro", [(1, 32768, 512, 0), (1, 40000, 2048, 1), (2, 32784, 1536, 2), (4, 33008, 6144, 1),
                                           (8, 32768, 1024, 0), (4, 65536, 2048, 2)])
def test_gemv_wide_layers_every_batch(G, S, batch, n, k, pro):
    """Layers of 32768 rows and more in the published format run the half-precision-MFMA kernel (16 rows per wave, K in
    pieces of 512): every output of batch 1 / 2 / 4 / 8 against the oracle with saturated activations, all three
    prologues, the residual and SwiGLU epilogues, and equal to the narrow-layer kernels on a slice of the same rows."""
    rng = np.random.default_rng(batch + n + k)
    codes, bc, ws, q = random_packed(rng, n, k)
    dc, db, dw = dev(codes), dev(bc), dev(ws)
    nw = bf16.to_bits(rng.lognormal(0, 0.3, k).astype(F32))
    if pro == 0:
        xq = rng.integers(-127, 128, (batch, k)).astype(np.int8)
        xq[0, :64] = 127
        xq[-1, -64:] = -127
        xs = (np.abs(rng.standard_normal(batch)) * 1e-2 + 1e-3).astype(F32)
        xin, xsc, kw = dev(xq), dev(xs), {}
    else:
        xb = bf16.to_bits((rng.standard_normal((batch, k)) * rng.lognormal(0, 1, k)).astype(F32))
        if pro == 1:
            xq, xs = linear.act_quant(bf16.from_bits(xb))
            kw = dict(pro=1)
        else:
            xq, xs, _ = linear.rmsnorm_quant(xb, nw, 1e-6, batch)
            kw = dict(pro=2, nw=dev(nw), eps=1e-6)
        xin, xsc = dev(xb), None
    if batch == 1:
        xin = xin[0]
    ref1 = linear.gemv(xq, xs, q, ws, 1)
    y1 = host(G.gemv(xin, dc, db, xsc, dw, n, 1, **kw)).reshape(batch, n)
    assert np.array_equal(y1, ref1)
    res = bf16.to_bits(rng.standard_normal((batch, n)).astype(F32))
    y2 = host(G.gemv(xin, dc, db, xsc, dw, n, 2, res=dev(res if batch > 1 else res[0]), **kw)).reshape(batch, n)
    assert np.array_equal(y2, linear.gemv(xq, xs, q, ws, 2, res))
    perm = linear.interleave_gate_up(n // 2)
    cp = codes.reshape(n, -1)[perm].reshape(-1)
    y3 = host(G.gemv(xin, dev(cp), dev(bc[perm]), xsc, dev(ws[perm]), n, 3, **kw)).reshape(batch, n // 2)
    assert np.array_equal(y3, linear.swiglu(ref1[:, :n // 2], ref1[:, n // 2:]))
    # the first 4096 rows as a narrow layer (the per-row kernels) give the same bits
    m = 4096
    ys = host(G.gemv(xin, dev(codes[:m * k // 8]), dev(bc[:m]), xsc, dev(ws[:m]), m, 1, **kw)).reshape(batch, m)
    assert np.array_equal(ys, y1[:, :m])


@pytest.mark.parametrize("batch,n,k,pro", [(4, 4096, 2048, 0), (2, 2048, 2048, 2), (4, 2048, 6144, 2), (8, 1024, 512, 1),
                                           (4, 12288, 2048, 1), (2, 48, 1024, 0)])
def test_gemv_narrow_layers_split_over_k(G, batch, n, k, pro):
    """Narrow layers with several activation rows (one 16-row group per workgroup, K split over its waves, partial totals
    through LDS): INT8 input, in-kernel quantization and the RMSNorm prologue, K of one to twelve pieces, every epilogue."""
    rng = np.random.default_rng(7 * batch + n + k)
    codes, bc, ws, q = random_packed(rng, n, k)
    dc, db, dw = dev(codes), dev(bc), dev(ws)
    nw = bf16.to_bits(rng.lognormal(0, 0.3, k).astype(F32))
    if pro == 0:
        xq = rng.integers(-127, 128, (batch, k)).astype(np.int8)
        xq[0] = 127
        xs = (np.abs(rng.standard_normal(batch)) * 1e-2 + 1e-3).astype(F32)
        xin, xsc, kw = dev(xq), dev(xs), {}
    else:
        xb = bf16.to_bits((rng.standard_normal((batch, k)) * rng.lognormal(0, 1, k)).astype(F32))
        xb[-1] = 0                                   # a zero row: scale 0, outputs 0
        if pro == 1:
            xq, xs = linear.act_quant(bf16.from_bits(xb))
            kw = dict(pro=1)
        else:
            xq, xs, _ = linear.rmsnorm_quant(xb, nw, 1e-6, batch)
            kw = dict(pro=2, nw=dev(nw), eps=1e-6)
        xin, xsc = dev(xb), None
    ref1 = linear.gemv(xq, xs, q, ws, 1)
    assert np.array_equal(host(G.gemv(xin, dc, db, xsc, dw, n, 1, **kw)), ref1)
    res = bf16.to_bits(rng.standard_normal((batch, n)).astype(F32))
    assert np.array_equal(host(G.gemv(xin, dc, db, xsc, dw, n, 2, res=dev(res), **kw)), linear.gemv(xq, xs, q, ws, 2, res))
    perm = linear.interleave_gate_up(n // 2)
    cp = codes.reshape(n, -1)[perm].reshape(-1)
    y3 = host(G.gemv(xin, dev(cp), dev(bc[perm]), xsc, dev(ws[perm]), n, 3, **kw))
    assert np.array_equal(y3, linear.swiglu(ref1[:, :n // 2], ref1[:, n // 2:]))
    for b in range(batch):                           # and every row equals its own batch-1 call
        one = host(G.gemv(xin[b], dc, db, None if xsc is None else xsc[b:b + 1], dw, n, 1, **kw))
        assert np.array_equal(one, ref1[b])


@pytest.mark.parametrize("n,k", [(36864, 2048), (2048, 2048), (512, 6144)])
def test_gemv_block_codes_at_an_odd_address(G, n, k):
    """Block codes that start at an odd byte address (a view into a larger buffer): the wide and the narrow batch
    kernels read them with 4- and 16-byte loads and are only chosen for aligned codes; every batch gives the bits of
    the aligned call."""
    rng = np.random.default_rng(n + k + 1)
    codes, bc, ws, q = random_packed(rng, n, k)
    dc, dw = dev(codes), dev(ws)
    aligned = dev(bc)
    buf = torch.zeros(bc.size + 64, dtype=torch.uint8, device="cuda")
    odd = buf[33:33 + bc.size].view(bc.shape)
    odd.copy_(aligned)
    assert odd.data_ptr() % 2 == 1
    for batch in (1, 2, 4, 8):
        xb, _ = llm_acts(rng, batch, k)
        dx = dev(xb) if batch > 1 else dev(xb)[0]
        ya = G.gemv(dx, dc, aligned, None, dw, n, 1, pro=1)
        yo = G.gemv(dx, dc, odd, None, dw, n, 1, pro=1)
        assert torch.equal(ya, yo), batch
