"""Row kernels of the model integrations on the GPU through the C ABI, bit-exact against the oracle's restatement
(whose parity with MLX's own rms_norm / swiglu is unpinned: MLX is not vendored in the reference), plus the
standard-MXFP4 import.  Mirrors e2e/test_sc_kernels.py:53-111,143-189."""
import numpy as np
import pytest
import torch

from oracle import bf16, layout, linear
from tests.util import blocked_layout, dev, host, llm_acts

pytestmark = pytest.mark.gpu
F32 = np.float32


@pytest.fixture(scope="module")
def S():
    from mxfp4_int8_m5_amd import sc_kernels
    return sc_kernels


@pytest.mark.parametrize("m,k", [(200, 2048), (3, 128), (65, 4096), (9, 1000), (70, 512), (33, 1536), (5, 3584), (2048, 2048),
                                 (130, 6144)])
def test_rmsnorm_quant(S, m, k):
    rng = np.random.default_rng(k + m)
    x = bf16.to_bits((rng.standard_normal((m, k)) * rng.lognormal(0, 1, (1, k))).astype(F32))
    nw = bf16.to_bits(rng.lognormal(0, 0.3, k).astype(F32))
    mp = S.pad_rows(m)
    rq, rs, rn = linear.rmsnorm_quant(x, nw, 1e-6, mp)
    xq, xs = S.rmsnorm_quant(dev(x), dev(nw), 1e-6)
    assert np.array_equal(host(xq), rq) and np.array_equal(host(xs), rs)
    xq, xs, xn = S.rmsnorm_quant_n(dev(x), dev(nw), torch.tensor([1e-6]))
    assert np.array_equal(host(xq), rq) and np.array_equal(host(xs), rs) and np.array_equal(host(xn), rn)
    assert not host(xq)[m:].any() and not host(xn)[m:].any()
    # against a float64 evaluation: within the 1e-2 bound
    xf, wf = bf16.from_bits(x).astype(np.float64), bf16.from_bits(nw).astype(np.float64)
    ref = wf * xf / np.sqrt((xf ** 2).mean(1, keepdims=True) + 1e-6)
    assert linear.rel_fro(bf16.from_bits(host(xn))[:m], ref) < 1e-2
    # the same codes block by block (the layout the large dense GEMM tiles read), where the shape allows it
    bq, bs, bn = S.rmsnorm_quant_n(dev(x), dev(nw), 1e-6, blocked=True)
    if k % 512 == 0 and k <= 4096:
        assert isinstance(bq, S.BlockedXq) and np.array_equal(host(bq.data), blocked_layout(rq))
        assert np.array_equal(host(bq.rows()), rq)
    else:
        assert np.array_equal(host(bq), rq)
    assert np.array_equal(host(bs), rs) and np.array_equal(host(bn), rn)


def test_res_norm_quant_and_res_epilogue(S):
    rng = np.random.default_rng(1)
    mp, k = 256, 2048
    acc = rng.integers(-2 ** 20, 2 ** 20, (mp, k)).astype(np.int32)
    xs = (np.abs(rng.standard_normal(mp)) * 1e-3).astype(F32)
    ws = (np.abs(rng.standard_normal(k)) * 1e-3).astype(F32)
    res = bf16.to_bits(rng.standard_normal((mp, k)).astype(F32))
    nw = bf16.to_bits(rng.lognormal(0, 0.3, k).astype(F32))
    h, xq, xs2 = S.res_norm_quant(dev(acc), dev(xs), dev(ws), dev(res), dev(nw), 1e-6)
    rh, rq, rs = linear.res_norm_quant(acc, xs, ws, res, nw, 1e-6)
    assert np.array_equal(host(h), rh) and np.array_equal(host(xq), rq) and np.array_equal(host(xs2), rs)
    assert np.array_equal(host(S.res_epilogue(dev(acc), dev(xs), dev(ws), dev(res))), rh)


def test_swiglu_quant(S):
    rng = np.random.default_rng(2)
    mp, f = 128, 6144
    acc = rng.integers(-2 ** 18, 2 ** 18, (mp, 2 * f)).astype(np.int32)
    xs = (np.abs(rng.standard_normal(mp)) * 1e-3).astype(F32)
    ws = (np.abs(rng.standard_normal(2 * f)) * 1e-2).astype(F32)
    xq, xs2 = S.swiglu_quant(dev(acc), dev(xs), dev(ws), torch.bfloat16)
    rq, rs = linear.swiglu_quant(acc, xs, ws)
    assert np.array_equal(host(xq), rq) and np.array_equal(host(xs2), rs)


def test_swiglu_exhaustive_gate_values(S):
    """All 65536 bf16 gate patterns through the GEMM's SwiGLU epilogue (e2e/test_sc_kernels.py:82-95): a K = 128 GEMM
    whose accumulators reproduce chosen bf16 values exactly (acc = value's integer significand, scale = power of 2)."""
    rng = np.random.default_rng(3)
    gb = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    gf = bf16.from_bits(gb)
    # an integer accumulator cannot produce -0.0; magnitudes outside 2^+-100 would leave FP32's normal range
    keep = np.isfinite(gf) & (np.abs(gf) < 2.0 ** 100) & ((np.abs(gf) > 2.0 ** -100) | (gb == 0))
    gb = gb[keep]
    ub = bf16.to_bits((rng.standard_normal(gb.size) * 3).astype(F32))
    # y = acc * xs * ws with acc in [-255, 255] (8-bit significand), xs = 1, ws = 2^e: exact
    def split(b):
        f = bf16.from_bits(b).astype(np.float64)
        m, e = np.frexp(f)
        return np.rint(m * 256).astype(np.int32), (e - 8).astype(np.int32)
    ga, ge = split(gb)
    ua, ue = split(ub)
    n_pairs = gb.size
    pad = (-n_pairs) % 4
    ga, ge, ua, ue = (np.concatenate([a, np.zeros(pad, a.dtype)]) for a in (ga, ge, ua, ue))
    half = ga.size
    # one token row; weight row n holds the integer in 2 columns (a = 127 * q1 + q2) against x = (127, 1, 0, ...)
    acc_rows = np.concatenate([ga, ua])
    k = 128
    wq = np.zeros((2 * half, k), np.int8)
    wq[:, 0] = np.sign(acc_rows) * (np.abs(acc_rows) // 127)
    wq[:, 1] = np.sign(acc_rows) * (np.abs(acc_rows) % 127)
    xq = np.zeros((4, k), np.int8)
    xq[:, 0], xq[:, 1] = 127, 1
    ws = np.ldexp(1.0, np.concatenate([ge, ue])).astype(F32)
    perm = linear.interleave_gate_up(half)
    y = host(S.mm_epi(dev(xq), dev(wq[perm]), dev(np.ones(4, F32)), dev(ws[perm]), 3, torch.bfloat16))[0]
    ref = linear.swiglu(np.concatenate([gb, np.zeros(pad, np.uint16)]), np.concatenate([ub, np.zeros(pad, np.uint16)]))
    assert np.array_equal(y[:n_pairs], ref[:n_pairs])


@pytest.mark.parametrize("from_acc", [True, False])
def test_qkv_headnorm(S, from_acc):
    rng = np.random.default_rng(4)
    hq, hk, d, L, mp = 16, 8, 128, 200, 256
    ntot = (hq + 2 * hk) * d
    qn = bf16.to_bits(rng.lognormal(0, 0.3, d).astype(F32))
    kn = bf16.to_bits(rng.lognormal(0, 0.3, d).astype(F32))
    if from_acc:
        acc = rng.integers(-2 ** 18, 2 ** 18, (mp, ntot)).astype(np.int32)
        xs = (np.abs(rng.standard_normal(mp)) * 1e-3).astype(F32)
        ws = (np.abs(rng.standard_normal(ntot)) * 1e-4).astype(F32)
        y = linear.scale_out(acc, xs, ws)
        q, k, v = S.qkv_epilogue_headnorm(dev(acc), dev(xs), dev(ws), dev(qn), dev(kn), 1e-6, L, hq, hk, d, torch.bfloat16)
    else:
        y = bf16.to_bits(rng.standard_normal((mp, ntot)).astype(F32))
        q, k, v = S.qkv_headnorm_y(dev(y), dev(qn), dev(kn), 1e-6, L, hq, hk, d)
    rq, rk, rv = linear.headnorm(y, qn, kn, 1e-6, L, hq, hk, d)
    assert np.array_equal(host(q), rq) and np.array_equal(host(k), rk) and np.array_equal(host(v), rv)


def test_qkv_fullnorm(S):
    rng = np.random.default_rng(5)
    h, d, L, mp = 16, 128, 200, 256
    y = bf16.to_bits(rng.standard_normal((mp, 3 * h * d)).astype(F32))
    qn = bf16.to_bits(rng.lognormal(0, 0.3, h * d).astype(F32))
    kn = bf16.to_bits(rng.lognormal(0, 0.3, h * d).astype(F32))
    q, k, v = S.qkv_fullnorm_y(dev(y), dev(qn), dev(kn), 1e-5, L, h, d)
    rq, rk, rv = linear.fullnorm(y, qn, kn, 1e-5, L, h, d)
    assert np.array_equal(host(q), rq) and np.array_equal(host(k), rk) and np.array_equal(host(v), rv)


def test_standard_mxfp4_import(S):
    """E2M1 nibbles + E8M0 scales in, the exact INT8 embedding out (north-star step 1 on a standard MXFP4 tensor)."""
    from mxfp4_int8_m5_amd import sc_format
    rng = np.random.default_rng(6)
    n, k = 192, 1024
    w = rng.standard_normal((n, k)) * 0.02
    w[:, 5] *= 8
    codes, bc, ws, q = layout.quantize(w)
    nib, e8 = layout.to_mxfp4(codes, bc, ws, n, k)
    c2, b2, w2 = sc_format.from_mxfp4(dev(nib), dev(e8))
    assert np.array_equal(host(b2), bc) and np.array_equal(host(w2), ws)
    assert np.array_equal(host(c2).view(np.uint32), codes)
    assert np.array_equal(host(S.unpack_i8(c2, b2, n, k, lazy=False)), q)
    e8[0, 0] = e8[0].min() + 7
    with pytest.raises(ValueError):
        sc_format.from_mxfp4(dev(nib), dev(e8))


@pytest.mark.parametrize("m,mp,k", [(5, 8, 128), (300, 384, 2048), (64, 64, 6144), (17, 17, 1536), (3, 3, 32)])
def test_rot_quant(m, mp, k):
    """Block Hadamard rotation + per-token INT8 (e2e/sc_kernels.py:231-275), bit-exact against the oracle's butterfly
    restatement: codes and scales, zero padding rows."""
    from mxfp4_int8_m5_amd import sc_kernels as S
    rng = np.random.default_rng(m + k)
    bits, x = llm_acts(rng, m, k)
    signs = S.rot_signs(k)
    assert np.array_equal(host(signs), linear.rot_signs(k))
    xq, xs = S.rot_quant(dev(bits), signs, mp)
    wq, ws = linear.rot_quant(x, linear.rot_signs(k), mp)
    assert np.array_equal(host(xq), wq) and np.array_equal(host(xs), ws)
