"""W4A8 linear-layer arithmetic after the weights are packed (numpy; test infrastructure): per-token INT8
activation quantization, the exact INT32 contraction, the scaling epilogues, and the batch-1 GEMV."""
import numpy as np

from . import bf16

F32 = np.float32


def pad_rows(m, tile=128):
    """Rows padded up to the GEMM tile (e2e/sc_kernels.py:476-477)."""
    return -(-m // tile) * tile


def act_quant(x, mp=None):
    """Per-token symmetric INT8 in FP32: s = amax/127, qi = s > 0 ? 1/s : 0, q = clamp(rint(x * qi), +-127);
    rows >= M are zero with scale 0.  x is FP32 holding bf16-representable values.
    The kernel formula of e2e/sc_kernels.py:200-229, whose numpy twin is e2e/test_sc_kernels.py:21-26."""
    x = np.asarray(x, F32)
    m, k = x.shape
    mp = m if mp is None else mp
    s = (np.abs(x).max(1) / F32(127)).astype(F32)
    with np.errstate(divide="ignore"):
        qi = np.where(s > 0, F32(1) / np.where(s > 0, s, F32(1)), F32(0)).astype(F32)
    q = np.clip(np.rint(x * qi[:, None]), -127, 127).astype(np.int8)
    xq = np.zeros((mp, k), np.int8)
    xs = np.zeros(mp, F32)
    xq[:m], xs[:m] = q, s
    return xq, xs


ROT_NORM = F32(0.17677669529663687)   # 1 / sqrt(32), e2e/sc_kernels.py:578


def rot_signs(k):
    """The sign vector of the rotation for input width k (e2e/sc_kernels.py:566-569)."""
    return np.random.default_rng(0).choice([-1.0, 1.0], size=k).astype(F32)


def rot_blocks(x, signs):
    """Randomized Hadamard rotation of every 32-wide block in FP32 with the butterfly order of the kernel
    (e2e/sc_kernels.py:231-256): signs, then inside each group of 4 values the stages (x+y, x-y, z+w, z-w) and
    (x+z, y+w, x-z, y-w), then across the 8 groups of a block the strides 1, 2, 4 with lower = lower + upper and
    upper = lower - upper; the result times 1/sqrt(32) is rounded to bf16.  x: FP32 [M, K] holding bf16 values."""
    x = np.asarray(x, F32) * np.asarray(signs, F32)[None, :]
    m, k = x.shape
    a = x.reshape(m, k // 32, 8, 4)
    a = np.stack([a[..., 0] + a[..., 1], a[..., 0] - a[..., 1], a[..., 2] + a[..., 3], a[..., 2] - a[..., 3]], -1)
    a = np.stack([a[..., 0] + a[..., 2], a[..., 1] + a[..., 3], a[..., 0] - a[..., 2], a[..., 1] - a[..., 3]], -1)
    t = np.arange(8)
    for h in (1, 2, 4):
        c = a[:, :, t ^ h, :]
        upper = ((t & h) != 0)[None, None, :, None]
        a = np.where(upper, c - a, a + c).astype(F32)
    return bf16.rnd((a * ROT_NORM).astype(F32)).reshape(m, k)


def rot_quant(x, signs, mp=None):
    """rot_blocks followed by the per-token INT8 of act_quant (e2e/sc_kernels.py:257-273)."""
    return act_quant(rot_blocks(x, signs), mp)


def act_quant_f64(x):
    """The float64 variant of sim/make_testcase.py:56-58 (xq = clip(rint(x / xscale))); differs from act_quant
    only at rare rounding ties.  Returned for the float reference path."""
    xf = np.asarray(x, np.float64)
    xscale = np.abs(xf).max(1) / 127
    xq = np.clip(np.rint(xf / xscale[:, None]), -127, 127).astype(np.int8)
    return xq, xscale


def int_gemm(xq, wq):
    """INT8 [M,K] x INT8 [N,K]^T -> INT32 [M,N], exact: float64 BLAS on integers below 2^53
    (sim/make_testcase.py:59, e2e/test_sc_kernels.py:47-51)."""
    acc = np.asarray(xq, np.float64) @ np.asarray(wq, np.float64).T
    return acc.astype(np.int64).astype(np.int32)


def scale_out(acc, xs, ws):
    """bf16 bits of (float(acc) * xs[m]) * ws[n], FP32 left to right (e2e/sc_kernels.py:101,
    e2e/test_sc_kernels.py:134)."""
    y = (np.asarray(acc).astype(F32) * np.asarray(xs, F32)[:, None]) * np.asarray(ws, F32)[None, :]
    return bf16.to_bits(y)


def exp_f32(a):
    """exp(a) for a >= 0 in FP32 from IEEE add / multiply / rint only, so that the same operation sequence in any
    IEEE FP32 implementation gives the same bits: n = rint(a log2 e), r = a - n ln2 (two-part), degree-7 Taylor
    polynomial by Horner, scaled by 2^n in two exact steps.  Inputs above 89 (and NaN) are taken as 89 (-> inf).
    Stands in for metal::precise::exp of e2e/sc_kernels.py:322 (parity with MLX unpinned)."""
    a = np.asarray(a, F32)
    a = np.where(a < F32(89.0), a, F32(89.0)).astype(F32)
    n = np.rint(a * F32(1.4426950408889634))
    r = (a - n * F32(0.693145751953125)) - n * F32(1.428606765330187e-06)
    p = F32(1.0 / 5040.0)
    for c in (1.0 / 720.0, 1.0 / 120.0, 1.0 / 24.0, 1.0 / 6.0, 0.5, 1.0, 1.0):
        p = p * r + F32(c)
    ni = n.astype(np.int32)
    h = ni >> 1
    with np.errstate(over="ignore"):
        return (p * np.ldexp(F32(1), h).astype(F32)) * np.ldexp(F32(1), ni - h).astype(F32)


def swiglu(g_bits, u_bits):
    """silu(g) * u on bf16 bit patterns with every operation rounded to bf16: e = bf16(exp|g|), y = 1/(1+e),
    sig = g < 0 ? y : 1 - y, silu = g sig, out = silu u.  e2e/sc_kernels.py:317-328."""
    g, u = bf16.from_bits(g_bits), bf16.from_bits(u_bits)
    with np.errstate(over="ignore", invalid="ignore"):
        e = bf16.rnd(exp_f32(np.abs(g)))
        y = bf16.rnd(F32(1) / bf16.rnd(F32(1) + e))
        sig = np.where(g < 0, y, bf16.rnd(F32(1) - y))
        silu = bf16.rnd(g * sig)
        return bf16.to_bits(silu * u)


def interleave_gate_up(f):
    """Row order g_2p, g_2p+1, u_2p, u_2p+1 of [gate; up] for the SwiGLU epilogue (e2e/sc_kernels.py:520-524)."""
    p = np.arange(f // 2)
    return np.stack([2 * p, 2 * p + 1, f + 2 * p, f + 2 * p + 1], 1).reshape(-1)


def epilogue(acc, xs, ws, epi, res_bits=None):
    """The GEMM epilogues on INT32 accumulators (e2e/sc_kernels.py:73-115):
    0: INT32 as is; 1: bf16(acc xs ws); 2: bf16(res + bf16(acc xs ws)); 3: SwiGLU of rows interleaved in groups of
    four columns (g, g, u, u) -> [M, N/2].  Returns uint16 bf16 bits (INT32 for epi 0)."""
    if epi == 0:
        return np.asarray(acc, np.int32)
    y = scale_out(acc, xs, ws)
    if epi == 1:
        return y
    if epi == 2:
        return bf16.to_bits(bf16.from_bits(res_bits) + bf16.from_bits(y))
    m, n = y.shape
    y4 = y.reshape(m, n // 4, 4)
    return swiglu(y4[:, :, 0:2], y4[:, :, 2:4]).reshape(m, n // 2)


def float_reference(x, wq, wscale):
    """The float path the 1e-2 relative-error bound is taken against: float64 activation quantization, exact
    accumulation, y = f32(acc * f32(xscale) * wscale).  sim/make_testcase.py:56-60."""
    xq, xscale = act_quant_f64(x)
    acc = xq.astype(np.float64) @ np.asarray(wq, np.float64).T
    return (acc * xscale[:, None].astype(F32) * np.asarray(wscale, F32)[None, :]).astype(F32)


def rel_fro(y, ref):
    y, ref = np.asarray(y, np.float64), np.asarray(ref, np.float64)
    return float(np.linalg.norm(y - ref) / max(np.linalg.norm(ref), 1e-300))


def gemv(xq, xs, wq, ws, epi, res_bits=None):
    """Batch-1 (or batch-B, row by row) decode: the GEMM row with the same epilogue (e2e/sc_decode.py:3,255-267).
    xq int8 [K] or [B, K], xs scalar or [B]."""
    xq2 = np.atleast_2d(xq)
    out = epilogue(int_gemm(xq2, wq), np.atleast_1d(np.asarray(xs, F32)), ws, epi,
                   None if res_bits is None else np.atleast_2d(res_bits))
    return out if np.ndim(xq) == 2 else out[0]


# ---- RMSNorm + quantization family (arithmetic order of this build's wave-64 kernels) ----------------------------

def _wave_sum(v):
    """Butterfly sum over the last axis (64 lanes): v += v[lane ^ off] for off = 32, 16, ..., 1.  Every lane ends
    with the same FP32 value; this fixes the reduction order the kernels use."""
    v = np.asarray(v, F32)
    lanes = np.arange(64)
    for off in (32, 16, 8, 4, 2, 1):
        v = v + v[..., lanes ^ off]
    return v[..., 0]


def row_sumsq(x):
    """Sum of squares of FP32 rows [M, K], K a multiple of 4: each of K/4 virtual threads sums its four squares in
    order; threads are summed 64 at a time by `_wave_sum` (missing lanes contribute 0), and the per-wave partials
    (at most 64 of them) by a second `_wave_sum`.  Mirrors the thread layout described at
    e2e/sc_kernels.py:120-122 with 64-lane waves."""
    x = np.asarray(x, F32)
    m, k = x.shape
    t = x.reshape(m, k // 4, 4)
    ss = np.zeros((m, k // 4), F32)
    for i in range(4):
        ss = ss + t[:, :, i] * t[:, :, i]
    nw = -(-(k // 4) // 64)
    pad = np.zeros((m, nw * 64), F32)
    pad[:, :k // 4] = ss
    part = _wave_sum(pad.reshape(m, nw, 64))
    pad2 = np.zeros((m, 64), F32)
    pad2[:, :nw] = part
    return _wave_sum(pad2)


def rmsnorm(x_bits, w_bits, eps):
    """bf16 RMSNorm rows: inv = 1/sqrt(ss/K + eps) in FP32, y = bf16(w * bf16(x * inv)).
    e2e/sc_kernels.py:134-141 (rsqrt taken as IEEE 1/sqrt)."""
    x = bf16.from_bits(x_bits)
    k = x.shape[1]
    inv = F32(1) / np.sqrt(row_sumsq(x) / F32(k) + F32(eps))
    return bf16.to_bits(bf16.from_bits(w_bits)[None, :] * bf16.rnd(x * inv[:, None]))


def rmsnorm_quant(x_bits, w_bits, eps, mp=None):
    """(xq int8 [Mp,K], xs f32 [Mp], xn bf16 bits [Mp,K]) of RMSNorm then per-token INT8.
    e2e/sc_kernels.py:123-174, 383-386."""
    xn = rmsnorm(x_bits, w_bits, eps)
    xq, xs = act_quant(bf16.from_bits(xn), mp)
    out = np.zeros((xq.shape[0], xn.shape[1]), np.uint16)
    out[:xn.shape[0]] = xn
    return xq, xs, out


def swiglu_quant(acc, xs, ws):
    """acc INT32 [Mp, 2F] (gate | up, not interleaved) -> per-token INT8 of swiglu(bf16 gate, bf16 up).
    e2e/sc_kernels.py:279-315."""
    y = scale_out(acc, xs, ws)
    f = y.shape[1] // 2
    a = swiglu(y[:, :f], y[:, f:])
    return act_quant(bf16.from_bits(a))


def res_epilogue(acc, xs, ws, res_bits):
    """h = bf16(res + bf16(acc xs ws)).  e2e/sc_kernels.py:191-197."""
    return epilogue(acc, xs, ws, 2, res_bits)


def res_norm_quant(acc, xs, ws, res_bits, w_bits, eps):
    """(h, xq, xs') : residual epilogue then RMSNorm + INT8 of h.  e2e/sc_kernels.py:177-189."""
    h = res_epilogue(acc, xs, ws, res_bits)
    xq, xs2, _ = rmsnorm_quant(h, w_bits, eps)
    return h, xq, xs2


def headnorm(y_bits, qn_bits, kn_bits, eps, length, hq, hk, d):
    """Qwen3 q/k/v split of bf16 y [Mp, (hq+2hk) d]: per-head RMSNorm of q and k heads (one wave per head, D/64
    values per lane summed in order then `_wave_sum`), outputs head-major [heads, L, d].
    e2e/sc_kernels.py:359-380 re-laid for 64 lanes."""
    y = bf16.from_bits(y_bits)[:length].reshape(length, hq + 2 * hk, d)
    per = d // 64
    t = y.reshape(length, hq + 2 * hk, 64, per)
    ss = np.zeros(t.shape[:3], F32)
    for i in range(per):
        ss = ss + t[..., i] * t[..., i]
    inv = F32(1) / np.sqrt(_wave_sum(ss) / F32(d) + F32(eps))
    yn = bf16.rnd(y * inv[..., None])
    q = bf16.to_bits(bf16.from_bits(qn_bits) * yn[:, :hq])
    k = bf16.to_bits(bf16.from_bits(kn_bits) * yn[:, hq:hq + hk])
    v = bf16.to_bits(y[:, hq + hk:])
    return q.transpose(1, 0, 2).copy(), k.transpose(1, 0, 2).copy(), v.transpose(1, 0, 2).copy()


def fullnorm(y_bits, qn_bits, kn_bits, eps, length, h, d):
    """OLMoE q/k/v split of bf16 y [Mp, 3 h d]: RMSNorm over the full h*d width of q and of k, outputs head-major.
    e2e/sc_kernels.py:388-423."""
    w = h * d
    y = y_bits[:length]
    q = rmsnorm(y[:, :w], qn_bits, eps).reshape(length, h, d)
    k = rmsnorm(y[:, w:2 * w], kn_bits, eps).reshape(length, h, d)
    v = y[:, 2 * w:].reshape(length, h, d)
    return q.transpose(1, 0, 2).copy(), k.transpose(1, 0, 2).copy(), v.transpose(1, 0, 2).copy()
