"""SC-MXFP4 weight quantizer and its exact INT8 embedding (numpy, float64; test infrastructure).

An MXFP4 row stores w = 2^e_b * v with v on the E2M1 grid and one exponent e_b per block along K.  When the
exponents of a row span at most 3, the row is exactly  w = 2^(E_lo - 1) * q  with the integers
q = 2 v 2^(e_b - E_lo),  |q| <= 12 * 8 = 96   (sim/mx_int8.py:1-11).

The reference hard-wires 32-wide blocks; `block` is a parameter here so that the 16-wide power-of-two variant runs
through the identical procedure."""
import numpy as np

LEVELS = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0])      # E2M1 magnitudes, sim/mx_int8.py:19
BOUNDS = (LEVELS[:-1] + LEVELS[1:]) * 0.5                          # the 7 midpoints, sim/mx_int8.py:20
INT_MAG = np.array([0, 1, 2, 3, 4, 6, 8, 12])                      # 2 x E2M1, sim/make_testcase.py:23
MAX_SPREAD = 3                                                      # sim/mx_int8.py:18


def level_index(a):
    """Index of the E2M1 level nearest to magnitude a (already clipped to <= 6): the number of midpoints that lie
    strictly below a, so an exact midpoint goes to the LOWER level (sim/mx_int8.py:25, searchsorted side='left')."""
    return np.digitize(a, BOUNDS, right=True)


def round_e2m1(x):
    """Nearest E2M1 value with sign, saturating at +-6 (sim/mx_int8.py:23-25)."""
    x = np.asarray(x, dtype=np.float64)
    return np.sign(x) * LEVELS[level_index(np.minimum(np.abs(x), 6.0))]


def _pow2(e):
    """2^e for integer-valued float e, exact by construction."""
    return np.ldexp(1.0, np.asarray(e).astype(np.int64))


def as_blocks(w, block=32):
    n, k = w.shape
    if k % block:
        raise ValueError(f"K={k} is not a multiple of the block size {block}")
    return w.reshape(n, k // block, block)


def _block_sq_err(b, e):
    """Squared error of quantizing blocks b (N, nb, B) at exponents e (N, nb); sim/mx_int8.py:34-36."""
    step = _pow2(e)[..., None]
    v = round_e2m1(b / step)
    return ((v * step - b) ** 2).sum(-1)


def block_exponents(w, rule="search", block=32):
    """Per-block exponents (N, K/block); -inf marks an all-zero block.  sim/mx_int8.py:39-65.

    spec:   floor(log2 amax) - 2
    search: the spec exponent, replaced by spec-1 and then by spec+1 whenever that is STRICTLY better in squared
            error (candidates are tried in that order, each against the best so far)."""
    b = as_blocks(np.asarray(w, dtype=np.float64), block)
    amax = np.abs(b).max(-1)
    empty = amax == 0
    with np.errstate(divide="ignore"):
        lg = np.log2(amax)
    lg[empty] = 0.0
    if rule == "ceil":
        e = np.ceil(lg - np.log2(6.0))
    else:
        e = np.floor(lg) - 2.0
    if rule == "search":
        chosen = e.copy()
        chosen_err = _block_sq_err(b, e)
        for delta in (-1.0, 1.0):
            trial = e + delta
            trial_err = _block_sq_err(b, trial)
            win = trial_err < chosen_err
            chosen = np.where(win, trial, chosen)
            chosen_err = np.where(win, trial_err, chosen_err)
        e = chosen
    e[empty] = -np.inf
    return e


def constrain_spread(e, max_spread=MAX_SPREAD):
    """Raise exponents so a row spans at most max_spread; zero blocks (-inf) land on the floor, an all-zero row
    gets floor -max_spread (top 0).  Whole-row chunks only.  sim/mx_int8.py:68-81."""
    top = e.max(-1, keepdims=True)
    top = np.where(np.isfinite(top), top, 0.0)
    return np.maximum(e, top - max_spread)


def e2m1_values(w, e, block=32):
    """E2M1 values v (N, nb, B) of w at (finite) block exponents e, and the dequantized weights.
    sim/mx_int8.py:84-89."""
    b = as_blocks(np.asarray(w, dtype=np.float64), block)
    step = _pow2(np.where(np.isfinite(e), e, 0.0))[..., None]
    v = round_e2m1(b / step)
    return v, (v * step).reshape(w.shape)


def embed_int8(v, e):
    """Exact INT8 operand of E2M1 values v (N, nb, B) at exponents e (N, nb): returns (q int8 (N, K), shift uint8
    (N, nb) in 0..3, E_lo (N,), row scale 2^(E_lo - 1) float64 (N,)).  sim/mx_int8.py:92-109 with whole-row chunks,
    plus the shift extraction of sim/make_testcase.py:31-34."""
    n, nb, bs = v.shape
    fin = np.isfinite(e)
    top = np.where(fin, e, -np.inf).max(-1, keepdims=True)
    top = np.where(np.isfinite(top), top, 0.0)
    filled = np.where(fin, e, top)               # -inf blocks take the row maximum before the minimum is formed
    e_lo = filled.min(-1, keepdims=True)
    shift = filled - e_lo
    if shift.max(initial=0) > MAX_SPREAD:
        raise ValueError(f"row exponent spread {int(shift.max())} > {MAX_SPREAD}: not INT8-embeddable")
    q = 2.0 * v * _pow2(shift)[..., None]
    if np.abs(q).max(initial=0) > 127 or not np.array_equal(q, np.rint(q)):
        raise ValueError("embedding is not an INT8 integer")
    # make_testcase.py:33-34 gives -inf blocks shift 0 (they take `lo`); with -inf -> top they would get top-lo.
    # Both agree after constrain_spread (no -inf left); mirror make_testcase for raw exponents:
    shift_out = np.where(fin, e, e_lo) - e_lo
    return (q.reshape(n, nb * bs).astype(np.int8), shift_out.astype(np.uint8), e_lo[:, 0],
            _pow2(e_lo[:, 0] - 1.0))


def nibble_codes(v):
    """4-bit codes sign<<3 | level index of E2M1 values (any shape); -0.0 has sign bit 0.
    sim/make_testcase.py:36-38."""
    mag = np.abs(v)
    idx = np.searchsorted(LEVELS, mag)
    if not np.array_equal(LEVELS[np.minimum(idx, 7)], mag):
        raise ValueError("value not on the E2M1 grid")
    return (idx | ((v < 0).astype(np.int64) << 3)).astype(np.uint8)


def pack_from_values(v, e):
    """Byte-shift layout from E2M1 values and block exponents, no re-quantization: (codes u8 [N, K/2] with even k
    in the low nibble, shifts u8 [N, nb], wscale f32 [N], q int8 [N, K]).  e2e/gptq_pack.py:29-47 and
    sim/make_testcase.py:29-44."""
    q, shift, _, scale = embed_int8(v, e)
    n = v.shape[0]
    c = nibble_codes(v.reshape(n, -1))
    packed = (c[:, 0::2] | (c[:, 1::2] << 4)).astype(np.uint8)
    # layout self-check, as the reference asserts (make_testcase.py:41-43)
    sh = np.repeat(shift.astype(np.int64), v.shape[2], axis=1)
    dec = np.where(c & 8, -1, 1) * (INT_MAG[c & 7] << sh)
    if not np.array_equal(dec, q):
        raise AssertionError("packed layout does not decode to the INT8 operand")
    return packed, shift, scale.astype(np.float32), q


def pack(w, block=32):
    """Float weights (N, K) -> byte-shift layout of the SC-MXFP4 quantization.  sim/make_testcase.py:26-44."""
    w = np.asarray(w, dtype=np.float64)
    e = constrain_spread(block_exponents(w, "search", block))
    v, _ = e2m1_values(w, e, block)
    return pack_from_values(v, e)


def exponent_spread(e):
    """max - min finite exponent per row (0 for an all-zero row).  sim/mx_int8.py:112-122."""
    fin = np.isfinite(e)
    hi = np.where(fin, e, -np.inf).max(-1)
    lo = np.where(fin, e, np.inf).min(-1)
    s = hi - lo
    return np.where(np.isfinite(s), s, 0.0)
