"""The integer-exact 4-bit format family  w[n,k] = base[n] * m[n, k // B] * sign * C[idx]  (numpy, float32
decisions; test infrastructure).  C is an 8-entry integer codebook, m comes from a small ascending multiplier set,
base is one float per row.  Follows sim/formats.py:20-107 (quantizer) and e2e/pack_format.py:35-76 (packing)."""
import math
from dataclasses import dataclass

import numpy as np

from . import layout as L

CODEBOOKS = {                                                     # sim/formats.py:20-27
    "e2m1": (0, 1, 2, 3, 4, 6, 8, 12),
    "int4": (0, 1, 2, 3, 4, 5, 6, 7),
    "s10": (0, 1, 2, 3, 4, 6, 8, 10),
    "s14": (0, 1, 2, 3, 5, 7, 10, 14),
    "c10": (0, 1, 2, 3, 4, 5, 7, 10),
    "c9": (0, 1, 2, 3, 4, 5, 7, 9),
}


@dataclass(frozen=True)
class Family:
    codebook: str
    block: int
    mults: tuple
    base_grid: int = 8      # candidate row bases per octave (sim/formats.py:35)

    def storage(self):
        """The packed-storage Format of this family member (e2e/pack_format.py:35-42): block-code width is
        ceil(log2 |mults|) rounded up to 1, 2, 4 or 8 bits."""
        need = max(1, math.ceil(math.log2(len(self.mults))))
        bits = next(b for b in (1, 2, 4, 8) if b >= need)
        return L.Format(block=self.block, code_mag=CODEBOOKS[self.codebook], mult=tuple(self.mults), bc_bits=bits)


def member(name):
    """Parse 'e2m1/B16/pow2' or 'e2m1/B16/M1..10' (keys of sim/formats.py:116-133)."""
    cb, b, m = name.split()[0].split("/")
    if m == "pow2":
        mults = (1, 2, 4, 8)
    else:
        lo, hi = m[1:].split("..")
        mults = tuple(range(int(lo), int(hi) + 1))
    return Family(cb, int(b[1:]), mults)


def _nearest(x, cb):
    """Signed nearest codebook magnitude, ties to the lower one, saturating (sim/formats.py:58-61)."""
    cuts = (cb[1:] + cb[:-1]) / 2
    return np.sign(x) * cb[np.digitize(np.minimum(np.abs(x), cb[-1]), cuts, right=True)]


def quantize(w, fam, rows_per_chunk=256):
    """Returns (dequantized f32 [N,K], q int8 [N,K], base f32 [N], block scales base*m f64 [N, K/B]).

    Per row: the largest base is amax / (max mult * max code); 8 candidates per octave below it are tried in
    descending order, each with the per-block multiplier of least squared error (first minimum on ties), and a
    candidate replaces the best so far only when its total error is strictly smaller.  All decisions in float32.
    sim/formats.py:64-107."""
    cb = np.asarray(CODEBOOKS[fam.codebook], np.float32)
    mults = np.asarray(fam.mults, np.float32)
    if cb.max() * mults.max() > 127:
        raise ValueError("format overflows INT8")
    n, k = w.shape
    nb = k // fam.block
    deq = np.empty((n, k), np.float32)
    qint = np.empty((n, k), np.int8)
    bases = np.empty(n, np.float32)
    bscale = np.empty((n, nb), np.float64)
    for r0 in range(0, n, rows_per_chunk):
        wb = np.asarray(w[r0:r0 + rows_per_chunk], np.float32).reshape(-1, nb, fam.block)
        rows = wb.shape[0]
        peak = np.abs(wb).max((1, 2))
        peak = np.where(peak == 0, np.float32(1.0), peak)
        top = peak / (mults[-1] * cb.max())
        best_err = np.full(rows, np.inf, np.float32)
        best_base = top.copy()
        best_mi = np.zeros((rows, nb), np.int64)
        for j in range(fam.base_grid):
            base = top * 2.0 ** (-j / fam.base_grid)
            err = np.empty((rows, nb, len(mults)), np.float32)
            for i in range(len(mults)):
                s = (base[:, None, None] * mults[None, None, :])[:, :, i:i + 1]
                err[:, :, i] = ((_nearest(wb / s, cb) * s - wb) ** 2).sum(-1)
            mi = err.argmin(-1)
            total = np.take_along_axis(err, mi[..., None], -1)[..., 0].sum(-1)
            win = total < best_err
            best_err[win], best_base[win], best_mi[win] = total[win], base[win], mi[win]
        m = mults[best_mi]
        s = best_base[:, None, None] * m[..., None]
        qi = _nearest(wb / s, cb) * m[..., None]
        if np.abs(qi).max() > 127:
            raise AssertionError("operand exceeds INT8")
        sl = slice(r0, r0 + rows)
        deq[sl] = (qi * best_base[:, None, None]).reshape(rows, k)
        qint[sl] = qi.reshape(rows, k).astype(np.int8)
        bases[sl] = best_base
        bscale[sl] = best_base.astype(np.float64)[:, None] * m
    return deq, qint, bases, bscale


def pack_parts(qi, base, bscale, fmt):
    """(INT8 operands, row bases, block scales) -> (codes, bcodes, wscale) in storage Format fmt, with the
    exactness checks of e2e/pack_format.py:53-76 (dead rows, base == 0, become exactly zero)."""
    n, k = qi.shape
    dead = base == 0
    qi = np.where(dead[:, None], 0, qi).astype(np.int64)
    safe = np.where(dead, 1.0, base).astype(np.float64)
    m = np.where(dead[:, None], 1.0, bscale / safe[:, None])
    mi = np.rint(m).astype(np.int64)
    if not np.array_equal(m, mi):
        raise AssertionError("block scale / row base is not an integer")
    mults = np.asarray(fmt.mult)
    bcode = np.searchsorted(mults, mi)
    if not np.array_equal(mults[np.minimum(bcode, len(mults) - 1)], mi):
        raise AssertionError("multiplier not in the table")
    per_elem = np.repeat(mi, fmt.block, axis=1)
    mag = np.abs(qi) // per_elem
    if not np.array_equal(mag * per_elem, np.abs(qi)):
        raise AssertionError("operand is not code x multiplier")
    cm = np.asarray(fmt.code_mag)
    idx = np.searchsorted(cm, mag)
    if not np.array_equal(cm[np.minimum(idx, 7)], mag):
        raise AssertionError("magnitude not in the codebook")
    code4 = (idx | ((qi < 0).astype(np.int64) << 3)).astype(np.uint8)
    codes, bc, ws = L.pack_rows(code4, bcode.astype(np.uint8), base, fmt)
    if not np.array_equal(L.decode(codes, bc, n, k, fmt), qi.astype(np.int8)):
        raise AssertionError("packed layout does not decode to the operand")
    return codes, bc, ws
