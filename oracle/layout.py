"""Packed storage of INT8-exact 4-bit weights (numpy; test infrastructure).

Row n of a (N, K) matrix is held as
  codes   uint32 [N*K/8]  eight 4-bit codes per word; element k = 8j + i sits in bits 4i..4i+3 of word j
                          (= the nibble-per-byte array, even k low, viewed little-endian); code = sign<<3 | idx
  bcodes  uint8 [N, K*bc_bits/(8*block)]  block b of a row in bits bc_bits*(b % per_byte) of byte b // per_byte
  wscale  f32 [N]
and decodes to q[n, k] = +-code_mag[idx] * mult[bcode[n, k // block]]   (e2e/sc_format.py:4-15)."""
from dataclasses import dataclass

import numpy as np

from . import quantizer as Q


@dataclass(frozen=True)
class Format:
    """Format descriptor with the invariants of e2e/sc_format.py:26-37."""
    block: int = 32
    code_mag: tuple = (0, 1, 2, 3, 4, 6, 8, 12)
    mult: tuple = (1, 2, 4, 8)
    bc_bits: int = 2

    def __post_init__(self):
        if self.block % 8:
            raise ValueError("block must be a multiple of 8 (one code word never straddles two blocks)")
        if self.bc_bits not in (1, 2, 4, 8) or len(self.mult) > 2 ** self.bc_bits:
            raise ValueError("bc_bits must be 1, 2, 4 or 8 and index every multiplier")
        if len(self.code_mag) != 8 or max(self.code_mag) * max(self.mult) > 127:
            raise ValueError("need 8 code magnitudes with max(code_mag) * max(mult) <= 127")

    @property
    def per_byte(self):
        return 8 // self.bc_bits

    def bits_per_weight(self, k):
        return 4 + self.bc_bits / self.block + 32 / k            # e2e/sc_format.py:43-44


DEFAULT = Format()


def _pack_bcodes(bcode, fmt):
    n, nb = bcode.shape
    if nb % fmt.per_byte:
        raise ValueError("blocks per row must fill whole block-code bytes")
    grp = bcode.astype(np.uint32).reshape(n, nb // fmt.per_byte, fmt.per_byte)
    sh = (np.arange(fmt.per_byte, dtype=np.uint32) * fmt.bc_bits)
    return (grp << sh).sum(-1).astype(np.uint8)


def pack_rows(code4, bcode, wscale, fmt=DEFAULT):
    """code4 u8 [N, K], bcode u8 [N, K/block], wscale [N] -> (codes u32 flat, bcodes u8, wscale f32).
    e2e/sc_format.py:66-80."""
    n, k = code4.shape
    if k % fmt.block or bcode.shape != (n, k // fmt.block) or bcode.max(initial=0) >= len(fmt.mult):
        raise ValueError("bad shapes or block code out of range")
    c = code4.astype(np.uint32).reshape(n, k // 8, 8)
    words = (c << (np.arange(8, dtype=np.uint32) * 4)).sum(-1, dtype=np.uint32)
    return words.reshape(-1), _pack_bcodes(bcode, fmt), np.asarray(wscale, np.float32)


def unpack_fields(codes, bcodes, n, k, fmt=DEFAULT):
    """(code4 u8 [N, K], bcode u8 [N, K/block]) of a packed matrix."""
    w = np.asarray(codes, np.uint32).reshape(n, k // 8, 1)
    c = ((w >> (np.arange(8, dtype=np.uint32) * 4)) & 0xF).reshape(n, k).astype(np.uint8)
    bb = np.asarray(bcodes, np.uint8).reshape(n, -1, 1)
    b = (bb >> (np.arange(fmt.per_byte, dtype=np.uint8) * fmt.bc_bits)) & (2 ** fmt.bc_bits - 1)
    return c, b.reshape(n, -1)[:, :k // fmt.block].astype(np.uint8)


def decode(codes, bcodes, n, k, fmt=DEFAULT):
    """Packed layout -> INT8 operand q [N, K].  e2e/sc_format.py:83-90."""
    c, b = unpack_fields(codes, bcodes, n, k, fmt)
    mag = np.asarray(fmt.code_mag, np.int32)[c & 7] * np.repeat(np.asarray(fmt.mult, np.int32)[b], fmt.block, 1)
    return np.where(c & 8, -mag, mag).astype(np.int8)


def from_shift_layout(codes_u8, shifts, wscale, fmt=DEFAULT):
    """Byte-shift layout (codes u8 [N, K/2], shifts u8 [N, K/32] in 0..3) -> this format; no requantization.
    e2e/sc_format.py:93-102."""
    if fmt.block * len(fmt.mult) == 0 or tuple(fmt.mult) != (1, 2, 4, 8):
        raise ValueError("the shift layout is a power-of-two multiplier format")
    words = np.ascontiguousarray(codes_u8, np.uint8).reshape(-1).view("<u4")
    return words.astype(np.uint32), _pack_bcodes(np.asarray(shifts, np.uint8), fmt), np.asarray(wscale, np.float32)


def quantize(w, fmt=DEFAULT):
    """Float weights -> (codes, bcodes, wscale, q int8) with the SC-MXFP4 quantizer.  e2e/sc_format.py:105-111
    (block 32); block 16 runs the same procedure on 16-wide blocks."""
    packed, shifts, wscale, q = Q.pack(w, fmt.block)
    codes, bc, ws = from_shift_layout(packed, shifts, wscale, fmt)
    return codes, bc, ws, q


# ---- standard MXFP4 view: the same nibbles plus one E8M0 byte per 32-block --------------------------------------

def to_mxfp4(codes, bcodes, wscale, n, k, fmt=DEFAULT):
    """(nibble bytes u8 [N, K/2], E8M0 u8 [N, K/32]) of a packed SC-MXFP4 matrix:
    E8M0 = log2(wscale) + 1 + shift + 127 and the code nibbles are OCP E2M1 nibbles unchanged.
    e2e/fused_qwen38.py:319-334."""
    if fmt != DEFAULT:
        raise ValueError("only the 32-block power-of-two format is a standard MXFP4 tensor")
    _, shift = unpack_fields(codes, bcodes, n, k, fmt)
    e = np.log2(np.asarray(wscale, np.float64))[:, None] + 1 + shift
    if not np.array_equal(e, np.rint(e)):
        raise ValueError("row scale is not a power of two")
    e8 = e + 127
    if e8.min() < 0 or e8.max() > 254:
        raise ValueError("exponent outside E8M0")
    return np.asarray(codes, "<u4").view(np.uint8).reshape(n, k // 2).copy(), e8.astype(np.uint8)


def from_mxfp4(nibbles, e8m0):
    """Standard MXFP4 tensor (nibbles u8 [N, K/2], E8M0 u8 [N, K/32]) -> (codes, bcodes, wscale) in the default
    format; raises when a row's exponents span more than 3.  Inverse of to_mxfp4; the CPU form of
    e2e/gptq_pack.py:29-47 when the input is already (values, exponents)."""
    e = np.asarray(e8m0, np.int32)
    lo = e.min(-1, keepdims=True)
    shift = e - lo
    if shift.max(initial=0) > Q.MAX_SPREAD:
        raise ValueError("row exponent spread > 3: not INT8-embeddable")
    wscale = np.ldexp(1.0, lo[:, 0] - 127 - 1).astype(np.float32)
    return from_shift_layout(nibbles, shift.astype(np.uint8), wscale, DEFAULT)
