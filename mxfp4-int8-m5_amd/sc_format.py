"""Storage format of the 4-bit weights, host side: the descriptor the kernels are called with and the bit-packing
of already-quantized codes.  Mirrors the interface of the reference's e2e/sc_format.py (Format, DEFAULT, pack_rows,
from_shift_layout); decoding runs on the GPU (sc_kernels.unpack_i8).

Layouts (row-major over N, K contiguous):
  codes   uint32 [N*K/8]   element k = 8j+i in bits 4i..4i+3 of word j; code = sign<<3 | index into code_mag
  bcodes  uint8 [N, K*bc_bits/(8*block)]   block b in bits bc_bits*(b % per_byte) of byte b // per_byte
  wscale  f32 [N]
"""
from dataclasses import dataclass

import numpy as np
import torch

from . import _lib


@dataclass(frozen=True)
class Format:
    block: int = 32
    code_mag: tuple = (0, 1, 2, 3, 4, 6, 8, 12)
    mult: tuple = (1, 2, 4, 8)
    bc_bits: int = 2
    inline_mult: bool = False   # accepted for interface compatibility; the kernels need no such hint

    def __post_init__(self):
        assert self.block % 8 == 0, "one code word (8 weights) must lie in one block"
        if not self.mult:   # MXFP4: the block bytes are E8M0 exponents, the multiplier is 2^(byte - the row's lowest)
            assert self.block == 32 and self.bc_bits == 8 and tuple(self.code_mag) == (0, 1, 2, 3, 4, 6, 8, 12)
            return
        assert self.bc_bits in (1, 2, 4, 8) and len(self.mult) <= 2 ** self.bc_bits
        assert len(self.code_mag) == 8 and max(self.code_mag) * max(self.mult) <= 127, "must fit INT8"

    @property
    def e8m0(self):
        """True for a standard MXFP4 tensor read in place (`MXFP4` below)."""
        return not self.mult

    @property
    def per_byte(self):
        return 8 // self.bc_bits

    def bits_per_weight(self, K):
        return 4 + self.bc_bits / self.block + 32 / K

    def c_struct(self):
        """The scmx_format passed across the C ABI."""
        if len(self.mult) > 16:
            raise ValueError("the kernels take at most 16 block multipliers")
        f = _lib.CFormat()
        f.block, f.bc_bits, f.n_mult = self.block, self.bc_bits, len(self.mult)
        for i, v in enumerate(self.code_mag):
            f.code_mag[i] = int(v)
        for i, v in enumerate(self.mult):
            f.mult[i] = int(v)
        return f


DEFAULT = Format()
# A standard MXFP4 tensor read in place (e2e/fused_qwen38.py:319-334): `codes` = its E2M1 nibble bytes, `bcodes` = its
# E8M0 bytes uint8 [N, K/32], `wscale` = mxfp4_row_scales(e8m0).  Taken by gemv, mm_epi / linear_w4a8 on a PackedWq,
# and moe_mm; 4.25 bits per weight + 32 / K.
MXFP4 = Format(block=32, mult=(), bc_bits=8)


def _pack_bcodes(bcode, fmt):
    n, nb = bcode.shape
    assert nb % fmt.per_byte == 0
    grp = bcode.astype(np.uint32).reshape(n, nb // fmt.per_byte, fmt.per_byte)
    return (grp << (np.arange(fmt.per_byte, dtype=np.uint32) * fmt.bc_bits)).sum(-1).astype(np.uint8)


def pack_rows(code4, bcode, wscale, fmt=None):
    """code4 uint8 [N, K] (sign << 3 | idx), bcode uint8 [N, K/block], wscale [N] -> (codes, bcodes, wscale)."""
    fmt = fmt or DEFAULT
    n, k = code4.shape
    assert k % fmt.block == 0 and bcode.max(initial=0) < len(fmt.mult)
    c = code4.astype(np.uint32).reshape(n, k // 8, 8)
    codes = (c << (np.arange(8, dtype=np.uint32) * 4)).sum(-1, dtype=np.uint32).reshape(-1)
    return codes, _pack_bcodes(np.asarray(bcode, np.uint8), fmt), np.asarray(wscale, np.float32)


def decode_numpy(codes, bcodes, N, K, fmt=None):
    """Host-side decode of a packed matrix to the INT8 operand q [N, K], for checks and tools (the kernels never
    call it; the device decode is sc_kernels.unpack_i8).  e2e/sc_format.py:83-90."""
    fmt = fmt or DEFAULT
    w = np.asarray(codes, np.uint32).reshape(N, K // 8)
    c = ((w[:, :, None] >> (4 * np.arange(8, dtype=np.uint32))) & 0xF).reshape(N, K).astype(np.int64)
    b = np.arange(K // fmt.block)
    bc = (np.asarray(bcodes, np.uint8)[:, b // fmt.per_byte].astype(np.int64) >> (fmt.bc_bits * (b % fmt.per_byte))) \
        & ((1 << fmt.bc_bits) - 1)
    mag = np.asarray(fmt.code_mag, np.int64)[c & 7] * np.repeat(np.asarray(fmt.mult, np.int64)[bc], fmt.block, axis=1)
    return np.where(c & 8, -mag, mag).astype(np.int8)


def from_shift_layout(codes_u32, shifts, wscale, fmt=None):
    """Byte-shift layout (codes, shifts uint8 [N, K/32] in 0..3, wscale) -> packed block codes; no requantization."""
    fmt = fmt or DEFAULT
    assert tuple(fmt.mult) == (1, 2, 4, 8), "the shift layout is the power-of-two format"
    return (np.asarray(codes_u32, np.uint32).reshape(-1), _pack_bcodes(np.asarray(shifts, np.uint8), fmt),
            np.asarray(wscale, np.float32))


def to_shift_layout(codes_u32, bcodes, wscale, fmt=None):
    """The inverse of from_shift_layout: packed 2-bit block codes -> shifts uint8 [N, K/32] (one byte per block), the
    layout of the round-to-nearest weight cache (e2e/w4a8_mlx.py:167-195)."""
    fmt = fmt or DEFAULT
    assert tuple(fmt.mult) == (1, 2, 4, 8), "the shift layout is the power-of-two format"
    bc = np.asarray(bcodes, np.uint8)
    parts = [(bc >> (fmt.bc_bits * j)) & ((1 << fmt.bc_bits) - 1) for j in range(fmt.per_byte)]
    shifts = np.stack(parts, axis=-1).reshape(bc.shape[0], -1)
    return np.asarray(codes_u32, np.uint32).reshape(-1), np.ascontiguousarray(shifts, np.uint8), np.asarray(wscale, np.float32)


def to_device(codes, bcodes, wscale, device="cuda"):
    """numpy packed arrays -> torch tensors (codes as int32 bit patterns; torch has no uint32 arithmetic)."""
    return (torch.from_numpy(np.ascontiguousarray(codes, np.uint32).view(np.int32)).to(device),
            torch.from_numpy(np.ascontiguousarray(bcodes, np.uint8)).to(device),
            torch.from_numpy(np.ascontiguousarray(wscale, np.float32)).to(device))


def from_mxfp4(nibbles, e8m0):
    """Standard MXFP4 on the GPU: nibbles uint8 [N, K/2] (E2M1 codes, even k low) and E8M0 uint8 [N, K/32] ->
    (codes, bcodes, wscale) of the default format.  Raises if a row's exponents span more than 3."""
    n, nb = e8m0.shape
    k = nb * 32
    assert nibbles.shape == (n, k // 2) and nibbles.dtype == torch.uint8 and e8m0.dtype == torch.uint8
    bc = torch.empty((n, nb // 4), dtype=torch.uint8, device=e8m0.device)
    ws = torch.empty(n, dtype=torch.float32, device=e8m0.device)
    status = torch.zeros(1, dtype=torch.int32, device=e8m0.device)
    _lib.call("scmx_mxfp4_to_sc", _lib.ptr(e8m0), _lib.ptr(bc), _lib.ptr(ws), _lib.ptr(status), n, k, _lib.stream())
    if int(status.item()) & 1:
        raise ValueError("a row's block exponents span more than 3: not INT8-embeddable")
    return nibbles.contiguous().view(torch.int32).reshape(-1), bc, ws


def mxfp4_row_scales(e8m0):
    """The row scales that let the kernels read a standard MXFP4 tensor in place (fmt=MXFP4): wscale [N] =
    2^(lowest E8M0 byte of the row - 128).  Raises if a row's exponents span more than 3 or hold the bytes 0 / 255."""
    n, nb = e8m0.shape
    assert e8m0.dtype == torch.uint8
    ws = torch.empty(n, dtype=torch.float32, device=e8m0.device)
    status = torch.zeros(1, dtype=torch.int32, device=e8m0.device)
    _lib.call("scmx_mxfp4_to_sc", _lib.ptr(e8m0), None, _lib.ptr(ws), _lib.ptr(status), n, nb * 32, _lib.stream())
    st = int(status.item())
    if st & 1:
        raise ValueError("a row's block exponents span more than 3: not INT8-embeddable")
    if st & 2:
        raise ValueError("exponent bytes 0 and 255 cannot be read in place; convert with from_mxfp4")
    return ws


def mxfp4_codes(nibbles):
    """The nibble bytes of a standard MXFP4 tensor [N, K/2] as the kernels' code words (a view, no copy)."""
    return nibbles.contiguous().view(torch.int32).reshape(-1)


def quantize(w, fmt=None, with_q=True):
    """(N, K) float weights (torch tensor on the GPU, float32 or bfloat16; a numpy array is uploaded as float32) ->
    (codes, bcodes, wscale, q) with the SC-MXFP4 quantizer running on the device, bit-identical to the host
    procedure of the reference (e2e/sc_format.py:105-111, sim/make_testcase.py:26-44).  fmt: DEFAULT (32-blocks) or
    the 16-block power-of-two format.  q is the INT8 operand [N, K] (None when with_q is false)."""
    fmt = fmt or DEFAULT
    if tuple(fmt.mult) != (1, 2, 4, 8) or fmt.bc_bits != 2 or fmt.block not in (16, 32) or \
            tuple(fmt.code_mag) != tuple(DEFAULT.code_mag):
        raise ValueError("the device quantizer produces the power-of-two formats with 16- or 32-wide blocks")
    if isinstance(w, np.ndarray):
        w = torch.from_numpy(np.ascontiguousarray(w, np.float32)).cuda()
    if w.dtype not in (torch.float32, torch.bfloat16):
        w = w.float()
    w = w.contiguous()
    n, k = w.shape
    codes = torch.empty(n * k // 8, dtype=torch.int32, device=w.device)
    bc = torch.empty((n, k // (4 * fmt.block)), dtype=torch.uint8, device=w.device)
    ws = torch.empty(n, dtype=torch.float32, device=w.device)
    _lib.call("scmx_quantize_sc", _lib.ptr(w), int(w.dtype == torch.bfloat16), n, k, fmt.block, _lib.ptr(codes),
              _lib.ptr(bc), _lib.ptr(ws), _lib.stream())
    q = None
    if with_q:
        q = torch.empty((n, k), dtype=torch.int8, device=w.device)
        _lib.call("scmx_unpack_i8", fmt.c_struct(), _lib.ptr(codes), _lib.ptr(bc), _lib.ptr(q), n, k, _lib.stream())
    return codes, bc, ws, q
