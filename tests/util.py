"""Shared helpers of the GPU parity tests: seeded inputs of the benchmark configurations and numpy <-> torch glue."""
import numpy as np
import torch

from oracle import bf16, layout

F32 = np.float32


def dev(a):
    """numpy -> CUDA tensor (uint32 as int32 bit patterns, uint16 as bfloat16 bit patterns)."""
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint32:
        return torch.from_numpy(a.view(np.int32)).cuda()
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16)).cuda().view(torch.bfloat16)
    return torch.from_numpy(a).cuda()


def host(t):
    """CUDA tensor -> numpy (bfloat16 as uint16 bit patterns)."""
    t = t.detach().contiguous().cpu()
    if t.dtype == torch.bfloat16:
        return t.view(torch.int16).numpy().view(np.uint16)
    return t.numpy()


def llm_weights(rng, n, k, outliers=True):
    """N(0, 0.02) weights with 0.5% of the input columns scaled by 8."""
    w = rng.standard_normal((n, k)) * 0.02
    if outliers:
        w[:, rng.choice(k, max(1, round(0.005 * k)), replace=False)] *= 8
    return w


def llm_acts(rng, m, k):
    """bf16 N(0, 1) activations with 1% of the channels scaled by 20, as (bf16 bits, FP32 values)."""
    x = rng.standard_normal((m, k))
    x[:, rng.choice(k, max(1, round(0.01 * k)), replace=False)] *= 20
    bits = bf16.to_bits(x.astype(F32))
    return bits, bf16.from_bits(bits)


def random_packed(rng, n, k, fmt=layout.DEFAULT):
    """Random codes and block codes in `fmt` (cheap stand-in for a quantized matrix): packed arrays + INT8 operand."""
    c4 = rng.integers(0, 16, (n, k)).astype(np.uint8)
    b = rng.integers(0, len(fmt.mult), (n, k // fmt.block)).astype(np.uint8)
    ws = np.exp2(rng.integers(-12, -6, n)).astype(F32)
    codes, bc, ws = layout.pack_rows(c4, b, ws, fmt)
    return codes, bc, ws, layout.decode(codes, bc, n, k, fmt)


def blocked_layout(xq):
    """INT8 activations [Mp, K] (Mp % 32 == 0, K % 32 == 0) -> the flat blocked layout of scmx_act_quant_blocked: 32 x 32
    blocks, block (m / 32, k / 32) at ((m / 32) * (K / 32) + k / 32) KB, inside it row r, k half h at (32 h + r) * 16."""
    mp, k = xq.shape
    return np.ascontiguousarray(xq.reshape(mp // 32, 32, k // 32, 2, 16).transpose(0, 2, 3, 1, 4)).reshape(-1)


def product_format(fmt):
    """oracle layout.Format -> the product's sc_format.Format."""
    from mxfp4_int8_m5_amd import sc_format
    return sc_format.Format(block=fmt.block, code_mag=tuple(fmt.code_mag), mult=tuple(fmt.mult), bc_bits=fmt.bc_bits)


FORMATS = [layout.Format(), layout.Format(block=16), layout.Format(block=32, mult=(1, 2, 3, 4)),
           layout.Format(block=16, mult=(1, 2, 3, 4, 5, 6, 8, 10), bc_bits=4),
           layout.Format(block=32, code_mag=(0, 1, 2, 3, 4, 5, 6, 7), mult=(1, 3, 9, 15)),
           layout.Format(block=16, mult=tuple(range(1, 11)), bc_bits=4)]     # "e2m1/B16/M1..10": consecutive multipliers
