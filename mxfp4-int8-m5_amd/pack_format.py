"""Packing float weights into a member of the integer-exact 4-bit format family
w[n, k] = base[n] * mult[n, k // B] * sign * code, on the device.  Mirrors the reference's e2e/pack_format.py
(sc_format_of :35-42, pack_matrix :45-50) with the quantizer of sim/formats.py:64-107 running as a HIP kernel
(scmx_quantize_family) instead of numpy; results are bit-identical."""
import math
import os

import numpy as np
import torch

from . import _lib
from . import sc_format as F

CODEBOOKS = {                                   # 8 code magnitudes per codebook, sim/formats.py:20-27
    "e2m1": (0, 1, 2, 3, 4, 6, 8, 12),
    "int4": (0, 1, 2, 3, 4, 5, 6, 7),
    "s10": (0, 1, 2, 3, 4, 6, 8, 10),
    "s14": (0, 1, 2, 3, 5, 7, 10, 14),
    "c10": (0, 1, 2, 3, 4, 5, 7, 10),
    "c9": (0, 1, 2, 3, 4, 5, 7, 9),
}


def slug(name):
    return name.replace("/", "_").replace(".", "")


def cache_path(repo, name, cache_dir):
    """File name of a model's packed cache in family member `name` (e2e/pack_format.py:79-80)."""
    return os.path.join(cache_dir, repo.replace("/", "--") + f"-fmt-{slug(name)}.safetensors")


def sc_format_of(name):
    """Format name "<codebook>/B<block>/pow2" or "<codebook>/B<block>/M<lo>..<hi>" (the keys of sim/formats.py:116-133)
    -> sc_format.Format for the kernels; the block-code width is ceil(log2 |mults|) rounded up to 1, 2, 4 or 8."""
    cb, b, m = name.split()[0].split("/")
    if m == "pow2":
        mults = (1, 2, 4, 8)
    else:
        lo, hi = m[1:].split("..")
        mults = tuple(range(int(lo), int(hi) + 1))
    need = max(1, math.ceil(math.log2(len(mults))))
    bits = next(x for x in (1, 2, 4, 8) if x >= need)
    return F.Format(block=int(b[1:]), code_mag=CODEBOOKS[cb], mult=mults, bc_bits=bits)


def pack_matrix(w, name, fmt=None):
    """float weights [N, K] (torch float32 / bfloat16, or numpy -> float32) -> (codes, bcodes, wscale, stats) in the
    family member `name`; wscale is the row base.  stats["exact_q"]: the packed layout decodes to code x multiplier
    by construction here (the host packer re-checks it, e2e/pack_format.py:70-74)."""
    fmt = fmt or sc_format_of(name)
    if isinstance(w, np.ndarray):
        w = torch.from_numpy(np.ascontiguousarray(w, np.float32)).cuda()
    if w.dtype not in (torch.float32, torch.bfloat16):
        w = w.float()
    w = w.contiguous()
    n, k = w.shape
    codes = torch.empty(n * k // 8, dtype=torch.int32, device=w.device)
    bc = torch.empty((n, k // fmt.block // fmt.per_byte), dtype=torch.uint8, device=w.device)
    ws = torch.empty(n, dtype=torch.float32, device=w.device)
    _lib.call("scmx_quantize_family", fmt.c_struct(), _lib.ptr(w), int(w.dtype == torch.bfloat16), n, k, _lib.ptr(codes),
              _lib.ptr(bc), _lib.ptr(ws), _lib.stream())
    return codes, bc, ws, dict(exact_q=True)
