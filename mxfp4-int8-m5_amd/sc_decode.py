"""Decode GEMV call surface (the reference's e2e/sc_decode.py) on torch tensors over libscmx.so.

`gemv` keeps the reference's signature; `rows` / `vpl` / `nsg` / `splitk` are accepted as hints (the kernel picks its
own launch shape and the result never depends on it).  New here: a 2-D `xq` [B, K] without `eidx` runs B input rows
against one pass over the weights (batch 2, 4 or 8) and returns [B, N]."""
import torch

from . import _lib
from . import sc_format as F
from . import sc_kernels as S

GEMV_TILE = (4, 16, 2)
GEMV_TILES = {}


def gemv(xq, codes, bcodes, xscale, wscale, N, epi, dtype=torch.bfloat16, res=None, nsg=None, eidx=None, xstride=0,
         pro=0, nw=None, eps=None, rows=None, vpl=None, shared=None, splitk=None, fmt=None):
    """W4A8 GEMV.  pro=0: xq int8 [K] (or rows) with xscale; pro=1: xq is a bf16 row quantized in the kernel;
    pro=2: RMSNorm(nw, eps) + INT8 in the kernel.  Output EPI 1: [N]; 2: [N] = res + y; 3: [N/2].
    xq [B, K] with B = 2 ... 8 rows shares one pass over the weights (3, 5, 6, 7 rows are padded to 4 / 8; more than 8
    rows take one pass per eight -- from a few dozen rows on the dense GEMM is the faster path).
    MoE (eidx int32 [S]): codes [E, ..], wscale [E, N]; slot j uses expert eidx[j] and input row j if xstride=1;
    shared=e adds one slot for expert e -> [S(+1), N or N/2]."""
    S._check_dtype(dtype)
    fmt = fmt or F.DEFAULT
    K = xq.shape[-1]
    no = N // 2 if epi == 3 else N
    batch, nslot = 1, 0
    if eidx is not None:
        nslot = eidx.numel()
        slots = nslot + (shared is not None)
        eidx = eidx if eidx.dtype == torch.int32 else eidx.view(torch.int32) if eidx.element_size() == 4 else eidx.to(torch.int32)
        out = torch.empty((slots, no), dtype=torch.bfloat16, device=xq.device)
    elif xq.dim() == 2 and xq.shape[0] > 8:   # more rows than one pass takes: eight at a time
        cut = lambda t, i: None if t is None else t[i:i + 8]   # noqa: E731
        return torch.cat([gemv(xq[i:i + 8], codes, bcodes, cut(xscale, i), wscale, N, epi, dtype, cut(res, i), nsg, None,
                               xstride, pro, nw, eps, rows, vpl, shared, splitk, fmt).reshape(-1, no)
                          for i in range(0, xq.shape[0], 8)])
    elif xq.dim() == 2 and xq.shape[0] in (3, 5, 6, 7):   # the kernels take 1, 2, 4 or 8 rows: pad with zero rows
        b, bp = xq.shape[0], 4 if xq.shape[0] == 3 else 8
        pad = lambda t: None if t is None else torch.cat([t, t.new_zeros((bp - b,) + tuple(t.shape[1:]))])   # noqa: E731
        return gemv(pad(xq), codes, bcodes, pad(xscale), wscale, N, epi, dtype, pad(res), nsg, None, xstride, pro, nw, eps,
                    rows, vpl, shared, splitk, fmt)[:b]
    elif xq.dim() == 2 and xq.shape[0] > 1:
        batch = xq.shape[0]
        out = torch.empty((batch, no), dtype=torch.bfloat16, device=xq.device)
    else:
        out = torch.empty(no, dtype=torch.bfloat16, device=xq.device)
    assert (pro == 0 and xq.dtype == torch.int8) or (pro in (1, 2) and xq.dtype == torch.bfloat16)
    _lib.call("scmx_gemv", fmt.c_struct(), _lib.ptr(xq), _lib.ptr(xscale) if pro == 0 else None, _lib.ptr(codes),
              _lib.ptr(bcodes), _lib.ptr(wscale), _lib.ptr(res) if epi == 2 else None, _lib.ptr(out), epi, pro,
              _lib.ptr(nw) if pro == 2 else None, S._eps(eps) if pro == 2 else 0.0, batch, N, K,
              _lib.ptr(eidx) if eidx is not None else None, nslot, xstride, -1 if shared is None else int(shared),
              _lib.stream())
    return out
