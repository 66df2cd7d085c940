"""Grouped expert GEMM call surface (the reference's e2e/sc_moe.py) on torch tensors over libscmx.so.

Token-expert assignments are sorted by expert (`route_sort`), expert e owns rows [off[e], off[e+1]) of the sorted
activations, and one launch of the grouped INT8-MFMA GEMM covers all experts, each workgroup unpacking its expert's
weight tile in LDS.  Unlike the reference, `moe_mm` needs no padding rows after the R sorted rows (row indices are
clamped inside the kernel) and can gather the activation rows itself: pass the UNSORTED `xq`/`xscale` with
`gather=tok` to skip the xq[tok] copy.
"""
import torch

from . import _lib
from . import sc_format as F
from . import sc_kernels as S


def route(logits, k, renorm=True, shared_logit=None):
    """Router on bf16 logits [M, E]: (inds int32 [M, k], scores bf16 [M, k]) = the k experts of largest softmax
    probability (float32 softmax rounded to bf16) and their probabilities, divided by their sum when `renorm`
    (e2e/fused_olmoe.py:183-192).  shared_logit bf16 [M]: a last slot with expert index E and score
    sigmoid(shared_logit), outputs [M, k + 1] (e2e/fused_qwen35.py:171-180).  Slots are listed by falling probability."""
    M, E = logits.shape
    assert logits.dtype == torch.bfloat16 and (shared_logit is None or shared_logit.dtype == torch.bfloat16)
    logits = logits.contiguous()
    if shared_logit is not None:
        shared_logit = shared_logit.reshape(M).contiguous()
    width = k + (shared_logit is not None)
    inds = torch.empty((M, width), dtype=torch.int32, device=logits.device)
    scores = torch.empty((M, width), dtype=torch.bfloat16, device=logits.device)
    _lib.call("scmx_route_topk", _lib.ptr(logits), _lib.ptr(shared_logit), M, E, k, int(bool(renorm)), _lib.ptr(inds),
              _lib.ptr(scores), _lib.stream())
    return inds, scores


def route_sort(inds, n_experts, tm):
    """inds int [M, topk] -> (pos [R], tok [R + tm], e_sorted [R], off [E+1], tstart [E+1], max M-tiles)."""
    M, k = inds.shape
    R = M * k
    inds = inds.to(torch.int32).contiguous()
    dev = inds.device
    pos = torch.empty(R, dtype=torch.int32, device=dev)
    tok = torch.empty(R + tm, dtype=torch.int32, device=dev)
    es = torch.empty(R, dtype=torch.int32, device=dev)
    off = torch.empty(n_experts + 1, dtype=torch.int32, device=dev)
    ts = torch.empty(n_experts + 1, dtype=torch.int32, device=dev)
    _lib.call("scmx_route_sort", _lib.ptr(inds), M, k, n_experts, tm, _lib.ptr(pos), _lib.ptr(tok), _lib.ptr(es),
              _lib.ptr(off), _lib.ptr(ts), _lib.stream())
    return pos, tok, es, off, ts, -(-R // tm) + n_experts


def row_tile(R, n_experts):
    """Row tile of the grouped GEMM for R assignments over n_experts: 256-row tiles (the fewest LDS bytes per MFMA) from
    about 96 rows per expert on, below that 64-row tiles (less padding, packed weights in LDS).  Measured on 64 experts
    of 2048 x 2048 / 2048 x 1024 with top-8 routing: 512 tokens 149 us with 64-row tiles against 169 with 256-row ones,
    1024 tokens 205 against 180."""
    return 256 if R >= 96 * n_experts else 64


def segments(expert_sorted, n_experts, tm):
    """Sorted expert id per row -> (off int32 [E+1], tstart int32 [E+1], max number of M-tiles)."""
    R = expert_sorted.shape[0]
    counts = torch.bincount(expert_sorted.to(torch.int64), minlength=n_experts).to(torch.int32)
    zero = torch.zeros(1, dtype=torch.int32, device=counts.device)
    off = torch.cat([zero, torch.cumsum(counts, 0).to(torch.int32)])
    tstart = torch.cat([zero, torch.cumsum((counts + tm - 1) // tm, 0).to(torch.int32)])
    return off, tstart, -(-R // tm) + n_experts


def _out(R, N, epi, dev):
    if epi == 0:
        return torch.empty((R, N), dtype=torch.int32, device=dev)
    return torch.empty((R, N // 2 if epi == 3 else N), dtype=torch.bfloat16, device=dev)


def moe_mm(xq, R, codes, bcodes, wscale, off, tstart, max_tiles, N, epi, xscale=None, dtype=torch.bfloat16,
           tile=(64, 64, 4), bk=128, gather=None, fmt=None):
    """Grouped W4A8 GEMM.  xq int8 [>= R, K] sorted by expert (or unsorted with gather=tok); packed expert weights
    codes [E, N*K/8], bcodes [E, N, ..], wscale f32 [E, N] -> INT32 [R, N] (EPI 0), bf16 [R, N] (1) or
    bf16 [R, N/2] (3, interleaved gate/up).  tile[0] is the row tile the segments were built for (64, 128 or 256)."""
    fmt = fmt or F.DEFAULT
    K = xq.shape[1]
    E = wscale.shape[0]
    assert xq.dtype == torch.int8 and (gather is not None or xq.shape[0] >= R)
    out = _out(R, N, epi, xq.device)
    _lib.call("scmx_moe_mm", fmt.c_struct(), _lib.ptr(xq), _lib.ptr(xscale), _lib.ptr(gather), R, _lib.ptr(codes),
              _lib.ptr(bcodes), _lib.ptr(wscale), _lib.ptr(off), _lib.ptr(tstart), E, tile[0], N, K, epi, _lib.ptr(out),
              _lib.stream())
    return out


def moe_mm_i8(xq, R, wq, wscale, off, tstart, max_tiles, N, epi, xscale=None, dtype=torch.bfloat16, tile=(64, 64, 4),
              gather=None):
    """Two-pass variant: wq int8 [E * N, K] already unpacked (unpack_experts)."""
    K = xq.shape[1]
    E = wscale.shape[0]
    if isinstance(wq, S.PackedWq):
        wq = wq.materialize()
    assert tuple(wq.shape) == (E * N, K)
    out = _out(R, N, epi, xq.device)
    _lib.call("scmx_moe_mm_i8", _lib.ptr(xq), _lib.ptr(xscale), _lib.ptr(gather), R, _lib.ptr(wq), _lib.ptr(wscale),
              _lib.ptr(off), _lib.ptr(tstart), E, tile[0], N, K, epi, _lib.ptr(out), _lib.stream())
    return out


def unpack_experts(codes, bcodes, N, K):
    """All experts' packed weights -> INT8 [E * N, K] (one unpack launch)."""
    E = codes.shape[0]
    return S.unpack_i8(codes.reshape(-1), bcodes.reshape(E * N, -1), E * N, K, lazy=False)


def moe_combine(y, pos, scores, res, w, eps, M, quant=True):
    """y bf16 [R, K] (sorted assignments), pos int32 [M*topk], scores bf16 [M, topk], res [Mp, K] ->
    (h [Mp, K], xq int8 [Mp, K], xscale [Mp]) with xq = INT8(rms_norm(h, w)); quant=False returns xq = xs = None.
    (The reference keeps this in e2e/fused_olmoe.py:87-97.)"""
    return _combine(y, pos, scores, None, res, w, eps, M, quant)


def moe_combine_split(y, pos, scores, sscore, res, w, eps, M):
    """moe_combine (no quantization) whose last slot's score is given separately (e2e/fused_olmoe.py:74-84)."""
    return _combine(y, pos, scores, sscore, res, w, eps, M, False)


def _combine(y, pos, scores, sscore, res, w, eps, M, quant):
    Mp, K = res.shape
    topk = scores.shape[1] + (1 if sscore is not None else 0)
    h = torch.empty_like(res)
    xq = torch.empty((Mp, K), dtype=torch.int8, device=res.device) if quant else None
    xs = torch.empty(Mp, dtype=torch.float32, device=res.device) if quant else None
    _lib.call("scmx_moe_combine", _lib.ptr(y), _lib.ptr(pos), _lib.ptr(scores), _lib.ptr(sscore), _lib.ptr(res),
              _lib.ptr(w) if quant else None, S._eps(eps) if quant else 0.0, _lib.ptr(h), _lib.ptr(xq), _lib.ptr(xs), M,
              Mp, K, topk, _lib.stream())
    return h, xq, xs
