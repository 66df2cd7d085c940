"""Dense prefill call surface: the function names, argument order and defaults of the reference's e2e/sc_kernels.py,
on torch (ROCm) tensors, backed by the HIP kernels of libscmx.so through its C ABI.

Conventions kept from the reference (e2e/sc_kernels.py:15-17): kernels take M rows and write Mp >= M rows, rows >= M
are zero; `deps` is accepted and ignored (it only ordered MLX's lazy graph — HIP streams are already ordered);
`tile` / `nt` are accepted as hints and never change a result.  `eps` may be a float or a 1-element tensor.

Difference by design: `unpack_i8` may return a `PackedWq` handle instead of an INT8 tensor (FUSE_UNPACK, default on).
`mm_epi` / `mm_i8_i32` given that handle run the GEMM whose workgroups unpack their weight tile in LDS, so the INT8
weights are never written to memory; `handle.materialize()` (or lazy=False) gives the reference's INT8 tensor.
"""
import numpy as np
import torch

from . import _lib
from . import sc_format as F

TM, TN, NSG, GROUP_M = 128, 64, 4, 8     # the reference's default tile (kept for pad_rows and as accepted hints)
FUSE_UNPACK = True


def set_format(fmt):
    """Switch the default weight format of every wrapper (the C ABI itself takes the format per call)."""
    F.DEFAULT = fmt


def pad_rows(M):
    return -(-M // TM) * TM


def _eps(eps):
    return float(eps) if not torch.is_tensor(eps) else float(eps.reshape(-1)[0].item())


def _check_dtype(dtype):
    if dtype not in (torch.bfloat16, None):
        raise ValueError("the kernels emit bfloat16 (the reference's model dtype)")


class PackedWq:
    """Packed weights standing in for the INT8 tensor unpack_i8 would produce."""

    def __init__(self, codes, bcodes, N, K, fmt, wscale=None):
        self.codes, self.bcodes, self.N, self.K, self.fmt = codes, bcodes, N, K, fmt
        self.wscale = wscale   # a standard MXFP4 tensor read in place decodes with its row scales (F.MXFP4)
        self.shape, self.dtype, self.device = (N, K), torch.int8, codes.device

    def materialize(self):
        return unpack_i8(self.codes, self.bcodes, self.N, self.K, lazy=False, fmt=self.fmt)

    def __getitem__(self, idx):          # row selection / permutation, as callers do on the INT8 tensor
        return self.materialize()[idx]

    def cpu(self):
        return self.materialize().cpu()


def unpack_i8(codes, bcodes, N, K, deps=(), lazy=None, fmt=None, wscale=None):
    """Packed codes (flat, 4-byte ints) + block codes uint8 [N, ..] -> INT8 [N, K].  fmt=F.MXFP4 (E8M0 bytes as block
    codes) exists as the lazy handle only and takes the row scales along (F.mxfp4_row_scales)."""
    fmt = fmt or F.DEFAULT
    if fmt.e8m0 and wscale is None:
        raise ValueError("the MXFP4 form decodes with its row scales: pass wscale=sc_format.mxfp4_row_scales(e8m0)")
    if FUSE_UNPACK if lazy is None else lazy:
        return PackedWq(codes, bcodes, N, K, fmt, wscale)
    assert codes.numel() * codes.element_size() == N * K // 2, "codes must hold N*K/2 bytes"
    wq = torch.empty((N, K), dtype=torch.int8, device=codes.device)
    _lib.call("scmx_unpack_i8", fmt.c_struct(), _lib.ptr(codes), _lib.ptr(bcodes), _lib.ptr(wq), N, K, _lib.stream())
    return wq


def act_quant(x, Mp=None, nt=256, deps=()):
    """Per-token symmetric INT8: x bf16 [M, K] -> (xq int8 [Mp, K], xscale f32 [Mp]); rows >= M zero."""
    M, K = x.shape
    Mp = Mp or pad_rows(M)
    assert x.dtype == torch.bfloat16
    xq = torch.empty((Mp, K), dtype=torch.int8, device=x.device)
    xs = torch.empty(Mp, dtype=torch.float32, device=x.device)
    _lib.call("scmx_act_quant", _lib.ptr(x), _lib.ptr(xq), _lib.ptr(xs), M, Mp, K, _lib.stream())
    return xq, xs


def rot_signs(K):
    """The sign vector of the block rotation for input width K (one per width, so q/k/v and gate/up share a rotated
    input); e2e/sc_kernels.py:566-569."""
    return torch.from_numpy(np.random.default_rng(0).choice([-1.0, 1.0], size=K).astype(np.float32)).cuda()


def rot_quant(x, signs, Mp=None, nt=512, deps=()):
    """x bf16 [M, K] -> (xq int8 [Mp, K], xscale f32 [Mp]): randomized Hadamard rotation of each 32-wide block, then
    per-token INT8 (e2e/sc_kernels.py:571-582)."""
    M, K = x.shape
    Mp = Mp or pad_rows(M)
    assert x.dtype == torch.bfloat16 and signs.dtype == torch.float32 and signs.numel() == K
    xq = torch.empty((Mp, K), dtype=torch.int8, device=x.device)
    xs = torch.empty(Mp, dtype=torch.float32, device=x.device)
    _lib.call("scmx_rot_quant", _lib.ptr(x), _lib.ptr(signs), _lib.ptr(xq), _lib.ptr(xs), M, Mp, K, _lib.stream())
    return xq, xs


def _gemm(xq, wq, xscale, wscale, epi, res):
    (M, K), N = xq.shape, wq.shape[0]
    assert xq.dtype == torch.int8 and wq.shape[1] == K
    if epi == 0:
        out = torch.empty((M, N), dtype=torch.int32, device=xq.device)
    else:
        out = torch.empty((M, N // 2 if epi == 3 else N), dtype=torch.bfloat16, device=xq.device)
    if epi == 2:
        assert res is not None and tuple(res.shape) == (M, N) and res.dtype == torch.bfloat16
    r = _lib.ptr(res) if epi == 2 else None
    if isinstance(xq, BlockedXq):
        if not isinstance(wq, PackedWq):
            raise ValueError("blocked activations multiply packed weights (unpack_i8's lazy handle)")
        _lib.call("scmx_mm_w4a8_blocked", wq.fmt.c_struct(), _lib.ptr(xq.data), _lib.ptr(xscale), _lib.ptr(wq.codes),
                  _lib.ptr(wq.bcodes), _lib.ptr(wscale if wscale is not None else wq.wscale), r, _lib.ptr(out), epi, M, N,
                  K, _lib.stream())
    elif isinstance(wq, PackedWq):
        _lib.call("scmx_mm_w4a8", wq.fmt.c_struct(), _lib.ptr(xq), _lib.ptr(xscale), _lib.ptr(wq.codes),
                  _lib.ptr(wq.bcodes), _lib.ptr(wscale if wscale is not None else wq.wscale), r, _lib.ptr(out), epi, M, N,
                  K, _lib.stream())
    else:
        assert wq.dtype == torch.int8
        _lib.call("scmx_mm_epi", _lib.ptr(xq), _lib.ptr(wq), _lib.ptr(xscale), _lib.ptr(wscale), r, _lib.ptr(out), epi,
                  M, N, K, _lib.stream())
    return out


def mm_i8_i32(xq, wq, deps=(), tile=None):
    """INT8 [M, K] x INT8 [N, K]^T -> INT32 [M, N] (wq: INT8 tensor or PackedWq)."""
    return _gemm(xq, wq, None, None, 0, None)


def mm_epi(xq, wq, xscale, wscale, epi, dtype=torch.bfloat16, res=None, deps=(), tile=None):
    """INT8 GEMM + in-register epilogue (EPI 1: scaled bf16, 2: + residual, 3: swiglu of interleaved gate/up)."""
    _check_dtype(dtype)
    assert epi in (1, 2, 3)
    return _gemm(xq, wq, xscale, wscale, epi, res)


class BlockedXq:
    """INT8 activations in the blocked layout (act_quant_blocked): what mm_epi / mm_i8_i32 take in place of the [Mp, K]
    tensor when the weights are packed (PackedWq)."""

    def __init__(self, data, M, K):
        self.data, self.shape, self.dtype, self.device = data, (M, K), torch.int8, data.device

    def rows(self):
        """The [Mp, K] tensor act_quant returns (a copy)."""
        Mp, K = self.data.numel() // self.shape[1], self.shape[1]
        return self.data.view(Mp // 32, K // 32, 2, 32, 16).permute(0, 3, 1, 2, 4).reshape(Mp, K)


def act_quant_blocked(x, Mp=None):
    """act_quant for prefill-sized GEMMs on packed weights: the same codes and scales with xq in 32 x 32 blocks in the
    order the MFMA takes them, so that the large GEMM tiles load activation fragments straight from memory
    (scmx_act_quant_blocked / scmx_mm_w4a8_blocked).  -> (BlockedXq, xscale f32 [Mp]), Mp a multiple of 32."""
    M, K = x.shape
    Mp = Mp or pad_rows(M)
    assert x.dtype == torch.bfloat16 and Mp % 32 == 0
    xq = torch.empty(Mp * K, dtype=torch.int8, device=x.device)
    xs = torch.empty(Mp, dtype=torch.float32, device=x.device)
    _lib.call("scmx_act_quant_blocked", _lib.ptr(x), _lib.ptr(xq), _lib.ptr(xs), M, Mp, K, _lib.stream())
    return BlockedXq(xq, Mp, K), xs   # Mp rows like act_quant's tensor: the padding rows are zeros


def linear_w4a8_workspace(M, K):
    """Bytes of workspace linear_w4a8 needs for M rows of K (the INT8 activations, then their scales)."""
    return int(_lib.load().scmx_linear_w4a8_workspace(M, K))


def linear_w4a8(x, codes, bcodes, wscale, N, epi=1, res=None, fmt=None, workspace=None):
    """One call for a whole W4A8 linear on bf16 activations [M, K]: the activation-quantization prologue and the
    fused-unpack GEMM are enqueued by a single C entry point (scmx_linear_w4a8).  Returns bf16 [M, N or N/2]."""
    fmt = fmt or F.DEFAULT
    M, K = x.shape
    assert x.dtype == torch.bfloat16 and epi in (1, 2, 3)
    need = _lib.load().scmx_linear_w4a8_workspace(M, K)
    if workspace is None or workspace.numel() * workspace.element_size() < need:
        workspace = torch.empty(need, dtype=torch.uint8, device=x.device)
    out = torch.empty((M, N // 2 if epi == 3 else N), dtype=torch.bfloat16, device=x.device)
    _lib.call("scmx_linear_w4a8", fmt.c_struct(), _lib.ptr(x), _lib.ptr(codes), _lib.ptr(bcodes), _lib.ptr(wscale),
              _lib.ptr(res) if epi == 2 else None, _lib.ptr(out), epi, M, N, K, _lib.ptr(workspace),
              workspace.numel() * workspace.element_size(), _lib.stream())
    return out


def interleave_gate_up(F_):
    """Row permutation of [gate (F rows); up (F rows)] into groups g_2p, g_2p+1, u_2p, u_2p+1 for EPI 3."""
    p = np.arange(F_ // 2)
    return np.stack([2 * p, 2 * p + 1, F_ + 2 * p, F_ + 2 * p + 1], 1).reshape(-1)


def _rms(x, w, eps, Mp, want_xn, blocked=False):
    M, K = x.shape
    Mp = Mp or pad_rows(M)
    assert x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16
    blocked = blocked and Mp % 32 == 0 and K % 512 == 0 and K <= 4096
    xq = torch.empty((Mp, K), dtype=torch.int8, device=x.device)
    xs = torch.empty(Mp, dtype=torch.float32, device=x.device)
    xn = torch.empty((Mp, K), dtype=torch.bfloat16, device=x.device) if want_xn else None
    _lib.call("scmx_rmsnorm_quant_blocked" if blocked else "scmx_rmsnorm_quant", _lib.ptr(x), _lib.ptr(w), _eps(eps),
              _lib.ptr(xq), _lib.ptr(xs), _lib.ptr(xn), M, Mp, K, _lib.stream())
    if blocked:
        xq = BlockedXq(xq.reshape(-1), Mp, K)   # Mp rows like the tensor it stands for: the padding rows are zeros
    return (xq, xs, xn) if want_xn else (xq, xs)


def rmsnorm_quant(x, w, eps, Mp=None, deps=(), blocked=False):
    """x [M, K] -> (xq int8 [Mp, K], xscale f32 [Mp]) of rms_norm(x, w, eps).  blocked: xq as a BlockedXq (the layout of
    act_quant_blocked) where the shape allows it (Mp % 32 == 0, K % 512 == 0, K <= 4096), by rows otherwise."""
    return _rms(x, w, eps, Mp, False, blocked)


def rmsnorm_quant_n(x, w, eps, Mp=None, deps=(), blocked=False):
    """rmsnorm_quant that also returns the normalized bf16 rows: (xq, xscale, xn [Mp, K])."""
    return _rms(x, w, eps, Mp, True, blocked)


def prefers_blocked(M, N, K):
    """Whether a dense [M, K] x [N, K]^T problem on packed weights runs faster from blocked activations."""
    return bool(_lib.load().scmx_mm_w4a8_prefers_blocked(M, N, K))


def res_norm_quant(acc, xscale, wscale, res, w, eps, deps=()):
    """h = res + bf16(acc * xscale * wscale); returns (h [Mp, K], xq, xscale') of rms_norm(h)."""
    Mp, K = acc.shape
    assert tuple(res.shape) == (Mp, K) and acc.dtype == torch.int32
    h = torch.empty_like(res)
    xq = torch.empty((Mp, K), dtype=torch.int8, device=acc.device)
    xs = torch.empty(Mp, dtype=torch.float32, device=acc.device)
    _lib.call("scmx_res_norm_quant", _lib.ptr(acc), _lib.ptr(xscale), _lib.ptr(wscale), _lib.ptr(res), _lib.ptr(w),
              _eps(eps), _lib.ptr(h), _lib.ptr(xq), _lib.ptr(xs), Mp, K, _lib.stream())
    return h, xq, xs


def res_epilogue(acc, xscale, wscale, res, deps=()):
    """h = res + bf16(acc * xscale * wscale)."""
    Mp, N = acc.shape
    h = torch.empty_like(res)
    _lib.call("scmx_res_norm_quant", _lib.ptr(acc), _lib.ptr(xscale), _lib.ptr(wscale), _lib.ptr(res), None, 0.0,
              _lib.ptr(h), None, None, Mp, N, _lib.stream())
    return h


def swiglu_quant(acc, xscale, wscale, dtype=torch.bfloat16, nt=512, deps=()):
    """acc [Mp, 2F] (gate | up) -> (xq int8 [Mp, F], xscale f32 [Mp]) of swiglu(bf16 gate, bf16 up)."""
    _check_dtype(dtype)
    Mp, F2 = acc.shape
    Fh = F2 // 2
    xq = torch.empty((Mp, Fh), dtype=torch.int8, device=acc.device)
    xs = torch.empty(Mp, dtype=torch.float32, device=acc.device)
    _lib.call("scmx_swiglu_quant", _lib.ptr(acc), _lib.ptr(xscale), _lib.ptr(wscale), _lib.ptr(xq), _lib.ptr(xs), Mp, Fh,
              _lib.stream())
    return xq, xs


def _headnorm(acc, xscale, wscale, y, qn, kn, eps, L, hq, hk, d, dev):
    q = torch.empty((hq, L, d), dtype=torch.bfloat16, device=dev)
    k = torch.empty((hk, L, d), dtype=torch.bfloat16, device=dev)
    v = torch.empty((hk, L, d), dtype=torch.bfloat16, device=dev)
    _lib.call("scmx_qkv_headnorm", _lib.ptr(acc), _lib.ptr(xscale), _lib.ptr(wscale), _lib.ptr(y), _lib.ptr(qn),
              _lib.ptr(kn), _eps(eps), _lib.ptr(q), _lib.ptr(k), _lib.ptr(v), L, hq, hk, d, _lib.stream())
    return q, k, v


def qkv_epilogue_headnorm(acc, xscale, wscale, qn, kn, eps, L, hq, hk, d, dtype=torch.bfloat16, deps=()):
    """Qwen3: acc [Mp, (hq + 2 hk) d] -> q [hq, L, d], k [hk, L, d], v [hk, L, d] (q/k per-head RMSNorm)."""
    _check_dtype(dtype)
    return _headnorm(acc, xscale, wscale, None, qn, kn, eps, L, hq, hk, d, acc.device)


def qkv_headnorm_y(y, qn, kn, eps, L, hq, hk, d, deps=()):
    """Qwen3: bf16 y [Mp, (hq + 2 hk) d] -> q, k, v head-major with per-head RMSNorm of q and k."""
    return _headnorm(None, None, None, y, qn, kn, eps, L, hq, hk, d, y.device)


def qkv_headnorm_rope(y, qn, kn, eps, L, hq, hk, d, kcache, vcache, pos, inv_freq, acc=None, xscale=None, wscale=None,
                      token_major=False):
    """qkv_headnorm_y (or, with acc / xscale / wscale, qkv_epilogue_headnorm) fused with the rotary embedding of q
    and k and the KV-cache append: returns q [hq, L, d]; k and v go to rows pos..pos+L-1 of kcache / vcache
    [hk, rows, d].  pos: int, or an int64 device tensor (for graph replay).  token_major=True stores q as [L, hq, d]
    and returns the [hq, L, d] view of it: an attention output that inherits this layout is [L, hq * d] without a
    transposing copy."""
    src = y if y is not None else acc
    q = torch.empty((L, hq, d) if token_major else (hq, L, d), dtype=torch.bfloat16, device=src.device)
    assert kcache.shape == vcache.shape and kcache.shape[0] == hk and kcache.shape[2] == d
    assert kcache.dtype == torch.bfloat16 and inv_freq.dtype == torch.float32 and inv_freq.numel() == d // 2
    dev_pos = pos if torch.is_tensor(pos) else None
    assert dev_pos is None or dev_pos.dtype == torch.int64
    _lib.call("scmx_qkv_headnorm_rope", _lib.ptr(acc), _lib.ptr(xscale), _lib.ptr(wscale), _lib.ptr(y), _lib.ptr(qn),
              _lib.ptr(kn), _eps(eps), _lib.ptr(q), _lib.ptr(kcache), _lib.ptr(vcache), L, hq, hk, d, _lib.ptr(inv_freq),
              _lib.ptr(dev_pos), 0 if dev_pos is not None else int(pos), kcache.shape[1], int(token_major), _lib.stream())
    return q.transpose(0, 1) if token_major else q


def attn_splits(rows):
    """Row ranges for the decode attention over up to `rows` cache rows: one workgroup per head reads a short context
    fastest, longer ones are cut into 8 ranges, beyond 8192 rows into 16 (measured: 8.6 / 10.2 / 16.3 / 34 us at
    1024 / 2048 / 4096 / 16000 rows against 23 / 43 / 86 / 354 us unsplit).  A split launch still serves contexts of
    up to 512 rows with one workgroup per head (decided on the device), so a graph captured for a long cache does not
    pay for the split while the context is short."""
    return 1 if rows <= 1024 else 8 if rows <= 8192 else 16


def _split_workspace(splits, hq, d, device):
    return torch.empty(splits * hq * (d + 2), dtype=torch.float32, device=device) if splits > 1 else None


def attn_decode(q, kcache, vcache, n, scale=None, splits=None):
    """Single-token attention: q bf16 [hq, 1, d] (or [hq, d]) against caches [hk, rows, d] whose first n rows are valid
    (n: int, or an int64 device tensor holding the position n - 1, for graph replay) -> bf16 [1, hq * d].
    splits: row ranges per head (default: by n, or by the cache size when n lives on the device)."""
    hq, d = q.shape[0], q.shape[-1]
    hk, rows, _ = kcache.shape
    out = torch.empty((1, hq * d), dtype=torch.bfloat16, device=q.device)
    dev_pos = n if torch.is_tensor(n) else None
    if splits is None:
        splits = attn_splits(rows if dev_pos is not None else int(n))
    work = _split_workspace(splits, hq, d, q.device)
    _lib.call("scmx_attn_decode", _lib.ptr(q), _lib.ptr(kcache), _lib.ptr(vcache), _lib.ptr(dev_pos),
              0 if dev_pos is not None else int(n), _lib.ptr(out), hq, hk, d, rows,
              float(scale if scale is not None else d ** -0.5), _lib.ptr(work), splits, _lib.stream())
    return out


def attn_prefill(q, kcache, vcache, off, scale=None):
    """Causal attention of L new tokens: q bf16 [hq, L, d], best as the view of [L, hq, d] storage that
    qkv_headnorm_rope returns with token_major=True (any other layout is copied into that one), caches [hk, rows, d]
    whose rows off .. off+L-1 hold the new tokens' keys and values -> bf16 [L, hq * d].  Head dim 128."""
    q = q.transpose(0, 1).contiguous()   # [L, hq, d] storage; no copy when q already is a view of it
    L, hq, d = q.shape
    hk, rows, _ = kcache.shape
    assert q.dtype == torch.bfloat16 and kcache.dtype == torch.bfloat16 and kcache.shape == vcache.shape
    out = torch.empty((L, hq * d), dtype=torch.bfloat16, device=q.device)
    _lib.call("scmx_attn_prefill", _lib.ptr(q), _lib.ptr(kcache), _lib.ptr(vcache), _lib.ptr(out), L, int(off), hq, hk, d,
              rows, float(scale if scale is not None else d ** -0.5), _lib.stream())
    return out


def attn_decode_qkv(y, qn, kn, eps, hq, hk, d, kcache, vcache, pos, inv_freq, scale=None, splits=None):
    """qkv_headnorm_rope at L = 1 followed by attn_decode, in one launch and with the same bits: y bf16
    [1, (hq + 2 hk) d] -> bf16 [1, hq * d]; the token's k and v land in row pos of the caches.  pos: int, or an int64
    device tensor (for graph replay)."""
    assert kcache.shape == vcache.shape and kcache.shape[0] == hk and kcache.shape[2] == d
    assert y.dtype == torch.bfloat16 and y.numel() == (hq + 2 * hk) * d and kcache.dtype == torch.bfloat16
    assert inv_freq.dtype == torch.float32 and inv_freq.numel() == d // 2
    out = torch.empty((1, hq * d), dtype=torch.bfloat16, device=y.device)
    dev_pos = pos if torch.is_tensor(pos) else None
    assert dev_pos is None or dev_pos.dtype == torch.int64
    if splits is None:
        splits = attn_splits(kcache.shape[1] if dev_pos is not None else int(pos) + 1)
    work = _split_workspace(splits, hq, d, y.device)
    _lib.call("scmx_attn_decode_qkv", _lib.ptr(y), _lib.ptr(qn), _lib.ptr(kn), _eps(eps), _lib.ptr(inv_freq),
              _lib.ptr(dev_pos), 0 if dev_pos is not None else int(pos), _lib.ptr(kcache), _lib.ptr(vcache), _lib.ptr(out),
              hq, hk, d, kcache.shape[1], float(scale if scale is not None else d ** -0.5), _lib.ptr(work), splits,
              _lib.stream())
    return out


def qkv_fullnorm_y(y, qn, kn, eps, L, h, d, deps=()):
    """OLMoE: bf16 y [Mp, 3 h d] -> q, k, v [h, L, d] with RMSNorm over the full h*d-wide q and k."""
    q, k, v = (torch.empty((h, L, d), dtype=torch.bfloat16, device=y.device) for _ in range(3))
    _lib.call("scmx_qkv_fullnorm", _lib.ptr(y), _lib.ptr(qn), _lib.ptr(kn), _eps(eps), _lib.ptr(q), _lib.ptr(k),
              _lib.ptr(v), L, h, d, _lib.stream())
    return q, k, v
