"""Packed-weight containers and their on-disk form.

Mirrors the pieces of the reference's model integrations that sit between the quantizer and the kernels:
  PackedWeight            e2e/fused_qwen3.py:35-59     row-concatenated packed linears sharing an input
  load_packed             e2e/fused_qwen3.py:62-72     byte-shift cache (codes / shifts / wscale) -> this format
  save_cache, load_cache  e2e/fused_olmoe.py:123-129, e2e/pack_format.py:99-108
                          one safetensors file, keys "<linear>.codes" (uint32), "<linear>.bcodes" (uint8),
                          "<linear>.wscale" (float32) with <linear> = "layers.{i}.{path}" or
                          "layers.{i}.experts.{name}.{e}"
  pack_weights            e2e/fused_olmoe.py:98-128    quantize every matrix of a {key: weight} mapping (on the device)
  mxfp4_scales            e2e/fused_qwen38.py:319-334  E8M0 block scales that make the code words a standard MXFP4 tensor
The files are what the reference writes with mx.save_safetensors, so caches move between the two implementations."""
import numpy as np
import torch

from . import sc_format as F
from . import sc_kernels as S

SUFFIXES = ("codes", "bcodes", "wscale")


class PackedWeight:
    """Row-concatenated packed SC-MXFP4 weights of one or more linears sharing an input (e2e/fused_qwen3.py:35-59).

    parts: list of (codes uint32 [N*K/8], bcodes uint8 [N, K/(block*per_byte)], wscale f32 [N]) numpy arrays (or
    torch tensors); perm: optional permutation of the concatenated rows (gate/up interleaving for the SwiGLU
    epilogue).  resident=True keeps an INT8 copy, otherwise unpack() hands the GEMM a lazy handle and the weights
    are decoded per tile."""

    def __init__(self, parts, resident=False, perm=None, fmt=None, device="cuda"):
        self.fmt = fmt or F.DEFAULT
        parts = [tuple(_host(a) for a in p) for p in parts]
        self.splits = [p[2].shape[0] for p in parts]
        self.N = sum(self.splits)
        self.K = parts[0][0].size * 8 // parts[0][2].shape[0]
        for c, b, w in parts:
            if c.size * 8 != w.shape[0] * self.K or b.shape != (w.shape[0], self.K // (self.fmt.block * self.fmt.per_byte)):
                raise ValueError("parts of one PackedWeight must share K and the format")
        codes = np.concatenate([p[0].view(np.uint32).reshape(p[2].shape[0], -1) for p in parts])
        bcodes = np.concatenate([p[1] for p in parts])
        wscale = np.concatenate([p[2] for p in parts]).astype(np.float32)
        self.perm = perm
        if perm is not None:
            perm = np.asarray(perm)
            codes, bcodes, wscale = codes[perm], bcodes[perm], wscale[perm]
        self.codes, self.bcodes, self.wscale = F.to_device(codes.reshape(-1), bcodes, wscale, device)
        self.wq = S.unpack_i8(self.codes, self.bcodes, self.N, self.K, lazy=False, fmt=self.fmt) if resident else None

    def unpack(self, deps=()):
        if self.wq is not None:
            return self.wq
        return S.unpack_i8(self.codes, self.bcodes, self.N, self.K, fmt=self.fmt)

    def nbytes(self):
        return sum(t.numel() * t.element_size() for t in (self.codes, self.bcodes, self.wscale))


def _host(a):
    if isinstance(a, torch.Tensor):
        a = a.detach().cpu()
        return a.numpy().view(np.uint32) if a.dtype == torch.int32 else a.numpy()
    return np.asarray(a)


def save_cache(path, flat):
    """flat: {"<linear>.codes" | ".bcodes" | ".wscale": array} (numpy or torch) -> one safetensors file with the
    reference's dtypes (codes uint32, bcodes uint8, wscale float32)."""
    from safetensors.numpy import save_file
    out = {}
    for key, a in flat.items():
        a = _host(a)
        kind = key.rsplit(".", 1)[-1]
        if kind == "codes":
            a = np.ascontiguousarray(a).view(np.uint32).reshape(-1)
        elif kind in ("bcodes", "shifts"):
            a = np.ascontiguousarray(a, np.uint8)
        elif kind == "wscale":
            a = np.ascontiguousarray(a, np.float32)
        else:
            raise ValueError(f"unexpected key {key!r}: want .codes / .bcodes / .wscale (or .shifts)")
        out[key] = a
    save_file(out, path)


def load_cache(path):
    """safetensors cache -> {linear: (codes uint32, bcodes uint8, wscale float32)} numpy arrays."""
    from safetensors.numpy import load_file
    flat = load_file(path)
    out = {}
    for key in sorted(k[: -len(".codes")] for k in flat if k.endswith(".codes")):
        missing = [s for s in SUFFIXES if f"{key}.{s}" not in flat]
        if missing:
            raise KeyError(f"{path}: {key} lacks {missing}")
        out[key] = (flat[key + ".codes"].view(np.uint32).reshape(-1), flat[key + ".bcodes"], flat[key + ".wscale"])
    return out


def load_packed(cache_path, n_layers, fmt=None, groups=None):
    """From the byte-shift cache (keys .codes / .shifts / .wscale per linear) to 2-bit block codes, per linear
    (e2e/fused_qwen3.py:62-72).  groups: {name: [paths]} (default: the dense Qwen3 block)."""
    from safetensors.numpy import load_file
    fmt = fmt or F.DEFAULT
    groups = groups or GROUPS
    flat = load_file(cache_path)
    out = {}
    for i in range(n_layers):
        for g in groups.values():
            for p in g:
                key = f"layers.{i}.{p}"
                out[key] = F.from_shift_layout(flat[key + ".codes"].view(np.uint32), flat[key + ".shifts"],
                                               flat[key + ".wscale"], fmt)
    return out


GROUPS = {"qkv": ["self_attn.q_proj", "self_attn.k_proj", "self_attn.v_proj"], "o": ["self_attn.o_proj"],
          "gu": ["mlp.gate_proj", "mlp.up_proj"], "down": ["mlp.down_proj"]}   # e2e/fused_qwen3.py:31-32


def pack_weights(weights, fmt=None):
    """{linear: float weight [N, K] (torch, any device; float32 or bfloat16)} -> flat {linear.codes|bcodes|wscale}
    of numpy arrays, quantized on the GPU with the bit-exact SC-MXFP4 quantizer (the reference spreads this over 14
    host processes, e2e/fused_olmoe.py:102-128).  Expert stacks [E, N, K] become "<linear>.{e}" entries."""
    flat = {}
    for key, w in weights.items():
        w = w if isinstance(w, torch.Tensor) else torch.from_numpy(np.asarray(w, np.float32))
        mats = {key: w} if w.dim() == 2 else {f"{key}.{e}": w[e] for e in range(w.shape[0])}
        for k2, m in mats.items():
            codes, bc, ws, _ = F.quantize(m.cuda(), fmt, with_q=False)
            flat[k2 + ".codes"] = codes.cpu().numpy().view(np.uint32)
            flat[k2 + ".bcodes"] = bc.cpu().numpy()
            flat[k2 + ".wscale"] = ws.cpu().numpy()
    return flat


def mxfp4_scales(pw, fmt=None):
    """Packed SC-MXFP4 matrix (anything with .bcodes [N, K/128], .wscale [N], .K) -> uint8 E8M0 scales [N, K/32]:
    with them the code words are a standard MXFP4 tensor, E8M0 = log2(wscale) + 1 + shift + 127
    (e2e/fused_qwen38.py:319-334).  Host arithmetic on the small scale arrays."""
    fmt = fmt or getattr(pw, "fmt", None) or F.DEFAULT
    if fmt.block != 32 or tuple(fmt.mult) != (1, 2, 4, 8) or tuple(fmt.code_mag) != (0, 1, 2, 3, 4, 6, 8, 12):
        raise ValueError("only the 32-block power-of-two format is a standard MXFP4 tensor")
    bc, ws = _host(pw.bcodes), _host(pw.wscale).astype(np.float64)
    b = np.arange(pw.K // 32)
    shifts = (bc[:, b // fmt.per_byte] >> (fmt.bc_bits * (b % fmt.per_byte))) & ((1 << fmt.bc_bits) - 1)
    e = np.log2(ws)[:, None] + 1 + shifts
    ei = np.rint(e)
    if not np.array_equal(e, ei):
        raise ValueError("row scale is not a power of two")
    if ei.min() + 127 < 0 or ei.max() + 127 > 254:
        raise ValueError("exponent outside E8M0")
    return np.ascontiguousarray((ei + 127).astype(np.uint8))
