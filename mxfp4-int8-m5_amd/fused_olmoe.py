"""OLMoE (mixture of experts: 64 experts, top-8) prefill and batch-1 decode through the W4A8 kernels: the torch-ROCm
counterpart of e2e/fused_olmoe.py:130-298 (FusedOlmoe) and e2e/decode.py:102-165 (DecodeOlmoe).

Per transformer block (e2e/fused_olmoe.py:1-16):
  y = mm_epi(xq, Wq|Wk|Wv) -> q, k, v = qkv_fullnorm_y(y)        q/k RMSNorm over the full width
  rope, KV cache, attention                                        torch ops (MLX ops in the reference)
  h = mm_epi(act_quant(o), Wo, + h)                                residual add in the GEMM epilogue
  xq, xs, xn = rmsnorm_quant_n(h)                                  INT8 for the experts, bf16 for the router
  router: bf16 linear (torch), softmax + top-k (+ renorm) kernel   route
  route_sort; act = moe_mm(xq, gather=tok, Wg|Wu, SwiGLU)          token rows read through the sort, no xq[tok] copy
  y = moe_mm(act_quant(act), Wd); h, xq, xs = moe_combine(y, scores, + h) + next block's RMSNorm + INT8
Expert weights stay packed; the grouped kernel decodes each expert's weight tile in LDS."""
from dataclasses import dataclass

import numpy as np
import torch
import torch.nn.functional as TF

from . import sc_decode as G
from . import sc_format as F
from . import sc_kernels as S
from . import sc_moe
from .fused_qwen3 import BF, KVCache, rms_norm
from .sc_weights import PackedWeight

# the reference keeps these two in its fused_olmoe module (e2e/fused_olmoe.py:74-97); the kernels live in sc_moe here
moe_combine = sc_moe.moe_combine
moe_combine_split = sc_moe.moe_combine_split

ATTN = ["self_attn.q_proj", "self_attn.k_proj", "self_attn.v_proj", "self_attn.o_proj"]   # e2e/fused_olmoe.py:28
EXPERTS = ["gate_proj", "up_proj", "down_proj"]                                            # e2e/fused_olmoe.py:29


@dataclass
class OlmoeArgs:
    hidden_size: int = 2048
    intermediate_size: int = 1024
    num_hidden_layers: int = 16
    num_attention_heads: int = 16
    num_experts: int = 64
    num_experts_per_tok: int = 8
    norm_topk_prob: bool = False
    rms_norm_eps: float = 1e-5
    rope_theta: float = 1e4
    vocab_size: int = 50304
    tie_word_embeddings: bool = False

    @property
    def num_key_value_heads(self):
        return self.num_attention_heads

    @property
    def head_dim(self):
        return self.hidden_size // self.num_attention_heads


class FusedOlmoe:
    def __init__(self, args, params, flat, tile=None, two_pass=False, sort="count", fmt=None, device="cuda"):
        """params: Hugging Face names ("model.embed_tokens.weight", "model.norm.weight", "lm_head.weight", per layer
        "model.layers.{i}.input_layernorm.weight", ".post_attention_layernorm.weight", ".self_attn.q_norm.weight",
        ".self_attn.k_norm.weight", ".mlp.gate.weight").  flat: {"layers.{i}.{path}": (codes, bcodes, wscale)} for the
        attention linears and "layers.{i}.experts.{name}.{e}" for the experts (the reference's cache keys).
        tile: row tile of the grouped GEMM (64, 128 or 256; None: by the rows per expert of each call,
        sc_moe.row_tile); two_pass: unpack all experts to INT8 first
        (e2e/fused_olmoe.py:133-138); sort: "count" (route_sort kernel) or "argsort" (array ops)."""
        self.args, self.device, self.tile, self.two_pass, self.sort = args, device, tile, two_pass, sort
        self.fmt = fmt if fmt is not None else F.Format()
        self.eps = float(args.rms_norm_eps)
        a = args
        E, Fi = a.num_experts, a.intermediate_size
        dev = lambda k: params[k].to(device=device, dtype=BF).contiguous()   # noqa: E731
        self.embed, self.norm = dev("model.embed_tokens.weight"), dev("model.norm.weight")
        self.lm_head = self.embed if a.tie_word_embeddings else dev("lm_head.weight")
        perm = S.interleave_gate_up(Fi)
        host = lambda t: t.cpu().numpy() if torch.is_tensor(t) else np.asarray(t)   # noqa: E731
        self.layers = []
        for i in range(a.num_hidden_layers):
            p = f"model.layers.{i}."
            nw = {n: dev(p + n + ".weight") for n in ("input_layernorm", "post_attention_layernorm", "self_attn.q_norm",
                                                      "self_attn.k_norm", "mlp.gate")}
            part = lambda q: flat[f"layers.{i}.{q}"]   # noqa: E731
            ws = {"qkv": PackedWeight([part(q) for q in ATTN[:3]], fmt=self.fmt, device=device),
                  "o": PackedWeight([part(ATTN[3])], fmt=self.fmt, device=device)}
            gu, dn = [], []
            for e in range(E):
                g, u, d = (tuple(host(x) for x in part(f"experts.{n}.{e}")) for n in EXPERTS)
                gu.append((np.concatenate([g[0].view(np.uint32).reshape(Fi, -1), u[0].view(np.uint32).reshape(Fi, -1)])[perm]
                           .reshape(-1), np.concatenate([g[1], u[1]])[perm], np.concatenate([g[2], u[2]])[perm]))
                dn.append((d[0].view(np.uint32).reshape(-1), d[1], d[2]))
            stack = lambda xs: F.to_device(np.stack([x[0] for x in xs]), np.stack([x[1] for x in xs]),   # noqa: E731
                                           np.stack([x[2] for x in xs]), device)
            self.layers.append((nw, ws, {"gu": stack(gu), "down": stack(dn)}))
        self.record = None   # set to a list to collect every block's (inds, scores), as the reference's checks do
        half = a.head_dim // 2
        self.inv_freq = 1.0 / (a.rope_theta ** (torch.arange(half, device=device, dtype=torch.float32) / half))

    def weight_bytes(self):
        n = 0
        for _, ws, ex in self.layers:
            n += ws["qkv"].nbytes() + ws["o"].nbytes() + sum(t.numel() * t.element_size() for t in ex["gu"] + ex["down"])
        return n

    def make_cache(self, max_len=4096):
        return [KVCache(self.args, max_len, self.device) for _ in self.layers]

    def rope(self, x, offset):
        L = x.shape[1]
        ang = torch.arange(offset, offset + L, device=x.device, dtype=torch.float32)[:, None] * self.inv_freq[None]
        cos, sin = ang.cos()[None], ang.sin()[None]
        x1, x2 = x.float().chunk(2, -1)
        return torch.cat([x1 * cos - x2 * sin, x2 * cos + x1 * sin], -1).to(x.dtype)

    def _attention(self, c, q, k, v, L):
        off = c.offset
        q, k = self.rope(q, off), self.rope(k, off)
        k, v = c.update_and_fetch(k, v)
        if L == 1:
            return S.attn_decode(q, c.k, c.v, off + 1)
        if q.shape[-1] == 128:   # this library's causal attention (head dim 128 only; q is copied to token-major)
            return S.attn_prefill(q, c.k, c.v, off)
        if off == 0:
            o = TF.scaled_dot_product_attention(q[None], k[None], v[None], is_causal=True)
        else:
            pos = torch.arange(off, off + L, device=q.device)[:, None]
            o = TF.scaled_dot_product_attention(q[None], k[None], v[None],
                                                attn_mask=torch.arange(off + L, device=q.device)[None] <= pos)
        return o[0].transpose(0, 1).reshape(L, -1).contiguous()

    def route(self, nw, xn, M):
        """mlx_lm's OlmoeSparseMoeBlock routing on the bf16 normalized rows (e2e/fused_olmoe.py:183-192): bf16 router
        linear (an array op, as in the reference), then one kernel for the float32 softmax, the k largest probabilities
        and the optional renormalisation."""
        logits = xn[:M] @ nw["mlp.gate"].T
        return sc_moe.route(logits, self.args.num_experts_per_tok, renorm=self.args.norm_topk_prob)

    def _experts(self, xq, xs, inds, scores, h, nn, ex, L, quant=True):
        a = self.args
        E, F2, D = a.num_experts, 2 * a.intermediate_size, a.hidden_size
        R = L * a.num_experts_per_tok
        tm = self.tile or sc_moe.row_tile(R, E)
        if self.sort == "count":
            pos, tok, _, off, tstart, maxt = sc_moe.route_sort(inds, E, tm)
        else:   # array ops, as mlx_lm's _gather_sort (e2e/fused_olmoe.py:225-231)
            flat_i = inds.flatten()
            order = torch.argsort(flat_i.to(torch.int64), stable=True)
            pos = torch.argsort(order).to(torch.int32)
            off, tstart, maxt = sc_moe.segments(flat_i[order].to(torch.int32), E, tm)
            tok = torch.cat([(order // a.num_experts_per_tok).to(torch.int32),
                             torch.zeros(tm, dtype=torch.int32, device=inds.device)])
        cg, bg, sg = ex["gu"]
        cd, bd, sd = ex["down"]
        t = (tm, 64, 4)
        if self.two_pass:
            act = sc_moe.moe_mm_i8(xq, R, sc_moe.unpack_experts(cg, bg, F2, D), sg, off, tstart, maxt, F2, 3, xs, tile=t,
                                   gather=tok)
        else:
            act = sc_moe.moe_mm(xq, R, cg, bg, sg, off, tstart, maxt, F2, 3, xs, tile=t, gather=tok, fmt=self.fmt)
        xq2, xs2 = S.act_quant(act, R)
        if self.two_pass:
            yd = sc_moe.moe_mm_i8(xq2, R, sc_moe.unpack_experts(cd, bd, D, F2 // 2), sd, off, tstart, maxt, D, 1, xs2, tile=t)
        else:
            yd = sc_moe.moe_mm(xq2, R, cd, bd, sd, off, tstart, maxt, D, 1, xs2, tile=t, fmt=self.fmt)
        return sc_moe.moe_combine(yd, pos, scores, h, nn, self.eps, L, quant=quant)

    def hidden(self, ids, cache=None):
        """Final normed hidden states [L, D] for prompt ids [L]."""
        S.set_format(self.fmt)
        a = self.args
        H, d = a.num_attention_heads, a.head_dim
        cache = cache if cache is not None else self.make_cache(max(4096, ids.numel()))
        h = self.embed[ids.reshape(-1)]
        L = h.shape[0]
        Mp = S.pad_rows(L)
        h = (TF.pad(h, (0, 0, 0, Mp - L)) if Mp != L else h).contiguous()
        nl = len(self.layers)
        xq, xs = S.rmsnorm_quant(h, self.layers[0][0]["input_layernorm"], self.eps, Mp)
        for i, (nw, ws, ex) in enumerate(self.layers):
            y = S.mm_epi(xq, ws["qkv"].unpack(), xs, ws["qkv"].wscale, 1)
            q, k, v = S.qkv_fullnorm_y(y, nw["self_attn.q_norm"], nw["self_attn.k_norm"], self.eps, L, H, d)
            o = self._attention(cache[i], q, k, v, L)
            wo = ws["o"].unpack()   # a prefill-sized GEMM on packed weights reads its activations in 32x32 blocks
            blocked = isinstance(wo, S.PackedWq) and S.prefers_blocked(Mp, ws["o"].N, ws["o"].K)
            xq, xs = S.act_quant_blocked(o, Mp) if blocked else S.act_quant(o, Mp)
            h = S.mm_epi(xq, wo, xs, ws["o"].wscale, 2, res=h)
            xq, xs, xn = S.rmsnorm_quant_n(h, nw["post_attention_layernorm"], self.eps)
            inds, scores = self.route(nw, xn, L)
            if self.record is not None:
                self.record.append((inds, scores))
            nn = self.layers[i + 1][0]["input_layernorm"] if i + 1 < nl else self.norm
            h, xq, xs = self._experts(xq, xs, inds, scores, h, nn, ex, L)
        return rms_norm(h[:L], self.norm, self.eps)

    def logits(self, h):
        return h @ self.lm_head.T

    def __call__(self, ids, cache=None):
        return self.logits(self.hidden(ids, cache))


class DecodeOlmoe:
    """Batch-1 decode from a FusedOlmoe (e2e/decode.py:102-165): GEMVs on the packed weights; the expert GEMVs gather
    the top-k experts' rows themselves (eidx), gate|up with the SwiGLU epilogue over 8 slots sharing the input row,
    down with one input row per slot; combine as in the prefill path."""

    def __init__(self, fused, fuse_prologue=False, head=True):
        self.f, self.args, self.fuse, self.head = fused, fused.args, fuse_prologue, head
        self.pos = torch.arange(fused.args.num_experts_per_tok, dtype=torch.int32, device=fused.device)

    def step(self, tok, cache):
        f, a = self.f, self.args
        S.set_format(f.fmt)
        H, d, D, k = a.num_attention_heads, a.head_dim, a.hidden_size, a.num_experts_per_tok
        F2 = 2 * a.intermediate_size
        fp = self.fuse is True
        h = f.embed[tok.reshape(-1)[:1]].contiguous()
        for i, (nw, ws, ex) in enumerate(f.layers):
            w = ws["qkv"]
            if fp:
                y = G.gemv(h, w.codes, w.bcodes, None, w.wscale, 3 * H * d, 1, pro=2, nw=nw["input_layernorm"], eps=f.eps,
                           fmt=f.fmt)
            else:
                xq, xs = S.rmsnorm_quant(h, nw["input_layernorm"], f.eps, 1)
                y = G.gemv(xq, w.codes, w.bcodes, xs, w.wscale, 3 * H * d, 1, fmt=f.fmt)
            q, kk, v = S.qkv_fullnorm_y(y[None], nw["self_attn.q_norm"], nw["self_attn.k_norm"], f.eps, 1, H, d)
            o = f._attention(cache[i], q, kk, v, 1)
            wo = ws["o"]
            if self.fuse:
                h = G.gemv(o, wo.codes, wo.bcodes, None, wo.wscale, D, 2, res=h, pro=1, fmt=f.fmt)[None]
            else:
                xq, xs = S.act_quant(o, 1)
                h = G.gemv(xq, wo.codes, wo.bcodes, xs, wo.wscale, D, 2, res=h, fmt=f.fmt)[None]
            xq, xs, xn = S.rmsnorm_quant_n(h, nw["post_attention_layernorm"], f.eps, 1)
            inds, scores = f.route(nw, xn, 1)
            e = inds.reshape(-1)
            cg, bg, sg = ex["gu"]
            cd, bd, sd = ex["down"]
            act = G.gemv(xq, cg, bg, xs, sg, F2, 3, eidx=e, xstride=0, fmt=f.fmt)                   # [k, F]
            if fp:
                yd = G.gemv(act, cd, bd, None, sd, D, 1, eidx=e, xstride=1, pro=1, fmt=f.fmt)        # [k, D]
            else:
                xq2, xs2 = S.act_quant(act, k)
                yd = G.gemv(xq2, cd, bd, xs2, sd, D, 1, eidx=e, xstride=1, fmt=f.fmt)
            h = sc_moe.moe_combine(yd, self.pos, scores, h, nw["post_attention_layernorm"], f.eps, 1, quant=False)[0]
        hn = rms_norm(h, f.norm, f.eps)
        return f.logits(hn) if self.head else hn
