"""Qwen3 (dense) prefill and batch-1 decode driven through the W4A8 kernels: the torch-ROCm counterpart of the
reference's model integrations e2e/fused_qwen3.py:82-301 (FusedQwen3) and e2e/decode.py:29-99 (DecodeQwen3).

Every linear of a block runs as SC-MXFP4 W4A8 (per-token INT8 activations, exact integer accumulation, scaling /
residual / SwiGLU epilogues); prefill attention is torch's scaled-dot-product attention (an MLX op in the reference); RoPE and
the KV-cache append, array ops in the reference, are fused into the q/k/v norm kernel, and the single-token attention
of the decode step is a kernel of this library that reads the position from device memory.  Weights arrive in Hugging Face layout: a dict of the non-linear parameters plus the packed linears under
the reference's cache keys "layers.{i}.{path}" (sc_weights.load_cache / pack_weights).

epilogue="gemm": scales, residual adds and SwiGLU in the GEMM's registers (bf16 out), e2e/fused_qwen3.py:224-255.
epilogue="row":  INT32 GEMM out, then the row kernels res_norm_quant / swiglu_quant / qkv_epilogue_headnorm,
                 e2e/fused_qwen3.py:257-308.
The decode step's fixed-shape halves can be captured in HIP graphs (graphs=True), which is what mx.compile does for
the reference (e2e/decode.py:30-33): one graph launch replaces about ten kernel launches per layer."""
import json
import os
from dataclasses import dataclass, fields

import torch
import torch.nn.functional as TF

from . import sc_decode as G
from . import sc_format as F
from . import sc_kernels as S
from .sc_weights import GROUPS, PackedWeight, pack_weights

BF = torch.bfloat16


@dataclass
class Qwen3Args:
    hidden_size: int = 2048
    intermediate_size: int = 6144
    num_hidden_layers: int = 28
    num_attention_heads: int = 16
    num_key_value_heads: int = 8
    head_dim: int = 128
    rms_norm_eps: float = 1e-6
    rope_theta: float = 1e6
    vocab_size: int = 151936
    tie_word_embeddings: bool = True


class KVCache:
    """Per-layer keys / values [heads, max_len, d] with a write offset (mlx_lm's KVCache.update_and_fetch)."""

    def __init__(self, args, max_len, device="cuda"):
        shape = (args.num_key_value_heads, max_len, args.head_dim)
        self.k = torch.zeros(shape, dtype=BF, device=device)
        self.v = torch.zeros(shape, dtype=BF, device=device)
        self.offset = 0

    def update_and_fetch(self, k, v):
        n = k.shape[1]
        if self.offset + n > self.k.shape[1]:
            raise ValueError("KV cache is full")
        self.k[:, self.offset:self.offset + n] = k
        self.v[:, self.offset:self.offset + n] = v
        self.offset += n
        return self.k[:, :self.offset], self.v[:, :self.offset]


def rms_norm(x, w, eps):
    v = x.float()
    return (v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps)).to(x.dtype) * w


class FusedQwen3:
    def __init__(self, args, params, packed, resident=False, epilogue="gemm", fmt=None, device="cuda"):
        """params: "model.embed_tokens.weight", "model.norm.weight", per layer "model.layers.{i}.input_layernorm.weight",
        ".post_attention_layernorm.weight", ".self_attn.q_norm.weight", ".self_attn.k_norm.weight" (+ "lm_head.weight"
        when the embeddings are not tied).  packed: {"layers.{i}.{path}": (codes, bcodes, wscale)}."""
        assert epilogue in ("gemm", "row")
        self.args, self.epilogue, self.device = args, epilogue, device
        self.fmt = fmt if fmt is not None else F.Format()
        self.eps = float(args.rms_norm_eps)
        dev = lambda k: params[k].to(device=device, dtype=BF).contiguous()   # noqa: E731
        self.embed = dev("model.embed_tokens.weight")
        self.norm = dev("model.norm.weight")
        self.lm_head = self.embed if args.tie_word_embeddings else dev("lm_head.weight")
        perm = {"gu": S.interleave_gate_up(args.intermediate_size)} if epilogue == "gemm" else {}
        self.layers = []
        for i in range(args.num_hidden_layers):
            p = f"model.layers.{i}."
            norms = {n: dev(p + n + ".weight") for n in
                     ("input_layernorm", "post_attention_layernorm", "self_attn.q_norm", "self_attn.k_norm")}
            ws = {g: PackedWeight([packed[f"layers.{i}.{path}"] for path in paths], resident, perm.get(g), self.fmt,
                                  device) for g, paths in GROUPS.items()}
            self.layers.append((norms, ws))
        self.sdpa_gqa = True    # let the attention op share KV heads between query heads instead of copying them
        self.attn_kernel = True  # prefill attention through scmx_attn_prefill where it applies, else torch's op
        half = args.head_dim // 2
        self.inv_freq = 1.0 / (args.rope_theta ** (torch.arange(half, device=device, dtype=torch.float32) / half))

    @classmethod
    def from_float(cls, args, state, **kw):
        """state: Hugging Face state dict with the block linears as float tensors; they are quantized on the GPU."""
        lin = {f"layers.{i}.{path}": state[f"model.layers.{i}.{path}.weight"]
               for i in range(args.num_hidden_layers) for paths in GROUPS.values() for path in paths}
        flat = pack_weights(lin, kw.get("fmt"))
        packed = {k: (flat[k + ".codes"], flat[k + ".bcodes"], flat[k + ".wscale"]) for k in lin}
        return cls(args, state, packed, **kw)

    def weight_bytes(self):
        return sum(w.nbytes() for _, ws in self.layers for w in ws.values())

    def make_cache(self, max_len=4096):
        return [KVCache(self.args, max_len, self.device) for _ in self.layers]

    # ---- pieces shared by prefill and decode --------------------------------------------------------------------
    def _qkv(self, c, L, nw, y=None, acc=None, xs=None, ws=None, pos=None):
        """Per-head RMSNorm of q and k, rotary embedding at positions pos..pos+L-1 (pos defaults to the cache offset;
        an int64 device tensor for graph replay) and the KV-cache append, in one kernel: returns q [hq, L, d]."""
        a = self.args
        return S.qkv_headnorm_rope(y, nw["self_attn.q_norm"], nw["self_attn.k_norm"], self.eps, L, a.num_attention_heads,
                                   a.num_key_value_heads, a.head_dim, c.k, c.v, c.offset if pos is None else pos,
                                   self.inv_freq, acc=acc, xscale=xs, wscale=ws, token_major=L > 1)

    def _attend(self, c, q, L):
        """q [hq, L, d] (already rotated) against the cache, whose rows offset..offset+L-1 were just written."""
        off = c.offset
        if off + L > c.k.shape[1]:
            raise ValueError("KV cache is full")
        c.offset = off + L
        k, v = c.k[:, :off + L], c.v[:, :off + L]
        hq, hk = q.shape[0], k.shape[0]
        if L == 1:
            return S.attn_decode(q, c.k, c.v, off + 1)
        if self.attn_kernel and q.shape[-1] == 128:   # this library's causal attention (head dim 128 only)
            return S.attn_prefill(q, c.k, c.v, off)
        gqa = {"enable_gqa": True} if hq != hk and self.sdpa_gqa else {}
        if hq != hk and not self.sdpa_gqa:
            k, v = k.repeat_interleave(hq // hk, 0), v.repeat_interleave(hq // hk, 0)
        if off == 0:
            o = TF.scaled_dot_product_attention(q[None], k[None], v[None], is_causal=True, **gqa)
        else:
            pos = torch.arange(off, off + L, device=q.device)[:, None]
            mask = torch.arange(off + L, device=q.device)[None] <= pos
            o = TF.scaled_dot_product_attention(q[None], k[None], v[None], attn_mask=mask, **gqa)
        # q arrives as the [hq, L, d] view of [L, hq, d] storage and the attention op lays its output out like q, so
        # this is a view; contiguous() copies only if a backend chose another layout
        return o[0].transpose(0, 1).reshape(L, -1).contiguous()

    def _embed(self, ids):
        h = self.embed[ids.reshape(-1)]
        L = h.shape[0]
        Mp = S.pad_rows(L)
        if Mp != L:
            h = TF.pad(h, (0, 0, 0, Mp - L))
        return h.contiguous(), L, Mp

    # ---- prefill ------------------------------------------------------------------------------------------------
    def hidden(self, ids, cache=None):
        """Final normed hidden states [L, D] for prompt ids [L] (prefill into a fresh or offset cache)."""
        S.set_format(self.fmt)
        cache = cache if cache is not None else self.make_cache(max(4096, ids.numel()))
        return (self._hidden_gemm_epi if self.epilogue == "gemm" else self._hidden_row_epi)(ids, cache)

    def _hidden_gemm_epi(self, ids, cache):
        a = self.args
        hq, hk, d = a.num_attention_heads, a.num_key_value_heads, a.head_dim
        h, L, Mp = self._embed(ids)
        nl = len(self.layers)
        # prefill-sized GEMMs on packed weights read their activations in 32x32 blocks (the quantizers write either layout)
        blk = {g: isinstance(w.unpack(), S.PackedWq) and S.prefers_blocked(Mp, w.N, w.K) for g, w in self.layers[0][1].items()}
        quant = lambda t, g, **kw: (S.act_quant_blocked(t, Mp) if blk[g] else S.act_quant(t, Mp, **kw))   # noqa: E731
        xq, xs = S.rmsnorm_quant(h, self.layers[0][0]["input_layernorm"], self.eps, Mp, blocked=blk["qkv"])
        for i, (nw, ws) in enumerate(self.layers):
            y = S.mm_epi(xq, ws["qkv"].unpack(), xs, ws["qkv"].wscale, 1)
            if cache[i].offset + L > cache[i].k.shape[1]:
                raise ValueError("KV cache is full")
            o = self._attend(cache[i], self._qkv(cache[i], L, nw, y=y), L)
            xq, xs = quant(o, "o")
            h = S.mm_epi(xq, ws["o"].unpack(), xs, ws["o"].wscale, 2, res=h)
            xq, xs = S.rmsnorm_quant(h, nw["post_attention_layernorm"], self.eps, blocked=blk["gu"])
            act = S.mm_epi(xq, ws["gu"].unpack(), xs, ws["gu"].wscale, 3)
            xq, xs = quant(act, "down", nt=512)
            h = S.mm_epi(xq, ws["down"].unpack(), xs, ws["down"].wscale, 2, res=h)
            if i + 1 < nl:
                xq, xs = S.rmsnorm_quant(h, self.layers[i + 1][0]["input_layernorm"], self.eps, blocked=blk["qkv"])
        return rms_norm(h[:L], self.norm, self.eps)

    def _hidden_row_epi(self, ids, cache):
        a = self.args
        hq, hk, d = a.num_attention_heads, a.num_key_value_heads, a.head_dim
        h, L, Mp = self._embed(ids)
        nl = len(self.layers)
        xq, xs = S.rmsnorm_quant(h, self.layers[0][0]["input_layernorm"], self.eps, Mp)
        for i, (nw, ws) in enumerate(self.layers):
            acc = S.mm_i8_i32(xq, ws["qkv"].unpack())
            if cache[i].offset + L > cache[i].k.shape[1]:
                raise ValueError("KV cache is full")
            o = self._attend(cache[i], self._qkv(cache[i], L, nw, acc=acc, xs=xs, ws=ws["qkv"].wscale), L)
            xq, xs = S.act_quant(o, Mp)
            acc = S.mm_i8_i32(xq, ws["o"].unpack())
            h, xq, xs = S.res_norm_quant(acc, xs, ws["o"].wscale, h, nw["post_attention_layernorm"], self.eps)
            acc = S.mm_i8_i32(xq, ws["gu"].unpack())
            xq, xs = S.swiglu_quant(acc, xs, ws["gu"].wscale)
            acc = S.mm_i8_i32(xq, ws["down"].unpack())
            if i + 1 < nl:
                h, xq, xs = S.res_norm_quant(acc, xs, ws["down"].wscale, h, self.layers[i + 1][0]["input_layernorm"],
                                             self.eps)
            else:
                h = S.res_epilogue(acc, xs, ws["down"].wscale, h)
        return rms_norm(h[:L], self.norm, self.eps)

    def logits(self, h):
        return h @ self.lm_head.T

    def __call__(self, ids, cache=None):
        """Logits for every position."""
        return self.logits(self.hidden(ids, cache))


class DecodeQwen3:
    """Batch-1 decode from a FusedQwen3 with epilogue="gemm": W4A8 GEMVs on the packed weights
    (e2e/decode.py:29-99).  fuse_prologue="act" (default): RMSNorm + INT8 as separate kernels, the per-token INT8 of
    the o / down inputs inside those GEMVs' prologues; True: every quantization in a GEMV prologue; False: all
    separate.  graphs=True captures the two fixed-shape halves of every layer in HIP graphs on first use;
    graphs="step" captures the whole step (all layers and the output head) as one graph per cache.  A graph holds raw
    pointers into the cache it was captured with, so the decoder keeps that cache object alive next to the graph and,
    handed a different one, captures again IN PLACE of the old entries: at most one cache (the latest) and its graphs
    are held, a fresh cache per prompt does not accumulate; `release(cache)` drops them before the next prompt.  Tensors returned by `step` are fresh in every mode (the graphs' static outputs are
    cloned).  fuse_attn=True (default): q/k norm, rotary embedding, cache append and the attention in one kernel;
    False: two kernels (same bits).  head="packed": the output projection quantized to the published SC-MXFP4 format
    (32-blocks, multipliers 1,2,4,8) whatever format the model's layers use."""

    def __init__(self, fused, fuse_prologue="act", graphs=False, head=True, fuse_attn=True):
        assert fused.epilogue == "gemm"
        self.f, self.args, self.fuse, self.head = fused, fused.args, fuse_prologue, head
        self.fuse_attn = fuse_attn
        self.graphs = {} if graphs else None
        self.whole_step = graphs == "step"
        self.pos = torch.zeros(1, dtype=torch.int64, device=fused.device)   # position of the token being decoded
        self.packed_head = None
        if head == "packed":   # the output projection as SC-MXFP4 too (quantized here, on the device): 4x fewer bytes
            self.head_fmt = F.Format()          # named explicitly: independent of the process-wide default format
            codes, bc, ws, _ = F.quantize(fused.lm_head, self.head_fmt, with_q=False)
            self.packed_head = (codes, bc, ws, fused.lm_head.shape[0])

    def _logits(self, h):
        f = self.f
        hn = rms_norm(h, f.norm, f.eps)
        if not self.head:
            return hn
        if self.packed_head is None:
            return f.logits(hn)
        codes, bc, ws, n = self.packed_head
        return G.gemv(hn, codes, bc, None, ws, n, 1, pro=1, fmt=self.head_fmt)[None]

    def _pre(self, h, nw, w, c, pos):
        f = self.f
        if self.fuse is True:
            y = G.gemv(h, w.codes, w.bcodes, None, w.wscale, w.N, 1, pro=2, nw=nw["input_layernorm"], eps=f.eps,
                       fmt=f.fmt)
        else:
            xq, xs = S.rmsnorm_quant(h, nw["input_layernorm"], f.eps, 1)
            y = G.gemv(xq, w.codes, w.bcodes, xs, w.wscale, w.N, 1, fmt=f.fmt)
        if self.fuse_attn:   # the attention output, not q: the token's k and v are in the cache afterwards
            a = self.args
            return S.attn_decode_qkv(y, nw["self_attn.q_norm"], nw["self_attn.k_norm"], f.eps, a.num_attention_heads,
                                     a.num_key_value_heads, a.head_dim, c.k, c.v, pos, f.inv_freq)
        return f._qkv(c, 1, nw, y=y[None], pos=pos)

    def _attn(self, c, q):
        """The attention output of the token whose q (or, fused, whose finished attention) _pre returned."""
        if not self.fuse_attn:
            return self.f._attend(c, q, 1)
        c.offset += 1
        return q

    def _post(self, o, h, nw, ws):
        f = self.f
        wo, wg, wd = ws["o"], ws["gu"], ws["down"]
        if self.fuse:
            h = G.gemv(o, wo.codes, wo.bcodes, None, wo.wscale, wo.N, 2, res=h, pro=1, fmt=f.fmt)[None]
        else:
            xq, xs = S.act_quant(o, 1)
            h = G.gemv(xq, wo.codes, wo.bcodes, xs, wo.wscale, wo.N, 2, res=h, fmt=f.fmt)[None]
        if self.fuse is True:
            act = G.gemv(h, wg.codes, wg.bcodes, None, wg.wscale, wg.N, 3, pro=2, nw=nw["post_attention_layernorm"],
                         eps=f.eps, fmt=f.fmt)
        else:
            xq, xs = S.rmsnorm_quant(h, nw["post_attention_layernorm"], f.eps, 1)
            act = G.gemv(xq, wg.codes, wg.bcodes, xs, wg.wscale, wg.N, 3, fmt=f.fmt)
        if self.fuse:
            return G.gemv(act[None], wd.codes, wd.bcodes, None, wd.wscale, wd.N, 2, res=h, pro=1, fmt=f.fmt)[None]
        xq, xs = S.act_quant(act[None], 1)
        return G.gemv(xq, wd.codes, wd.bcodes, xs, wd.wscale, wd.N, 2, res=h, fmt=f.fmt)[None]

    def _capture(self, key, fn, inputs, owner=None):
        """Capture fn(*static copies of inputs) once per (key, owner); returns (graph, static inputs, static outputs).
        `owner` is the object whose memory the captured kernels point into (a cache or one of its layers).  A key
        names a slot of the step ("step", ("pre", layer), ("post", layer)), never an object, and a slot holds the graph
        of ONE owner: capturing for another cache replaces the entry, so the store keeps at most one cache (the most
        recent one) and its graphs alive however many prompts come by, each with a fresh cache.  Alternating between
        two live caches therefore re-captures at every switch; give each its own decoder."""
        if self._lookup(key, owner) is None:
            static = [t.clone() for t in inputs]
            s = torch.cuda.Stream()
            s.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(s):
                fn(*static)                                   # warm-up outside the capture
            torch.cuda.current_stream().wait_stream(s)
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                out = fn(*static)
            self.graphs[key] = (g, static, out, owner)
        return self.graphs[key]

    def _lookup(self, key, owner):
        """The entry stored under key if it was captured for this very owner object; an entry of another owner is
        dropped (with its graph, static buffers and the reference that kept the old cache alive)."""
        entry = self.graphs.get(key)
        if entry is not None and entry[3] is not owner:
            del self.graphs[key]
            entry = None
        return entry

    def _replay(self, key, fn, inputs, owner=None):
        g, static, out, _ = self._capture(key, fn, inputs, owner)
        for dst, src in zip(static, inputs):
            dst.copy_(src)
        g.replay()
        return out

    def release(self, cache=None):
        """Drop the captured graphs bound to `cache` (all graphs when None) together with the references that keep
        their caches alive."""
        if self.graphs is None:
            return
        if cache is None:
            self.graphs.clear()
            return
        owners = [cache] + list(cache)
        for key in [k for k, e in self.graphs.items() if any(e[3] is o for o in owners)]:
            del self.graphs[key]

    # ---- the whole step as one HIP graph -----------------------------------------------------------------------
    # Everything that changes from token to token lives in device memory (token id, position): the fused
    # norm + rotary + append kernel and the attention kernel read the position from there, so the launch sequence is
    # identical for every token and one graph replay per token replaces every launch of the step and its host-side
    # preparation.
    def _step_static(self, tok, cache):
        f = self.f
        h = f.embed.index_select(0, tok)
        for i, (nw, ws) in enumerate(f.layers):
            c = cache[i]
            q = self._pre(h, nw, ws["qkv"], c, self.pos)
            h = self._post(q if self.fuse_attn else S.attn_decode(q, c.k, c.v, self.pos), h, nw, ws)
        return self._logits(h)

    def step(self, tok, cache):
        """tok: int64 [1] -> logits [1, V] (or the final hidden row when head is False)."""
        f = self.f
        S.set_format(f.fmt)
        off = cache[0].offset
        if off >= cache[0].k.shape[1]:
            raise ValueError("KV cache is full")
        tok = tok.reshape(-1)[:1]
        if self.graphs is not None:
            self.pos.fill_(off)
        if self.whole_step:
            out = self._replay(("step",), lambda t: self._step_static(t, cache), [tok], owner=cache)
            for c in cache:
                c.offset = off + 1
            return out.clone()     # the graph's static output is overwritten by the next replay
        h = f.embed[tok].contiguous()   # [1, D]
        for i, (nw, ws) in enumerate(f.layers):
            c = cache[i]
            if self.graphs is None:
                q = self._pre(h, nw, ws["qkv"], c, off)
            else:
                q = self._replay(("pre", i), lambda x, nw=nw, w=ws["qkv"], c=c: self._pre(x, nw, w, c, self.pos), [h],
                                 owner=c)
            o = self._attn(c, q)
            if self.graphs is None:
                h = self._post(o, h, nw, ws)
            else:
                h = self._replay(("post", i), lambda x, r, nw=nw, ws=ws: self._post(x, r, nw, ws), [o, h])
        return self._logits(h)      # new tensors: the final norm never returns a graph's static buffer


# ---- from a checkpoint directory -----------------------------------------------------------------------------------

def read_checkpoint(model_dir):
    """A local Hugging Face checkpoint directory (config.json + *.safetensors) -> (Qwen3Args, state dict of CPU
    tensors).  Nothing is fetched: the directory must hold the files."""
    from safetensors import safe_open
    with open(os.path.join(model_dir, "config.json")) as fh:
        cfg = json.load(fh)
    known = {f.name for f in fields(Qwen3Args)}
    kw = {k: v for k, v in cfg.items() if k in known}
    if "head_dim" not in kw:
        kw["head_dim"] = cfg["hidden_size"] // cfg["num_attention_heads"]
    args = Qwen3Args(**kw)
    files = sorted(f for f in os.listdir(model_dir) if f.endswith(".safetensors"))
    if not files:
        raise FileNotFoundError(f"{model_dir}: no .safetensors weight files")
    state = {}
    for name in files:
        with safe_open(os.path.join(model_dir, name), framework="pt", device="cpu") as fh:
            for key in fh.keys():
                state[key] = fh.get_tensor(key)
    return args, state


def load_fused(model_dir, cache_dir, resident=False, epilogue="gemm", packed="rtn"):
    """The counterpart of e2e/fused_qwen3.py:304-338 for a checkpoint directory on disk: returns (FusedQwen3,
    tokenizer or None).  packed="rtn": round-to-nearest SC-MXFP4 in the byte-shift cache
    "<name>-scmxfp4.safetensors" under cache_dir (keys layers.{i}.{path}.codes / .shifts / .wscale, the file the
    reference's pack_model writes, e2e/w4a8_mlx.py:175-195), packed on the GPU on first use; "gptq": the same format
    from "<name>-scmxfp4-gptq.safetensors", which must exist (the GPTQ packer is not part of this library);
    "fmt:<family member>": the cache of e2e/pack_format.py, written on first use by the device quantizer of the
    family.  The rotated-basis caches ("rot:", "rotdown:") are not supported."""
    from . import pack_format as PF
    from . import sc_weights as W
    args, state = read_checkpoint(model_dir)
    name = os.path.basename(os.path.normpath(model_dir))
    n_layers = args.num_hidden_layers
    lin = lambda: {f"layers.{i}.{path}": state[f"model.layers.{i}.{path}.weight"]   # noqa: E731
                   for i in range(n_layers) for paths in GROUPS.values() for path in paths}
    os.makedirs(cache_dir, exist_ok=True)
    fmt = None
    if packed.startswith(("rot:", "rotdown:")):
        raise NotImplementedError("weights packed in the rotated basis are not supported by this driver")
    if packed.startswith("fmt:"):
        member = packed[4:]
        fmt = PF.sc_format_of(member)
        cache = PF.cache_path(name, member, cache_dir)
        if not os.path.exists(cache):
            flat = {}
            for key, w in lin().items():
                codes, bc, ws, _ = PF.pack_matrix(w.cuda(), member, fmt)
                flat[key + ".codes"], flat[key + ".bcodes"], flat[key + ".wscale"] = codes, bc, ws
            W.save_cache(cache, flat)
        pk = W.load_cache(cache)
    elif packed in ("rtn", "gptq"):
        cache = os.path.join(cache_dir, name + {"rtn": "-scmxfp4.safetensors", "gptq": "-scmxfp4-gptq.safetensors"}[packed])
        if not os.path.exists(cache):
            if packed == "gptq":
                raise FileNotFoundError(f"{cache} is missing (written by the reference's e2e/gptq_pack.py)")
            flat, out = pack_weights(lin()), {}
            for key in sorted(k[:-6] for k in flat if k.endswith(".codes")):
                c, sh, ws = F.to_shift_layout(flat[key + ".codes"], flat[key + ".bcodes"], flat[key + ".wscale"])
                out[key + ".codes"], out[key + ".shifts"], out[key + ".wscale"] = c, sh, ws
            W.save_cache(cache, out)
        pk = W.load_packed(cache, n_layers)
    else:
        raise ValueError(f"unknown packed={packed!r}")
    tok = None
    if any(os.path.exists(os.path.join(model_dir, f)) for f in ("tokenizer.json", "tokenizer_config.json")):
        from transformers import AutoTokenizer
        tok = AutoTokenizer.from_pretrained(model_dir, local_files_only=True)
    return FusedQwen3(args, state, pk, resident=resident, epilogue=epilogue, fmt=fmt), tok
