"""Qwen3.5-MoE (256 routed experts, top-8, plus one shared expert that every token visits): the sparse-MoE half of a
transformer block through the W4A8 kernels, prefill and batch-1 decode.  The torch-ROCm counterpart of
e2e/fused_qwen35.py:171-180 (route), :259-293 (FusedQwen35._moe_fn), :205-219 (expert stacks, gate|up interleave),
e2e/decode.py:168-215 (DecodeQwen35's moe / moe_lean) and of the synthetic-weight block e2e/bench_moe_q38.py:60-105.

  xq, xs, xn = rmsnorm_quant_n(h)                       INT8 rows for the experts, bf16 rows for the router
  inds9, scores9 = route(xn)                            softmax -> top-8 -> renormalise; slot 9 = shared expert, score sigmoid
  route_sort over E + 1 experts
  act = moe_mm(xq, gather=tok, Wg|Wu, SwiGLU)           the shared expert is expert E of the same grouped launch
  y = moe_mm(act_quant(act), Wd)
  h = moe_combine(y, scores9, + h)                      sequential bf16 sum over the 9 slots = mlx_lm's
                                                        (y * scores).sum(-2) + sigmoid(g) * y_shared (e2e/fused_qwen35.py:12-15)

The other half of a Qwen3.5 block -- Gated DeltaNet / gated attention after the projections -- is mlx_lm's own model code
in the reference (e2e/fused_qwen35.py:120-168) and is not part of this library; its projections are ordinary dense
layers (sc_kernels.mm_epi / sc_decode.gemv on a sc_weights.PackedWeight)."""
from dataclasses import dataclass

import numpy as np
import torch

from . import sc_decode as G
from . import sc_format as F
from . import sc_kernels as S
from . import sc_moe

BF = torch.bfloat16
EXPERTS = ["gate_proj", "up_proj", "down_proj"]   # e2e/fused_qwen35.py:37


@dataclass
class Qwen35MoeArgs:
    hidden_size: int = 2048
    moe_intermediate_size: int = 512
    num_experts: int = 256
    num_experts_per_tok: int = 8
    rms_norm_eps: float = 1e-6


def route(gate_w, sg_w, xn, k):
    """Qwen3NextSparseMoeBlock routing on bf16 normalized rows xn [M, D] (e2e/fused_qwen35.py:171-180): the two bf16
    linears are array ops as in the reference; one kernel does softmax (float32) -> k largest -> renormalise and
    appends the shared expert as slot k with index E and score sigmoid(xn . sg_w).  -> (inds int32, scores bf16) [M, k+1]."""
    return sc_moe.route(xn @ gate_w.T, k, renorm=True, shared_logit=xn @ sg_w.T)


def pack_experts(gate, up, down, fmt=None, fmt_name=None):
    """Float expert weights with the shared expert LAST (gate, up [E+1, F, D]; down [E+1, D, F]; torch, any device) ->
    {"experts.<name>.codes|bcodes|wscale"} numpy stacks over the E + 1 experts, the reference's cache layout
    (e2e/fused_qwen35.py:94-103), quantized on the GPU: SC-MXFP4 (fmt: 32- or 16-wide blocks) or, with fmt_name, a
    member of the format family (pack_format.pack_matrix)."""
    flat = {}
    for name, w in zip(EXPERTS, (gate, up, down)):
        e1, n, k = w.shape
        m = w.reshape(e1 * n, k).cuda()            # the quantizers work row by row: one launch for the whole stack
        if fmt_name:
            from . import pack_format
            c, b, s, _ = pack_format.pack_matrix(m, fmt_name, fmt)
        else:
            c, b, s, _ = F.quantize(m, fmt or F.Format(), with_q=False)
        flat[f"experts.{name}.codes"] = c.cpu().numpy().view(np.uint32).reshape(e1, n, k // 8)
        flat[f"experts.{name}.bcodes"] = b.cpu().numpy().reshape(e1, n, -1)
        flat[f"experts.{name}.wscale"] = s.cpu().numpy().reshape(e1, n)
    return flat


class Qwen35Moe:
    def __init__(self, args, post_norm, gate_w, sg_w, flat, prefix="", tile=None, two_pass="auto", fmt=None, device="cuda"):
        """post_norm [D]: the post-attention RMSNorm weight; gate_w [E, D]: router; sg_w [1, D]: shared_expert_gate.
        flat: {prefix + "experts.<gate_proj|up_proj|down_proj>.<codes|bcodes|wscale>"} stacked over E + 1 experts, shared
        expert last (pack_experts, or a cache written by the reference's pack_qwen35).  tile: row tile of the grouped
        GEMM (None: by the rows per expert of each call); two_pass: unpack all experts to INT8 first
        ("auto": from 256 rows per expert on, e2e/fused_qwen35.py:268)."""
        self.args, self.device, self.tile, self.two_pass = args, device, tile, two_pass
        self.fmt = fmt if fmt is not None else F.Format()
        self.eps = float(args.rms_norm_eps)
        E1, Fi, D = args.num_experts + 1, args.moe_intermediate_size, args.hidden_size
        dev = lambda t: torch.as_tensor(t).to(device=device, dtype=BF).contiguous()   # noqa: E731
        self.pn, self.gate_w, self.sg_w = dev(post_norm), dev(gate_w), dev(sg_w).reshape(1, D)
        host = lambda k: (lambda t: t.cpu().numpy() if torch.is_tensor(t) else np.asarray(t))(flat[prefix + k])   # noqa: E731
        perm = S.interleave_gate_up(Fi)
        ek = lambda n, s: host(f"experts.{n}.{s}")   # noqa: E731
        # gate rows and up rows of an expert side by side, then in the order the SwiGLU epilogue pairs them
        gu_c = np.concatenate([ek("gate_proj", "codes").view(np.uint32).reshape(E1, Fi, -1),
                               ek("up_proj", "codes").view(np.uint32).reshape(E1, Fi, -1)], 1)[:, perm].reshape(E1, -1)
        gu_b = np.concatenate([ek("gate_proj", "bcodes").reshape(E1, Fi, -1), ek("up_proj", "bcodes").reshape(E1, Fi, -1)], 1)[:, perm]
        gu_s = np.concatenate([ek("gate_proj", "wscale").reshape(E1, Fi), ek("up_proj", "wscale").reshape(E1, Fi)], 1)[:, perm]
        self.gu = F.to_device(gu_c, gu_b, gu_s, device)
        self.down = F.to_device(ek("down_proj", "codes").view(np.uint32).reshape(E1, -1), ek("down_proj", "bcodes").reshape(E1, D, -1),
                                ek("down_proj", "wscale").reshape(E1, D), device)
        assert self.gu[0].shape[1] == 2 * Fi * D // 8 and self.down[0].shape[1] == D * Fi // 8
        self.pos = torch.arange(args.num_experts_per_tok + 1, dtype=torch.int32, device=device)
        self.record = None   # set to a list to collect (inds9, scores9) of every call, as the reference's checks do

    @classmethod
    def from_float(cls, args, post_norm, gate_w, sg_w, gate, up, down, fmt=None, fmt_name=None, **kw):
        """gate, up [E+1, F, D], down [E+1, D, F] float weights, shared expert last."""
        if fmt_name and fmt is None:
            from . import pack_format
            fmt = pack_format.sc_format_of(fmt_name)
        return cls(args, post_norm, gate_w, sg_w, pack_experts(gate, up, down, fmt, fmt_name), fmt=fmt, **kw)

    def weight_bytes(self):
        return sum(t.numel() * t.element_size() for t in self.gu + self.down)

    def _route(self, xn):
        inds9, scores9 = route(self.gate_w, self.sg_w, xn, self.args.num_experts_per_tok)
        if self.record is not None:
            self.record.append((inds9, scores9))
        return inds9, scores9

    def prefill(self, h, L):
        """h bf16 [Mp, D] (rows >= L are padding) -> h + MoE(rms_norm(h)) [Mp, D]; the reference's moe()
        (e2e/fused_qwen35.py:270-289)."""
        a = self.args
        S.set_format(self.fmt)
        k, E1, F2, D = a.num_experts_per_tok, a.num_experts + 1, 2 * a.moe_intermediate_size, a.hidden_size
        R = L * (k + 1)
        tm = self.tile or sc_moe.row_tile(R, E1)
        two_pass = self.two_pass if self.two_pass != "auto" else R // E1 >= 256
        xq, xs, xn = S.rmsnorm_quant_n(h, self.pn, self.eps)
        inds9, scores9 = self._route(xn[:L])
        pos, tok, _, off, tstart, maxt = sc_moe.route_sort(inds9, E1, tm)
        (cg, bg, sg), (cd, bd, sd), t = self.gu, self.down, (tm, 64, 4)
        if two_pass:
            act = sc_moe.moe_mm_i8(xq, R, sc_moe.unpack_experts(cg, bg, F2, D), sg, off, tstart, maxt, F2, 3, xs, tile=t,
                                   gather=tok)
        else:
            act = sc_moe.moe_mm(xq, R, cg, bg, sg, off, tstart, maxt, F2, 3, xs, tile=t, gather=tok, fmt=self.fmt)
        xq2, xs2 = S.act_quant(act, R)
        if two_pass:
            yd = sc_moe.moe_mm_i8(xq2, R, sc_moe.unpack_experts(cd, bd, D, F2 // 2), sd, off, tstart, maxt, D, 1, xs2, tile=t)
        else:
            yd = sc_moe.moe_mm(xq2, R, cd, bd, sd, off, tstart, maxt, D, 1, xs2, tile=t, fmt=self.fmt)
        return sc_moe.moe_combine(yd, pos, scores9, h, self.pn, self.eps, L, quant=False)[0]

    def decode(self, h, lean=True):
        """One token, h bf16 [1, D] -> [1, D]: the expert GEMVs gather the 8 routed experts' rows themselves, gate|up over
        9 slots sharing the input row, down with one input row per slot (e2e/decode.py:187-214).  lean: the shared
        expert is the GEMVs' implicit last slot, its gate a separate input of the combine, and the down GEMV quantizes
        its 9 input rows itself; same result as lean=False."""
        a = self.args
        S.set_format(self.fmt)
        k, E, F2, D = a.num_experts_per_tok, a.num_experts, 2 * a.moe_intermediate_size, a.hidden_size
        xq, xs, xn = S.rmsnorm_quant_n(h, self.pn, self.eps, 1)
        inds9, scores9 = self._route(xn)
        (cg, bg, sg), (cd, bd, sd) = self.gu, self.down
        if lean:
            e = inds9[0, :k]
            act = G.gemv(xq, cg, bg, xs, sg, F2, 3, eidx=e, xstride=0, shared=E, fmt=self.fmt)                # [9, F]
            yd = G.gemv(act, cd, bd, None, sd, D, 1, eidx=e, xstride=1, shared=E, pro=1, fmt=self.fmt)        # [9, D]
            return sc_moe.moe_combine_split(yd, self.pos, scores9[:, :k].contiguous(), scores9[0, k:].contiguous(), h,
                                            self.pn, self.eps, 1)[0]
        e = inds9.reshape(-1)
        act = G.gemv(xq, cg, bg, xs, sg, F2, 3, eidx=e, xstride=0, fmt=self.fmt)
        xq2, xs2 = S.act_quant(act, k + 1)
        yd = G.gemv(xq2, cd, bd, xs2, sd, D, 1, eidx=e, xstride=1, fmt=self.fmt)
        return sc_moe.moe_combine(yd, self.pos, scores9, h, self.pn, self.eps, 1, quant=False)[0]
