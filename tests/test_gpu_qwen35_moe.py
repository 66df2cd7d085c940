"""The Qwen3.5-MoE half-block (routed experts + the shared expert as one more expert) on the GPU: against a float32
torch block with the dequantized weights, prefill variants against each other bit for bit, batch-1 decode against the
prefill rows bit for bit, and the real shape of BASELINE config 4.  Mirrors the checks of e2e/bench_moe_q38.py:189-212
and e2e/check_fused_qwen35.py (prefill vs a float model; decode vs prefill)."""
import numpy as np
import pytest
import torch

from oracle import layout

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def default_format_afterwards():
    """The block selects its weight format globally at every call (as the reference's set_format does); leave the
    default behind for whatever runs next."""
    yield
    from mxfp4_int8_m5_amd import sc_format, sc_kernels
    sc_kernels.set_format(sc_format.Format())


def rel(a, b):
    a, b = a.float().cpu(), b.float().cpu()
    return float((a - b).norm() / b.norm())


def make_block(fmt=None, fmt_name=None, seed=30, **kw):
    from mxfp4_int8_m5_amd import fused_qwen35 as Q
    args = Q.Qwen35MoeArgs(hidden_size=256, moe_intermediate_size=128, num_experts=8, num_experts_per_tok=2)
    g = torch.Generator().manual_seed(seed)
    rnd = lambda *s, sc=1.0: torch.randn(*s, generator=g) * sc   # noqa: E731
    D, Fi, E1 = args.hidden_size, args.moe_intermediate_size, args.num_experts + 1
    w = dict(pn=(1 + rnd(D, sc=0.1)).bfloat16().float(), gate_w=rnd(E1 - 1, D, sc=4 * D ** -0.5).bfloat16().float(),
             sg_w=rnd(1, D, sc=2 * D ** -0.5).bfloat16().float(), gate=rnd(E1, Fi, D, sc=D ** -0.5),
             up=rnd(E1, Fi, D, sc=D ** -0.5), down=rnd(E1, D, Fi, sc=Fi ** -0.5))
    flat = Q.pack_experts(w["gate"], w["up"], w["down"], fmt, fmt_name)
    blk = Q.Qwen35Moe(args, w["pn"], w["gate_w"], w["sg_w"], flat, fmt=fmt, **kw)
    return Q, args, w, flat, blk


def hidden_rows(L, Mp, D, seed):
    h = torch.zeros(Mp, D)
    h[:L] = torch.randn(L, D, generator=torch.Generator().manual_seed(seed))
    return h.bfloat16().cuda()


def float_block(args, w, flat, fmt, h, routing):
    """h + sum over the 9 slots of score x expert(rms_norm(h)) in float32 on the CPU, with the dequantized weights, no
    activation quantization, and the routing of the run under test."""
    ofmt = layout.Format(block=fmt.block, code_mag=tuple(fmt.code_mag), mult=tuple(fmt.mult), bc_bits=fmt.bc_bits)

    cache = {}

    def weight(name, e):
        if (name, e) not in cache:
            cache[name, e] = dequantized(name, e)
        return cache[name, e]

    def dequantized(name, e):
        c, b, s = (flat[f"experts.{name}.{p}"][e] for p in ("codes", "bcodes", "wscale"))
        n = s.shape[0]
        return torch.from_numpy(layout.decode(c.reshape(-1), b, n, c.size * 8 // n, ofmt).astype(np.float32) * s[:, None])

    h = h.float().cpu()
    x = h * torch.rsqrt(h.pow(2).mean(-1, keepdim=True) + args.rms_norm_eps) * w["pn"]
    inds, scores = (t.cpu() for t in routing)
    y = torch.zeros_like(h)
    for t in range(inds.shape[0]):
        for j in range(inds.shape[1]):
            e = int(inds[t, j])
            act = torch.nn.functional.silu(x[t] @ weight("gate_proj", e).T) * (x[t] @ weight("up_proj", e).T)
            y[t] += float(scores[t, j]) * (act @ weight("down_proj", e).T)
    return h + y, y


@pytest.mark.parametrize("fmt_i,fmt_name", [(0, None), (1, None), (5, "e2m1/B16/M1..10")])
def test_prefill_against_float_block(fmt_i, fmt_name):
    from tests.util import FORMATS, product_format
    fmt = product_format(FORMATS[fmt_i])
    Q, args, w, flat, blk = make_block(fmt, fmt_name)
    L, Mp = 45, 128
    h = hidden_rows(L, Mp, args.hidden_size, 31)
    blk.record = []
    out = blk.prefill(h, L)
    inds9, scores9 = blk.record[0]
    E = args.num_experts
    assert inds9.shape == (L, 3) and bool((inds9[:, 2] == E).all()) and bool((inds9[:, :2] < E).all())
    ref, delta = float_block(args, w, flat, fmt, h[:L], blk.record[0])
    assert rel(out[:L], ref) < 2e-2, rel(out[:L], ref)
    assert rel(out[:L].float().cpu() - h[:L].float().cpu(), delta) < 5e-2
    assert float(delta.norm() / ref.norm()) > 0.2          # the MoE term is a real part of the result


def test_prefill_variants_agree_bit_for_bit():
    """Row tile, two-pass (all experts unpacked to INT8 first) and in-kernel unpack compute the same integers."""
    Q, args, w, flat, blk = make_block()
    L, Mp = 200, 256
    h = hidden_rows(L, Mp, args.hidden_size, 32)
    base = blk.prefill(h, L)
    for kw in (dict(tile=64), dict(tile=128, two_pass=True), dict(tile=256), dict(two_pass=False)):
        other = Q.Qwen35Moe(args, w["pn"], w["gate_w"], w["sg_w"], flat, **kw).prefill(h, L)
        assert torch.equal(other[:L], base[:L]), kw


@pytest.mark.parametrize("fmt_i", [0, 1])
def test_decode_equals_the_prefill_rows(fmt_i):
    """The 9-slot expert GEMVs, either way of feeding the shared expert, give the bits of the grouped GEMM path."""
    from tests.util import FORMATS, product_format
    fmt = product_format(FORMATS[fmt_i])
    Q, args, w, flat, blk = make_block(fmt)
    L, Mp = 20, 128
    h = hidden_rows(L, Mp, args.hidden_size, 33)
    full = blk.prefill(h, L)
    for t in (0, 7, 19):
        row = h[t:t + 1].contiguous()
        lean, plain = blk.decode(row, lean=True), blk.decode(row, lean=False)
        assert torch.equal(lean, plain)
        assert torch.equal(lean[0], full[t])


def test_config4_block_at_its_real_shape():
    """256 routed experts + the shared one, hidden 2048, expert width 512, top-8, 16-wide blocks, 2048 tokens:
    float weights quantized on the device, the block's prefill does not depend on the row tile, and the batch-1 decode
    of single tokens reproduces their prefill rows bit for bit."""
    from mxfp4_int8_m5_amd import fused_qwen35 as Q, sc_format as F
    args = Q.Qwen35MoeArgs()
    D, Fi, E1, L = args.hidden_size, args.moe_intermediate_size, args.num_experts + 1, 2048
    g = torch.Generator(device="cuda").manual_seed(34)
    rnd = lambda *s, sc=1.0: torch.randn(*s, generator=g, device="cuda") * sc   # noqa: E731
    fmt = F.Format(block=16)
    bias = rnd(E1 - 1, 1, sc=1.5)
    blk = Q.Qwen35Moe.from_float(args, 1 + rnd(D, sc=0.1), rnd(E1 - 1, D, sc=D ** -0.5) * (1 + bias.abs()), rnd(1, D, sc=D ** -0.5),
                                 rnd(E1, Fi, D, sc=0.02), rnd(E1, Fi, D, sc=0.02), rnd(E1, D, Fi, sc=0.02), fmt=fmt)
    nw = E1 * 3 * Fi * D
    assert blk.weight_bytes() == nw // 2 + nw // 64 + E1 * (2 * Fi + D) * 4     # nibbles + 2 bits per 16 + row scales
    h = (rnd(L, D)).bfloat16()
    blk.record = []
    out = blk.prefill(h, L)
    inds9, _ = blk.record[0]
    counts = torch.bincount(inds9.flatten().long(), minlength=E1)
    assert int(counts[E1 - 1]) == L and int(counts.sum()) == L * 9
    assert bool(torch.isfinite(out.float()).all())
    blk.tile = 256
    assert torch.equal(blk.prefill(h, L), out)
    for t in (0, 1000, 2047):
        assert torch.equal(blk.decode(h[t:t + 1].contiguous())[0], out[t])
