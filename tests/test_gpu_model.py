"""Model-level checks of the Qwen3 integration (prefill in both epilogue styles, batch-1 decode, HIP-graph replay)
on a small random model.  The kernels themselves are pinned bit-exactly elsewhere; here the composition is checked
against a plain float32 torch model that uses the dequantized weights, within the W4A8 tolerance, and the decode path
against the prefill path, as the reference does in e2e/check_fused.py and e2e/check_decode.py."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def default_format_afterwards():
    """The model drivers select their weight format globally (as the reference's set_format does); leave the default
    behind for whatever runs next."""
    yield
    from mxfp4_int8_m5_amd import sc_format, sc_kernels
    sc_kernels.set_format(sc_format.Format())


@pytest.fixture(scope="module")
def tiny():
    return make_tiny(4, 2, 64)


def make_tiny(hq, hk, head_dim, hidden=256):
    from mxfp4_int8_m5_amd import fused_qwen3 as Q, sc_weights as W
    args = Q.Qwen3Args(hidden_size=hidden, intermediate_size=512, num_hidden_layers=2, num_attention_heads=hq,
                       num_key_value_heads=hk, head_dim=head_dim, vocab_size=320, rope_theta=1e4)
    g = torch.Generator().manual_seed(0)
    rnd = lambda *s, sc=1.0: torch.randn(*s, generator=g) * sc   # noqa: E731
    state = {"model.embed_tokens.weight": rnd(args.vocab_size, args.hidden_size),
             "model.norm.weight": 1 + rnd(args.hidden_size, sc=0.1)}
    shapes = {"self_attn.q_proj": (hq * head_dim, hidden), "self_attn.k_proj": (hk * head_dim, hidden),
              "self_attn.v_proj": (hk * head_dim, hidden), "self_attn.o_proj": (hidden, hq * head_dim),
              "mlp.gate_proj": (512, hidden), "mlp.up_proj": (512, hidden), "mlp.down_proj": (hidden, 512)}
    for i in range(args.num_hidden_layers):
        p = f"model.layers.{i}."
        for n in ("input_layernorm", "post_attention_layernorm"):
            state[p + n + ".weight"] = 1 + rnd(args.hidden_size, sc=0.1)
        for n in ("self_attn.q_norm", "self_attn.k_norm"):
            state[p + n + ".weight"] = 1 + rnd(args.head_dim, sc=0.1)
        for n, (o, k) in shapes.items():
            state[p + n + ".weight"] = rnd(o, k, sc=k ** -0.5)
    state = {k: v.to(torch.bfloat16).float() for k, v in state.items()}     # bf16-representable parameters
    lin = {f"layers.{i}.{n}": state[f"model.layers.{i}.{n}.weight"] for i in range(2) for n in shapes}
    flat = W.pack_weights(lin)
    packed = {k: (flat[k + ".codes"], flat[k + ".bcodes"], flat[k + ".wscale"]) for k in lin}
    return Q, args, state, packed


def float_model(Q, args, state, packed, ids):
    """float32 torch on the CPU: the same network with the dequantized 4-bit weights and no activation quantization."""
    from oracle import layout
    a = args
    hq, hk, d, eps = a.num_attention_heads, a.num_key_value_heads, a.head_dim, a.rms_norm_eps

    def weight(i, n):
        c, b, s = packed[f"layers.{i}.{n}"]
        rows = s.shape[0]
        k = c.size * 8 // rows
        return torch.from_numpy(layout.decode(c, b, rows, k).astype(np.float32) * s[:, None])

    def norm(x, w):
        return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * w

    def rope(x):
        L = x.shape[1]
        half = d // 2
        inv = 1.0 / (a.rope_theta ** (torch.arange(half, dtype=torch.float32) / half))
        ang = torch.arange(L, dtype=torch.float32)[:, None] * inv[None]
        x1, x2 = x.chunk(2, -1)
        return torch.cat([x1 * ang.cos() - x2 * ang.sin(), x2 * ang.cos() + x1 * ang.sin()], -1)

    h = state["model.embed_tokens.weight"][ids]
    L = h.shape[0]
    for i in range(a.num_hidden_layers):
        p = f"model.layers.{i}."
        x = norm(h, state[p + "input_layernorm.weight"])
        q = (x @ weight(i, "self_attn.q_proj").T).view(L, hq, d).transpose(0, 1)
        k = (x @ weight(i, "self_attn.k_proj").T).view(L, hk, d).transpose(0, 1)
        v = (x @ weight(i, "self_attn.v_proj").T).view(L, hk, d).transpose(0, 1)
        q, k = rope(norm(q, state[p + "self_attn.q_norm.weight"])), rope(norm(k, state[p + "self_attn.k_norm.weight"]))
        k, v = k.repeat_interleave(hq // hk, 0), v.repeat_interleave(hq // hk, 0)
        o = torch.nn.functional.scaled_dot_product_attention(q[None], k[None], v[None], is_causal=True)[0]
        h = h + o.transpose(0, 1).reshape(L, -1) @ weight(i, "self_attn.o_proj").T
        x = norm(h, state[p + "post_attention_layernorm.weight"])
        g, u = x @ weight(i, "mlp.gate_proj").T, x @ weight(i, "mlp.up_proj").T
        h = h + (torch.nn.functional.silu(g) * u) @ weight(i, "mlp.down_proj").T
    return norm(h, state["model.norm.weight"])


def rel(a, b):
    a, b = a.float().cpu(), b.float().cpu()
    return float((a - b).norm() / b.norm())


@pytest.mark.parametrize("epilogue", ["gemm", "row"])
def test_prefill_against_float_model(tiny, epilogue):
    Q, args, state, packed = tiny
    ids = torch.randint(0, args.vocab_size, (70,), generator=torch.Generator().manual_seed(1))
    m = Q.FusedQwen3(args, state, packed, epilogue=epilogue)
    h = m.hidden(ids.cuda())
    ref = float_model(Q, args, state, packed, ids)
    assert h.shape == ref.shape
    assert rel(h, ref) < 3e-2, rel(h, ref)       # two blocks of INT8 activations + bf16 residual stream


def test_prefill_from_blocked_activations_gives_the_same_bits(monkeypatch):
    """Prefill-sized GEMMs read their activations in 32x32 blocks (every quantizer of the block writes that layout); with
    the choice forced on for a small model the hidden states equal those of the row layout bit for bit."""
    Q, args, state, packed = make_tiny(4, 2, 64, hidden=512)
    from mxfp4_int8_m5_amd import sc_kernels as S
    ids = torch.randint(0, args.vocab_size, (150,), generator=torch.Generator().manual_seed(5)).cuda()
    m = Q.FusedQwen3(args, state, packed)
    by_rows = m.hidden(ids)
    seen = []
    real = S.act_quant_blocked
    monkeypatch.setattr(S, "prefers_blocked", lambda M, N, K: True)
    monkeypatch.setattr(S, "act_quant_blocked", lambda *a, **k: (seen.append(1), real(*a, **k))[1])
    in_blocks = m.hidden(ids)
    assert len(seen) == 2 * args.num_hidden_layers          # the o_proj and down inputs of every block
    assert torch.equal(in_blocks, by_rows)
    assert rel(by_rows, float_model(Q, args, state, packed, ids.cpu())) < 3e-2


def test_prefill_with_this_librarys_attention_kernel():
    """Head dim 128: the prefill runs scmx_attn_prefill; against the float model, against the same driver on torch's
    attention op, and a second chunk appended behind the first (attention at an offset) against one pass over both."""
    Q, args, state, packed = make_tiny(4, 2, 128)
    ids = torch.randint(0, args.vocab_size, (200,), generator=torch.Generator().manual_seed(21)).cuda()
    m = Q.FusedQwen3(args, state, packed)
    assert m.attn_kernel
    h = m.hidden(ids)
    ref = float_model(Q, args, state, packed, ids.cpu())
    assert rel(h, ref) < 4e-2, rel(h, ref)
    m2 = Q.FusedQwen3(args, state, packed)
    m2.attn_kernel = False
    assert rel(h, m2.hidden(ids)) < 2e-2      # two attention kernels' rounding through two blocks of INT8 activations
    cache = m.make_cache(256)
    first = m.hidden(ids[:130], cache)
    second = m.hidden(ids[130:], cache)
    assert cache[0].offset == 200
    assert torch.equal(first, h[:130]) and rel(second, h[130:]) < 2e-2


def test_resident_int8_weights_give_the_same_result(tiny):
    Q, args, state, packed = tiny
    ids = torch.randint(0, args.vocab_size, (33,), generator=torch.Generator().manual_seed(2)).cuda()
    a = Q.FusedQwen3(args, state, packed).hidden(ids)
    b = Q.FusedQwen3(args, state, packed, resident=True).hidden(ids)
    assert torch.equal(a, b)                       # fused unpack and the INT8 copy feed the same integers to the MFMAs


def test_from_float_quantizes_on_the_device(tiny):
    Q, args, state, packed = tiny
    ids = torch.randint(0, args.vocab_size, (20,), generator=torch.Generator().manual_seed(3)).cuda()
    a = Q.FusedQwen3(args, state, packed).hidden(ids)
    b = Q.FusedQwen3.from_float(args, state).hidden(ids)
    assert torch.equal(a, b)


@pytest.mark.parametrize("fuse", ["act", True, False])
def test_decode_continues_the_prefill(tiny, fuse):
    """Prefill L tokens, decode the next 3 one by one: the hidden rows equal those of one prefill over L + 3 tokens
    up to the attention kernels' rounding (the linears see identical INT8 rows in both paths)."""
    Q, args, state, packed = tiny
    ids = torch.randint(0, args.vocab_size, (40,), generator=torch.Generator().manual_seed(4)).cuda()
    m = Q.FusedQwen3(args, state, packed)
    full = m.hidden(ids)
    cache = m.make_cache(64)
    m.hidden(ids[:37], cache)
    dec = Q.DecodeQwen3(m, fuse_prologue=fuse, head=False)
    rows = torch.cat([dec.step(ids[37 + j:38 + j], cache) for j in range(3)])
    assert cache[0].offset == 40
    assert rel(rows, full[37:]) < 2e-2, rel(rows, full[37:])


def test_decode_graph_replays_match_eager_steps(tiny):
    """Each captured half is replayed on every step; between replays the program runs its eager attention and cache
    updates.  Every step's logits must equal the eager decoder's bit for bit."""
    Q, args, state, packed = tiny
    ids = torch.randint(0, args.vocab_size, (24,), generator=torch.Generator().manual_seed(5)).cuda()
    m = Q.FusedQwen3(args, state, packed)
    c1, c2 = m.make_cache(64), m.make_cache(64)
    m.hidden(ids[:16], c1)
    m.hidden(ids[:16], c2)
    eager, graphed = Q.DecodeQwen3(m), Q.DecodeQwen3(m, graphs=True)
    for j in range(16, 24):
        a = eager.step(ids[j:j + 1], c1)
        b = graphed.step(ids[j:j + 1], c2)
        torch.cuda.synchronize()
        assert a.shape == (1, args.vocab_size) and torch.equal(a, b), j


def test_whole_step_graph_follows_the_eager_decoder(tiny):
    """One graph per step with attention over the whole cache buffer under a position mask: equal to the eager
    decoder up to the attention kernel's summation order, on every replay (positions and tokens change between
    replays, and so does the cache content the replayed kernels read)."""
    Q, args, state, packed = tiny
    ids = torch.randint(0, args.vocab_size, (30,), generator=torch.Generator().manual_seed(6)).cuda()
    m = Q.FusedQwen3(args, state, packed)
    c1, c2 = m.make_cache(48), m.make_cache(48)
    m.hidden(ids[:16], c1)
    m.hidden(ids[:16], c2)
    eager, graphed = Q.DecodeQwen3(m, head=False), Q.DecodeQwen3(m, graphs="step", head=False)
    for j in range(16, 30):
        a = eager.step(ids[j:j + 1], c1)
        b = graphed.step(ids[j:j + 1], c2).clone()
        torch.cuda.synchronize()
        assert c2[0].offset == j + 1
        assert rel(b, a) < 1e-2, (j, rel(b, a))
    assert rel(c2[1].k[:, :30], c1[1].k[:, :30]) < 1e-2 and float(c2[1].k[:, 30:].abs().max()) == 0.0


@pytest.mark.parametrize("L,pos,from_acc", [(1, 17, False), (70, 0, False), (33, 5, True)])
def test_fused_headnorm_rope_append_against_separate_ops(L, pos, from_acc):
    """scmx_qkv_headnorm_rope = qkv_headnorm (pinned bit-exactly elsewhere) + float32 rotary embedding + cache write:
    q and the written cache rows match the separate ops to bf16 rounding (sin / cos come from different routines);
    cache rows outside pos..pos+L-1 are untouched; a device-resident position gives the same bits as a host one."""
    from mxfp4_int8_m5_amd import sc_kernels as S
    hq, hk, d, rows = 4, 2, 128, 96
    g = torch.Generator(device="cuda").manual_seed(L)
    n = (hq + 2 * hk) * d
    qn = (1 + 0.1 * torch.randn(d, device="cuda", generator=g)).to(torch.bfloat16)
    kn = (1 + 0.1 * torch.randn(d, device="cuda", generator=g)).to(torch.bfloat16)
    inv_freq = 1.0 / (1e4 ** (torch.arange(d // 2, device="cuda", dtype=torch.float32) / (d // 2)))
    kw = {}
    if from_acc:
        acc = torch.randint(-20000, 20000, (L, n), device="cuda", dtype=torch.int32, generator=g)
        xs, ws = torch.rand(L, device="cuda", generator=g) * 1e-2, torch.rand(n, device="cuda", generator=g) * 1e-2
        y, kw = None, dict(acc=acc, xscale=xs, wscale=ws)
        q0, k0, v0 = S.qkv_epilogue_headnorm(acc, xs, ws, qn, kn, 1e-6, L, hq, hk, d)
    else:
        y = torch.randn(L, n, device="cuda", generator=g).to(torch.bfloat16)
        q0, k0, v0 = S.qkv_headnorm_y(y, qn, kn, 1e-6, L, hq, hk, d)

    def rope(x):
        ang = torch.arange(pos, pos + L, device="cuda", dtype=torch.float32)[:, None] * inv_freq[None]
        x1, x2 = x.float().chunk(2, -1)
        return torch.cat([x1 * ang.cos() - x2 * ang.sin(), x2 * ang.cos() + x1 * ang.sin()], -1).to(x.dtype)
    kc = torch.full((hk, rows, d), 7.0, device="cuda", dtype=torch.bfloat16)
    vc = torch.full((hk, rows, d), 7.0, device="cuda", dtype=torch.bfloat16)
    q = S.qkv_headnorm_rope(y, qn, kn, 1e-6, L, hq, hk, d, kc, vc, pos, inv_freq, **kw)
    assert rel(q, rope(q0)) < 4e-3 and rel(kc[:, pos:pos + L], rope(k0)) < 4e-3
    assert torch.equal(vc[:, pos:pos + L], v0)
    for c in (kc, vc):
        assert bool((c[:, :pos] == 7).all()) and bool((c[:, pos + L:] == 7).all())
    kc2, vc2 = torch.zeros_like(kc), torch.zeros_like(vc)
    qt = S.qkv_headnorm_rope(y, qn, kn, 1e-6, L, hq, hk, d, kc.clone(), vc.clone(), pos, inv_freq, token_major=True, **kw)
    assert qt.shape == q.shape and torch.equal(qt, q) and qt.transpose(0, 1).is_contiguous()    # same values, [L, hq, d] storage
    q2 = S.qkv_headnorm_rope(y, qn, kn, 1e-6, L, hq, hk, d, kc2, vc2, torch.tensor([pos], device="cuda"), inv_freq, **kw)
    assert torch.equal(q2, q) and torch.equal(kc2[:, pos:pos + L], kc[:, pos:pos + L])
    with pytest.raises(ValueError):
        S.qkv_headnorm_rope(y, qn, kn, 1e-6, L, hq, hk, d, kc, vc, rows - L + 1, inv_freq, **kw)


def test_headnorm_rope_many_rows_equal_few_rows_at_a_time():
    """Head dim 128 on many rows runs a kernel with sixteen lanes per head; a few rows run the general one (a wave per
    head).  Both must give the same bits: 70 rows at once against the same rows eight at a time, q and both caches,
    with the rotary embedding and (dense outputs) without."""
    from mxfp4_int8_m5_amd import sc_kernels as S
    hq, hk, d, rows, L, pos = 16, 8, 128, 128, 70, 9
    g = torch.Generator(device="cuda").manual_seed(3)
    n = (hq + 2 * hk) * d
    qn = (1 + 0.1 * torch.randn(d, device="cuda", generator=g)).to(torch.bfloat16)
    kn = (1 + 0.1 * torch.randn(d, device="cuda", generator=g)).to(torch.bfloat16)
    inv_freq = 1.0 / (1e6 ** (torch.arange(d // 2, device="cuda", dtype=torch.float32) / (d // 2)))
    y = (torch.randn(L, n, device="cuda", generator=g) * torch.rand(L, 1, device="cuda", generator=g) * 4).to(torch.bfloat16)
    kc, vc = (torch.zeros((hk, rows, d), device="cuda", dtype=torch.bfloat16) for _ in range(2))
    q = S.qkv_headnorm_rope(y, qn, kn, 1e-6, L, hq, hk, d, kc, vc, pos, inv_freq)
    kc2, vc2 = torch.zeros_like(kc), torch.zeros_like(vc)
    for r0 in range(0, L, 8):
        r1 = min(L, r0 + 8)
        qp = S.qkv_headnorm_rope(y[r0:r1].contiguous(), qn, kn, 1e-6, r1 - r0, hq, hk, d, kc2, vc2, pos + r0, inv_freq)
        assert torch.equal(qp, q[:, r0:r1])
    assert torch.equal(kc2, kc) and torch.equal(vc2, vc)
    q0, k0, v0 = S.qkv_headnorm_y(y, qn, kn, 1e-6, L, hq, hk, d)
    for r0 in range(0, L, 8):
        r1 = min(L, r0 + 8)
        qp, kp, vp = S.qkv_headnorm_y(y[r0:r1].contiguous(), qn, kn, 1e-6, r1 - r0, hq, hk, d)
        assert torch.equal(qp, q0[:, r0:r1]) and torch.equal(kp, k0[:, r0:r1]) and torch.equal(vp, v0[:, r0:r1])


@pytest.mark.parametrize("hq,hk,d,rows,n", [(16, 8, 128, 512, 129), (4, 4, 64, 40, 1), (8, 2, 256, 300, 300), (16, 8, 128, 8192, 5000),
                                            (16, 8, 128, 4096, 3000)])
def test_attn_decode_against_torch(hq, hk, d, rows, n):
    from mxfp4_int8_m5_amd import sc_kernels as S
    g = torch.Generator(device="cuda").manual_seed(n)
    q = torch.randn(hq, 1, d, device="cuda", generator=g).to(torch.bfloat16)
    kc = torch.randn(hk, rows, d, device="cuda", generator=g).to(torch.bfloat16)
    vc = torch.randn(hk, rows, d, device="cuda", generator=g).to(torch.bfloat16)
    rep = hq // hk
    ref = torch.nn.functional.scaled_dot_product_attention(
        q.float()[None], kc[:, :n].float().repeat_interleave(rep, 0)[None], vc[:, :n].float().repeat_interleave(rep, 0)[None])
    ref = ref[0].transpose(0, 1).reshape(1, hq * d)
    o = S.attn_decode(q, kc, vc, n)
    assert o.shape == (1, hq * d) and rel(o, ref) < 6e-3, rel(o, ref)
    o2 = S.attn_decode(q, kc, vc, torch.tensor([n - 1], device="cuda"), splits=S.attn_splits(n))   # position from device memory
    assert torch.equal(o2, o)
    for sp in (2, 7, 32):                                                      # rows cut into ranges, merged by a second kernel
        o3 = S.attn_decode(q, kc, vc, n, splits=sp)
        assert rel(o3, ref) < 6e-3 and rel(o3, o) < 3e-3, (sp, rel(o3, ref))
        assert torch.equal(S.attn_decode(q, kc, vc, torch.tensor([n - 1], device="cuda"), splits=sp), o3)
    with pytest.raises(ValueError):
        S.attn_decode(q, kc, vc, rows + 1)


@pytest.mark.parametrize("hq,hk,d,rows,pos", [(16, 8, 128, 512, 128), (4, 4, 64, 40, 0), (8, 2, 256, 300, 299),
                                               (32, 8, 128, 2048, 1500), (6, 3, 128, 64, 31)])
def test_attn_decode_qkv_equals_the_two_kernels(hq, hk, d, rows, pos):
    """Norm + rotary + append + attention in one launch: the attention output and the appended cache rows carry the
    same bits as qkv_headnorm_rope followed by attn_decode, with the position as an argument and from device memory;
    no other cache row is touched."""
    from mxfp4_int8_m5_amd import sc_kernels as S
    g = torch.Generator(device="cuda").manual_seed(pos + d)
    y = (torch.randn(1, (hq + 2 * hk) * d, device="cuda", generator=g) * 2).to(torch.bfloat16)
    qn = (1 + 0.1 * torch.randn(d, device="cuda", generator=g)).to(torch.bfloat16)
    kn = (1 + 0.1 * torch.randn(d, device="cuda", generator=g)).to(torch.bfloat16)
    inv_freq = (1e6 ** (-torch.arange(0, d, 2, dtype=torch.float32) / d)).cuda()
    kc = torch.randn(hk, rows, d, device="cuda", generator=g).to(torch.bfloat16)
    vc = torch.randn(hk, rows, d, device="cuda", generator=g).to(torch.bfloat16)
    k1, v1, k2, v2, k3, v3 = kc.clone(), vc.clone(), kc.clone(), vc.clone(), kc.clone(), vc.clone()
    q = S.qkv_headnorm_rope(y, qn, kn, 1e-6, 1, hq, hk, d, k1, v1, pos, inv_freq)
    ref = S.attn_decode(q, k1, v1, pos + 1)
    sp = S.attn_splits(pos + 1)                      # the same row ranges in every call: same summation order
    assert sp == (1 if pos < 1024 else 8)
    out = S.attn_decode_qkv(y, qn, kn, 1e-6, hq, hk, d, k2, v2, pos, inv_freq)
    assert torch.equal(out, ref)
    assert torch.equal(k2, k1) and torch.equal(v2, v1)
    assert not torch.equal(k2[:, pos], kc[:, pos])                       # the row was written
    out3 = S.attn_decode_qkv(y, qn, kn, 1e-6, hq, hk, d, k3, v3, torch.tensor([pos], device="cuda"), inv_freq, splits=sp)
    assert torch.equal(out3, ref) and torch.equal(k3, k1) and torch.equal(v3, v1)
    with pytest.raises(ValueError):
        S.attn_decode_qkv(y, qn, kn, 1e-6, hq, hk, d, k2, v2, rows, inv_freq)


@pytest.mark.parametrize("graphs", [False, True, "step"])
def test_fused_attention_decoder_equals_the_two_kernel_decoder(tiny, graphs):
    Q, args, state, packed = tiny
    ids = torch.randint(0, args.vocab_size, (22,), generator=torch.Generator().manual_seed(8)).cuda()
    m = Q.FusedQwen3(args, state, packed)
    c1, c2 = m.make_cache(32), m.make_cache(32)
    m.hidden(ids[:16], c1)
    m.hidden(ids[:16], c2)
    two, one = Q.DecodeQwen3(m, graphs=graphs, fuse_attn=False), Q.DecodeQwen3(m, graphs=graphs, fuse_attn=True)
    for j in range(16, 22):
        a = two.step(ids[j:j + 1], c1).clone()
        b = one.step(ids[j:j + 1], c2).clone()
        torch.cuda.synchronize()
        assert c1[0].offset == c2[0].offset == j + 1
        assert torch.equal(a, b), j
    assert all(torch.equal(x.k, z.k) and torch.equal(x.v, z.v) for x, z in zip(c1, c2))


@pytest.mark.parametrize("hq,hk,L,off,rows", [(16, 8, 2048, 0, 2048), (4, 4, 300, 0, 512), (8, 2, 70, 33, 128),
                                               (2, 1, 1, 0, 4), (6, 3, 129, 1000, 1200), (4, 2, 64, 64, 128)])
def test_attn_prefill_against_torch(hq, hk, L, off, rows):
    """Causal attention of L new tokens behind `off` cached ones (head dim 128): float32 softmax(q k^T) v of the same
    bf16 inputs in torch within 1e-2 (bf16 probabilities and output); ragged last query and key tiles, grouped
    heads, a cache longer than what is valid (rows past off + L hold NaN and must not be read into the result)."""
    from mxfp4_int8_m5_amd import sc_kernels as S
    d = 128
    g = torch.Generator(device="cuda").manual_seed(L + off)
    q = torch.randn(L, hq, d, device="cuda", generator=g).to(torch.bfloat16)
    kc = torch.randn(hk, rows, d, device="cuda", generator=g).to(torch.bfloat16)
    vc = torch.randn(hk, rows, d, device="cuda", generator=g).to(torch.bfloat16)
    kc[:, off + L:] = float("nan")
    vc[:, off + L:] = float("nan")
    n = off + L
    rep = hq // hk
    kf = kc[:, :n].float().repeat_interleave(rep, 0)
    vf = vc[:, :n].float().repeat_interleave(rep, 0)
    s = torch.einsum("lhd,hnd->hln", q.float(), kf) * d ** -0.5
    mask = torch.arange(n, device="cuda")[None, :] <= (off + torch.arange(L, device="cuda"))[:, None]
    p = torch.softmax(s.masked_fill(~mask[None], float("-inf")), -1)
    ref = torch.einsum("hln,hnd->lhd", p, vf).reshape(L, hq * d)
    o = S.attn_prefill(q.transpose(0, 1), kc, vc, off)          # the [hq, L, d] view, as the norm kernel hands it over
    assert o.shape == (L, hq * d) and not torch.isnan(o).any()
    assert rel(o, ref) < 1e-2, rel(o, ref)
    assert torch.equal(S.attn_prefill(q.transpose(0, 1).contiguous(), kc, vc, off), o)     # head-major storage: copied
    with pytest.raises(ValueError):
        S.attn_prefill(q.transpose(0, 1), kc, vc, rows - L + 1)


def test_packed_output_head(tiny):
    """head="packed": logits through the W4A8 GEMV on the quantized output projection, against the bf16 head."""
    Q, args, state, packed = tiny
    ids = torch.randint(0, args.vocab_size, (12,), generator=torch.Generator().manual_seed(7)).cuda()
    m = Q.FusedQwen3(args, state, packed)
    c1, c2 = m.make_cache(32), m.make_cache(32)
    m.hidden(ids[:11], c1)
    m.hidden(ids[:11], c2)
    a = Q.DecodeQwen3(m).step(ids[11:], c1)
    b = Q.DecodeQwen3(m, head="packed").step(ids[11:], c2)
    assert b.shape == a.shape and rel(b, a) < 0.15      # 4-bit weights on a 256-wide hidden state
    assert int(a.argmax()) == int(b.argmax()) or rel(b, a) < 0.1


def test_packed_output_head_of_a_family_format_model(tiny, tmp_path):
    """The packed head keeps the published format when the model's layers use another one (16-blocks, 4-bit block
    codes), whether the decoder is built before or after the model's first pass selected its format."""
    Q, args, state, packed = tiny
    ckpt, cache_dir = str(tmp_path / "tiny-qwen3"), str(tmp_path / "cache")
    _write_checkpoint(ckpt, args, state)
    ids = torch.randint(0, args.vocab_size, (12,), generator=torch.Generator().manual_seed(8)).cuda()
    m, _ = Q.load_fused(ckpt, cache_dir, packed="fmt:e2m1/B16/M1..10")
    early = Q.DecodeQwen3(m, head="packed")                   # built before any pass set the model's format
    c0, c1, c2 = m.make_cache(32), m.make_cache(32), m.make_cache(32)
    for c in (c0, c1, c2):
        m.hidden(ids[:11], c)
    late = Q.DecodeQwen3(m, head="packed")                    # built after
    a = Q.DecodeQwen3(m).step(ids[11:], c0)
    b = early.step(ids[11:], c1)
    c = late.step(ids[11:], c2)
    assert torch.equal(b, c)
    assert rel(b, a) < 0.15


def test_one_decoder_over_successive_caches(tiny):
    """A decoder with captured graphs used for one prompt after another, each with a cache of its own: every step equals
    the eager decoder's on the same cache content, and graphs of a released cache are dropped."""
    import gc
    Q, args, state, packed = tiny
    gen = torch.Generator().manual_seed(9)
    m = Q.FusedQwen3(args, state, packed)
    for graphs in (True, "step"):
        dec, eager = Q.DecodeQwen3(m, graphs=graphs), Q.DecodeQwen3(m)
        for prompt in range(4):
            ids = torch.randint(0, args.vocab_size, (14,), generator=gen).cuda()
            c1, c2 = m.make_cache(32), m.make_cache(32)
            m.hidden(ids[:10], c1)
            m.hidden(ids[:10], c2)
            for j in range(10, 14):
                a = eager.step(ids[j:j + 1], c1)
                b = dec.step(ids[j:j + 1], c2)
                torch.cuda.synchronize()
                assert rel(b, a) < 1e-2, (graphs, prompt, j)
            kept = b
            if prompt % 2:
                dec.release(c2)
                assert not any(e[3] is c2 or any(e[3] is c for c in c2) for e in dec.graphs.values())
            del c1, c2
            gc.collect()
        assert torch.equal(kept, b)            # returned logits are not aliased by later steps


def _write_checkpoint(path, args, state):
    import dataclasses
    import json
    import os
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    cfg = dataclasses.asdict(args)
    cfg.update(model_type="qwen3", architectures=["Qwen3ForCausalLM"])
    with open(os.path.join(path, "config.json"), "w") as fh:
        json.dump(cfg, fh)
    keys = sorted(state)
    half = len(keys) // 2   # two shards, as large checkpoints come
    save_file({k: state[k].to(torch.bfloat16).contiguous() for k in keys[:half]}, os.path.join(path, "model-00001-of-00002.safetensors"))
    save_file({k: state[k].to(torch.bfloat16).contiguous() for k in keys[half:]}, os.path.join(path, "model-00002-of-00002.safetensors"))


def test_load_fused_from_a_checkpoint_directory(tiny, tmp_path):
    """config.json + sharded safetensors on disk -> packed on the device on first use (byte-shift cache, the
    reference's file layout), read back from the cache on the second; both equal the model quantized in memory."""
    import os
    from safetensors.numpy import load_file
    Q, args, state, packed = tiny
    ckpt, cache_dir = str(tmp_path / "tiny-qwen3"), str(tmp_path / "cache")
    _write_checkpoint(ckpt, args, state)
    ids = torch.randint(0, args.vocab_size, (50,), generator=torch.Generator().manual_seed(11)).cuda()
    ref = Q.FusedQwen3(args, state, packed).hidden(ids)
    m1, tok = Q.load_fused(ckpt, cache_dir)
    assert tok is None and m1.args == args
    cache = os.path.join(cache_dir, "tiny-qwen3-scmxfp4.safetensors")
    flat = load_file(cache)
    key = "layers.1.mlp.down_proj"
    assert flat[key + ".shifts"].shape == (256, 512 // 32) and flat[key + ".shifts"].max() <= 3
    assert flat[key + ".codes"].dtype == np.uint32 and flat[key + ".wscale"].dtype == np.float32
    assert torch.equal(m1.hidden(ids), ref)
    stamp = os.path.getmtime(cache)
    m2, _ = Q.load_fused(ckpt, cache_dir, resident=True, epilogue="row")
    assert os.path.getmtime(cache) == stamp                      # second use reads the cache
    assert rel(m2.hidden(ids), ref) < 1e-2
    with pytest.raises(FileNotFoundError):
        Q.load_fused(ckpt, cache_dir, packed="gptq")
    with pytest.raises(NotImplementedError):
        Q.load_fused(ckpt, cache_dir, packed="rot:e2m1/B32/pow2")


def test_load_fused_in_a_family_format(tiny, tmp_path):
    import os
    Q, args, state, packed = tiny
    ckpt, cache_dir = str(tmp_path / "tiny-qwen3"), str(tmp_path / "cache")
    _write_checkpoint(ckpt, args, state)
    ids = torch.randint(0, args.vocab_size, (40,), generator=torch.Generator().manual_seed(12)).cuda()
    member = "e2m1/B16/M1..10"
    m, _ = Q.load_fused(ckpt, cache_dir, packed="fmt:" + member)
    assert os.path.exists(os.path.join(cache_dir, "tiny-qwen3-fmt-e2m1_B16_M110.safetensors"))
    assert m.fmt.block == 16 and m.fmt.bc_bits == 4
    ref = Q.FusedQwen3(args, state, packed).hidden(ids)
    assert rel(m.hidden(ids), ref) < 0.25                        # two different 4-bit quantizations of one model
    m_again, _ = Q.load_fused(ckpt, cache_dir, packed="fmt:" + member)
    assert torch.equal(m_again.hidden(ids), m.hidden(ids))


# ---- OLMoE ---------------------------------------------------------------------------------------------------------

@pytest.fixture(scope="module")
def tiny_moe():
    return make_tiny_moe(4)


def make_tiny_moe(heads):
    from mxfp4_int8_m5_amd import fused_olmoe as O, sc_weights as W
    args = O.OlmoeArgs(hidden_size=256, intermediate_size=128, num_hidden_layers=2, num_attention_heads=heads,
                       num_experts=8, num_experts_per_tok=2, vocab_size=300)
    g = torch.Generator().manual_seed(10)
    rnd = lambda *s, sc=1.0: torch.randn(*s, generator=g) * sc   # noqa: E731
    D, Fi, E = args.hidden_size, args.intermediate_size, args.num_experts
    state = {"model.embed_tokens.weight": rnd(args.vocab_size, D), "model.norm.weight": 1 + rnd(D, sc=0.1),
             "lm_head.weight": rnd(args.vocab_size, D, sc=D ** -0.5)}
    lin = {}
    for i in range(2):
        p = f"model.layers.{i}."
        for n in ("input_layernorm", "post_attention_layernorm", "self_attn.q_norm", "self_attn.k_norm"):
            state[p + n + ".weight"] = 1 + rnd(D, sc=0.1)
        state[p + "mlp.gate.weight"] = rnd(E, D, sc=4 * D ** -0.5)       # a decisive router
        for n in O.ATTN:
            lin[f"layers.{i}.{n}"] = rnd(D, D, sc=D ** -0.5)
        lin[f"layers.{i}.experts.gate_proj"] = rnd(E, Fi, D, sc=D ** -0.5)
        lin[f"layers.{i}.experts.up_proj"] = rnd(E, Fi, D, sc=D ** -0.5)
        lin[f"layers.{i}.experts.down_proj"] = rnd(E, D, Fi, sc=Fi ** -0.5)
    state = {k: v.to(torch.bfloat16).float() for k, v in state.items()}
    flat = W.pack_weights(lin)
    packed = {k[:-len(".codes")]: (flat[k], flat[k[:-5] + "bcodes"], flat[k[:-5] + "wscale"]) for k in flat if k.endswith(".codes")}
    return O, args, state, packed


def moe_float_model(args, state, packed, ids, routing):
    """float32 torch on the CPU with the dequantized weights, no activation quantization, and the routing decisions
    of the run under test (a near-tie in the router would otherwise send a token to other experts)."""
    from oracle import layout
    a = args
    H, d, eps, E = a.num_attention_heads, a.head_dim, a.rms_norm_eps, a.num_experts

    def weight(key):
        c, b, s = packed[key]
        rows = s.shape[0]
        return torch.from_numpy(layout.decode(c, b, rows, c.size * 8 // rows).astype(np.float32) * s[:, None])

    def norm(x, w):
        return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * w

    def rope(x):
        L, half = x.shape[1], d // 2
        ang = torch.arange(L, dtype=torch.float32)[:, None] * (1.0 / (a.rope_theta ** (torch.arange(half).float() / half)))[None]
        x1, x2 = x.chunk(2, -1)
        return torch.cat([x1 * ang.cos() - x2 * ang.sin(), x2 * ang.cos() + x1 * ang.sin()], -1)

    h = state["model.embed_tokens.weight"][ids]
    L = h.shape[0]
    for i in range(a.num_hidden_layers):
        p, lk = f"model.layers.{i}.", f"layers.{i}."
        x = norm(h, state[p + "input_layernorm.weight"])
        q = norm(x @ weight(lk + "self_attn.q_proj").T, state[p + "self_attn.q_norm.weight"]).view(L, H, d).transpose(0, 1)
        k = norm(x @ weight(lk + "self_attn.k_proj").T, state[p + "self_attn.k_norm.weight"]).view(L, H, d).transpose(0, 1)
        v = (x @ weight(lk + "self_attn.v_proj").T).view(L, H, d).transpose(0, 1)
        o = torch.nn.functional.scaled_dot_product_attention(rope(q)[None], rope(k)[None], v[None], is_causal=True)[0]
        h = h + o.transpose(0, 1).reshape(L, -1) @ weight(lk + "self_attn.o_proj").T
        x = norm(h, state[p + "post_attention_layernorm.weight"])
        inds, scores = (t.cpu() for t in routing[i])
        y = torch.zeros_like(h)
        for t in range(L):
            for j in range(inds.shape[1]):
                e = int(inds[t, j])
                g = x[t] @ weight(f"{lk}experts.gate_proj.{e}").T
                u = x[t] @ weight(f"{lk}experts.up_proj.{e}").T
                y[t] += float(scores[t, j]) * ((torch.nn.functional.silu(g) * u) @ weight(f"{lk}experts.down_proj.{e}").T)
        h = h + y
    return norm(h, state["model.norm.weight"])


@pytest.mark.parametrize("kw", [dict(tile=64), dict(tile=256, two_pass=True), dict(tile=128, sort="argsort"), dict()])
def test_olmoe_prefill_against_float_model(tiny_moe, kw):
    O, args, state, packed = tiny_moe
    ids = torch.randint(0, args.vocab_size, (45,), generator=torch.Generator().manual_seed(11))
    m = O.FusedOlmoe(args, state, packed, **kw)
    m.record = []
    h = m.hidden(ids.cuda())
    ref = moe_float_model(args, state, packed, ids, m.record)
    assert rel(h, ref) < 4e-2, rel(h, ref)


def test_olmoe_prefill_from_blocked_activations_gives_the_same_bits(tiny_moe, monkeypatch):
    """The attention output projection of a long prompt reads blocked activations; forced on for the small model, the
    hidden states are those of the row layout bit for bit."""
    from mxfp4_int8_m5_amd import sc_kernels as S
    O, args, state, packed = tiny_moe
    ids = torch.randint(0, args.vocab_size, (90,), generator=torch.Generator().manual_seed(14)).cuda()
    m = O.FusedOlmoe(args, state, packed, tile=64)
    by_rows = m.hidden(ids)
    seen = []
    real = S.act_quant_blocked
    monkeypatch.setattr(S, "prefers_blocked", lambda M, N, K: True)
    monkeypatch.setattr(S, "act_quant_blocked", lambda *a, **k: (seen.append(1), real(*a, **k))[1])
    assert torch.equal(m.hidden(ids), by_rows) and len(seen) == args.num_hidden_layers


def test_olmoe_prefill_with_head_dim_128():
    """Two heads of 128: the prefill attention runs through scmx_attn_prefill (q copied to token-major first)."""
    O, args, state, packed = make_tiny_moe(2)
    ids = torch.randint(0, args.vocab_size, (70,), generator=torch.Generator().manual_seed(13))
    m = O.FusedOlmoe(args, state, packed, tile=64)
    m.record = []
    h = m.hidden(ids.cuda())
    assert rel(h, moe_float_model(args, state, packed, ids, m.record)) < 4e-2


@pytest.mark.parametrize("fuse", [False, "o", True])
def test_olmoe_decode_continues_the_prefill(tiny_moe, fuse):
    O, args, state, packed = tiny_moe
    ids = torch.randint(0, args.vocab_size, (30,), generator=torch.Generator().manual_seed(12)).cuda()
    m = O.FusedOlmoe(args, state, packed, tile=64)
    full = m.hidden(ids)
    cache = m.make_cache(64)
    m.hidden(ids[:27], cache)
    dec = O.DecodeOlmoe(m, fuse_prologue=fuse, head=False)
    rows = torch.cat([dec.step(ids[27 + j:28 + j], cache) for j in range(3)])
    assert rel(rows, full[27:]) < 3e-2, rel(rows, full[27:])
    logits = O.DecodeOlmoe(m).step(ids[:1], m.make_cache(8))
    assert logits.shape == (1, args.vocab_size)


@pytest.mark.parametrize("renorm", [False, True])
def test_olmoe_kernel_router_against_array_op_routing(tiny_moe, renorm):
    """The router kernel lists a token's experts by falling probability (ties by rising index); the array-op routing it
    replaced (softmax in float32 -> bf16, `topk(sorted=False)`, optional renormalisation: the reference's
    e2e/fused_olmoe.py:183-192 with argpartition's order) leaves the order open.  The weighted combine adds the slots
    one after another in bf16, so the order can move the last bit of a sum and nothing more: the same experts are
    chosen for every token, with the same scores, and the block outputs of the two routings differ by bf16 rounding."""
    import types
    O, args, state, packed = tiny_moe
    args = O.OlmoeArgs(**{**args.__dict__, "norm_topk_prob": renorm})
    ids = torch.randint(0, args.vocab_size, (60,), generator=torch.Generator().manual_seed(21)).cuda()
    m = O.FusedOlmoe(args, state, packed, tile=64)
    m.record = []
    h_kernel = m.hidden(ids)
    kernel_routing = [(i.clone(), s.clone()) for i, s in m.record]

    def array_route(self, nw, xn, M):
        logits = xn[:M] @ nw["mlp.gate"].T
        p = torch.softmax(logits.float(), -1).to(torch.bfloat16)
        scores, inds = torch.topk(p, self.args.num_experts_per_tok, dim=-1, sorted=False)
        if self.args.norm_topk_prob:
            scores = scores / scores.sum(-1, keepdim=True)
        return inds.to(torch.int32), scores

    m2 = O.FusedOlmoe(args, state, packed, tile=64)
    m2.route = types.MethodType(array_route, m2)
    m2.record = []
    h_array = m2.hidden(ids)
    # layer 0 sees identical inputs: same expert sets, same score per chosen expert
    (ik, sk), (ia, sa) = kernel_routing[0], m2.record[0]
    order_k, order_a = ik.long().argsort(-1), ia.long().argsort(-1)
    assert torch.equal(ik.long().gather(-1, order_k), ia.long().gather(-1, order_a))
    dk, da = sk.float().gather(-1, order_k), sa.float().gather(-1, order_a)
    assert float((dk - da).abs().max()) <= 2.0 ** -7 * float(da.abs().max())          # one bf16 step at most
    assert rel(h_kernel, h_array) < 1e-2, rel(h_kernel, h_array)
