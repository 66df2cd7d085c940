"""Mixture-of-experts parity on the GPU through the C ABI: token sort contract, grouped GEMM against per-expert
float64 integer GEMMs (uneven segments, empty experts), epilogues, the two-pass variant, the weighted combine.
Mirrors e2e/sc_moe.py:209-244 and e2e/test_sc_kernels.py:190-205."""
import numpy as np
import pytest
import torch

from oracle import bf16, layout, linear, moe
from tests.util import FORMATS, dev, host, llm_acts, product_format, random_packed

pytestmark = pytest.mark.gpu
F32 = np.float32


@pytest.fixture(scope="module")
def M():
    from mxfp4_int8_m5_amd import sc_moe
    return sc_moe


def skewed_routing(rng, tokens, experts, topk):
    """softmax(N(0,1) logits + N(0,1.5) expert bias) -> top-k experts and renormalised bf16 scores."""
    logits = rng.standard_normal((tokens, experts)) + rng.standard_normal(experts) * 1.5
    p = np.exp(logits - logits.max(1, keepdims=True))
    p /= p.sum(1, keepdims=True)
    inds = np.argsort(-p, axis=1)[:, :topk]
    sc = np.take_along_axis(p, inds, 1)
    sc /= sc.sum(1, keepdims=True)
    return inds.astype(np.int32), bf16.to_bits(sc.astype(F32))


@pytest.mark.parametrize("m,topk,e,tm", [(75, 8, 8, 64), (4096, 8, 64, 128), (2048, 9, 257, 64), (1, 8, 64, 64),
                                         (300, 1, 1024, 128), (1000, 5, 1024, 64), (515, 8, 300, 128)])
def test_route_sort_contract(M, m, topk, e, tm):
    rng = np.random.default_rng(m + e)
    inds, _ = skewed_routing(rng, m, e, topk)
    if e == 8:
        inds[inds == 3] = 2          # an empty expert
    pos, tok, es, off, ts, mt = M.route_sort(dev(inds), e, tm)
    moe.check_route_sort(inds, e, tm, host(pos), host(tok), host(es), host(off), host(ts))
    assert mt == -(-m * topk // tm) + e
    ro = moe.route_sort(inds, e, tm)
    assert np.array_equal(host(off), ro[3]) and np.array_equal(host(ts), ro[4]) and np.array_equal(host(es), ro[2])
    o2, t2, mt2 = M.segments(es, e, tm)
    assert np.array_equal(host(o2), ro[3]) and np.array_equal(host(t2), ro[4]) and mt2 == mt


@pytest.mark.parametrize("m,e,k,renorm,shared", [(4096, 64, 8, True, False), (2048, 256, 8, True, True), (4096, 64, 8, False, False),
                                                 (1, 64, 8, True, False), (77, 257, 9, True, False), (300, 1000, 64, False, True), (40, 1024, 3, True, False),
                                                 (129, 8, 8, True, True), (50, 5, 1, True, False),
                                                 # the sizes either side of each build of the kernel (1, 2, 4, 8, 16 experts per lane)
                                                 (33, 65, 4, True, False), (20, 128, 8, True, True), (10, 129, 2, False, False),
                                                 (12, 512, 8, True, False), (9, 513, 6, True, True)])
def test_router_against_oracle(M, m, e, k, renorm, shared):
    """Softmax -> top-k -> renormalisation (-> shared-expert slot with its sigmoid gate) on config 3 / config 4 router
    logits (N(0,1) + N(0,1.5) expert bias, bf16): expert indices and bf16 scores bit for bit against the oracle
    (e2e/fused_olmoe.py:183-192, e2e/fused_qwen35.py:171-180)."""
    rng = np.random.default_rng(m + e + k)
    lb = bf16.to_bits((rng.standard_normal((m, e)) + rng.standard_normal(e) * 1.5).astype(F32))
    if m > 4:
        lb[1] = lb[1, 0]                      # a token with all-equal logits: ties resolved by rising index
        lb[2, : e // 2] = lb[2, 0]
    gl = bf16.to_bits((rng.standard_normal(m) * 3).astype(F32)) if shared else None
    inds, scores = M.route(dev(lb), k, renorm=renorm, shared_logit=None if gl is None else dev(gl))
    ri, rs = moe.route(lb, k, renorm, gl)
    assert np.array_equal(host(inds), ri)
    assert np.array_equal(host(scores), rs)
    # and the result feeds the sort: every token's slots are distinct experts
    pos, tok, es, off, ts, mt = M.route_sort(inds, e + int(shared), 64)
    moe.check_route_sort(ri, e + int(shared), 64, host(pos), host(tok), host(es), host(off), host(ts))


def test_router_bad_arguments(M):
    lg = torch.zeros((4, 2000), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ValueError):
        M.route(lg, 8)                         # more than 1024 experts
    with pytest.raises(ValueError):
        M.route(lg[:, :4].contiguous(), 8)     # k > E


@pytest.mark.parametrize("tm", [64, 128, 256])
def test_grouped_gemm_uneven_segments(M, tm):
    """8 experts, 600 rows, experts 3 and 7 empty (e2e/sc_moe.py:213-215): INT32 exact, EPI 1 and 3 bit-exact,
    two-pass variant identical."""
    rng = np.random.default_rng(0)
    e, n, k, r = 8, 256, 512, 600
    ex = np.sort(rng.choice(e - 1, r, p=np.r_[0.4, np.full(e - 2, 0.6 / (e - 2))])).astype(np.int32)
    ex[ex == 3] = 2
    packs = [layout.quantize(rng.standard_normal((n, k)) * 0.02) for _ in range(e)]
    codes, bc, ws = (np.stack([p[i] for p in packs]) for i in range(3))
    wq = np.stack([p[3] for p in packs])
    xq = rng.integers(-127, 128, (r, k)).astype(np.int8)
    xs = (np.abs(rng.standard_normal(r)) * 1e-2).astype(F32)
    ref = moe.moe_int_gemm(xq, ex, wq)
    off, tstart, mt = M.segments(dev(ex), e, tm)
    dc, db, dw = dev(codes), dev(bc), dev(ws)
    acc = host(M.moe_mm(dev(xq), r, dc, db, dw, off, tstart, mt, n, 0, tile=(tm, 64, 4)))
    assert np.array_equal(acc, ref)
    y1 = host(M.moe_mm(dev(xq), r, dc, db, dw, off, tstart, mt, n, 1, dev(xs), tile=(tm, 64, 4)))
    assert np.array_equal(y1, moe.moe_epilogue(ref, xs, ws, ex, 1))
    y3 = host(M.moe_mm(dev(xq), r, dc, db, dw, off, tstart, mt, n, 3, dev(xs), tile=(tm, 64, 4)))
    assert np.array_equal(y3, moe.moe_epilogue(ref, xs, ws, ex, 3))
    wq8 = M.unpack_experts(dc, db, n, k)
    assert np.array_equal(host(wq8), wq.reshape(e * n, k))
    acc2 = host(M.moe_mm_i8(dev(xq), r, wq8, dw, off, tstart, mt, n, 0, tile=(tm, 64, 4)))
    assert np.array_equal(acc2, ref)


@pytest.mark.parametrize("i", range(len(FORMATS)))
def test_grouped_gemm_formats(M, i):
    """Two experts with the same random-code weights, uneven segments (e2e/test_formats.py:46-52)."""
    fmt = FORMATS[i]
    rng = np.random.default_rng(80 + i)
    n, k, m = 256, 2048, 128
    codes, bc, ws, q = random_packed(rng, n, k, fmt)
    xq = rng.integers(-127, 128, (m, k)).astype(np.int8)
    ex = np.sort(rng.integers(0, 2, m)).astype(np.int32)
    off, tstart, mt = M.segments(dev(ex), 2, 64)
    acc = host(M.moe_mm(dev(xq), m, dev(np.stack([codes, codes])), dev(np.stack([bc, bc])), dev(np.stack([ws, ws])),
                        off, tstart, mt, n, 0, fmt=product_format(fmt)))
    assert np.array_equal(acc, linear.int_gemm(xq, q))


def test_moe_block_with_fused_gather_and_combine(M):
    """A whole expert block at reduced width: route_sort -> grouped gate|up GEMM with SwiGLU reading token rows through
    `gather` -> act_quant -> grouped down GEMM -> weighted combine; every stage against the oracle, and the result
    independent of the order inside the segments."""
    from mxfp4_int8_m5_amd import sc_kernels as S
    rng = np.random.default_rng(3)
    tokens, e, topk, d, f, tm = 300, 16, 4, 256, 128, 64
    inds, scores = skewed_routing(rng, tokens, e, topk)
    gu = [random_packed(rng, 2 * f, d) for _ in range(e)]
    dn = [random_packed(rng, d, f) for _ in range(e)]
    perm = linear.interleave_gate_up(f)
    gc = np.stack([p[0].reshape(2 * f, -1)[perm].reshape(-1) for p in gu])
    gb = np.stack([p[1][perm] for p in gu])
    gw = np.stack([p[2][perm] for p in gu])
    gq = np.stack([p[3][perm] for p in gu])
    dcodes, dbc, dws, dq = (np.stack([p[i] for p in dn]) for i in range(4))
    xb = bf16.to_bits(rng.standard_normal((tokens, d)).astype(F32))
    res = bf16.to_bits(rng.standard_normal((tokens, d)).astype(F32))
    # GPU
    xq, xs = S.act_quant(dev(xb), Mp=tokens)
    pos, tok, es, off, ts, mt = M.route_sort(dev(inds), e, tm)
    r = tokens * topk
    act = M.moe_mm(xq, r, dev(gc), dev(gb), dev(gw), off, ts, mt, 2 * f, 3, xs, tile=(tm, 64, 4), gather=tok)
    aq, as_ = S.act_quant(act, Mp=r)
    yd = M.moe_mm(aq, r, dev(dcodes), dev(dbc), dev(dws), off, ts, mt, d, 1, as_, tile=(tm, 64, 4))
    h, _, _ = M.moe_combine(yd, pos, dev(scores), dev(res), None, None, tokens, quant=False)
    # oracle, with the GPU's own permutation (the order inside a segment is free)
    pos_h, tok_h, es_h = host(pos), host(tok)[:r], host(es)
    moe.check_route_sort(inds, e, tm, pos_h, host(tok), es_h, host(off), host(ts))
    rq, rs = linear.act_quant(bf16.from_bits(xb))
    acc1 = moe.moe_int_gemm(rq[tok_h], es_h, gq)
    act_ref = moe.moe_epilogue(acc1, rs[tok_h], gw, es_h, 3)
    assert np.array_equal(host(act), act_ref)
    aq_ref, as_ref = linear.act_quant(bf16.from_bits(act_ref))
    yd_ref = moe.moe_epilogue(moe.moe_int_gemm(aq_ref, es_h, dq), as_ref, dws, es_h, 1)
    assert np.array_equal(host(yd), yd_ref)
    h_ref = moe.combine(yd_ref, pos_h, scores, res, tokens)
    assert np.array_equal(host(h), h_ref)
    # the same block from the oracle's stable sort gives the same residual stream
    p2, t2, e2, *_ = moe.route_sort(inds, e, tm)
    a2 = moe.moe_epilogue(moe.moe_int_gemm(rq[t2[:r]], e2, gq), rs[t2[:r]], gw, e2, 3)
    q2, s2 = linear.act_quant(bf16.from_bits(a2))
    y2 = moe.moe_epilogue(moe.moe_int_gemm(q2, e2, dq), s2, dws, e2, 1)
    assert np.array_equal(moe.combine(y2, p2, scores, res, tokens), h_ref)


def test_combine_with_next_norm_and_split(M):
    rng = np.random.default_rng(2)
    m, mp, topk, k = 200, 256, 8, 2048
    inds = np.stack([rng.permutation(64)[:topk] for _ in range(m)]).astype(np.int32)
    pos, *_ = moe.route_sort(inds, 64, 64)
    y = bf16.to_bits(rng.standard_normal((m * topk, k)).astype(F32))
    sc = bf16.to_bits(np.abs(rng.standard_normal((m, topk))).astype(F32) * 0.2)
    res = bf16.to_bits((rng.standard_normal((mp, k)) * 2).astype(F32))
    nw = bf16.to_bits(rng.lognormal(0, 0.3, k).astype(F32))
    h, xq, xs = M.moe_combine(dev(y), dev(pos), dev(sc), dev(res), dev(nw), 1e-5, m)
    h_ref = moe.combine(y, pos, sc, res, m)
    assert np.array_equal(host(h), h_ref)
    rq, rs, _ = linear.rmsnorm_quant(h_ref, nw, 1e-5)
    assert np.array_equal(host(xq), rq) and np.array_equal(host(xs), rs)
    h2, _, _ = M.moe_combine_split(dev(y), dev(pos), dev(np.ascontiguousarray(sc[:, :-1])),
                                   dev(np.ascontiguousarray(sc[:, -1])), dev(res), None, None, m)
    assert np.array_equal(host(h2), h_ref)


def test_config3_olmoe_shape_property(M):
    """BASELINE config 3 at full size (64 experts, top-8, 4096 tokens, hidden 2048): the grouped INT32 accumulators
    of the down projection (K = 1024) for every row against per-expert float64 GEMMs."""
    rng = np.random.default_rng(33)
    tokens, e, topk, d, f = 4096, 64, 8, 2048, 1024
    inds, _ = skewed_routing(rng, tokens, e, topk)
    codes1, bc1, ws1, q1 = random_packed(rng, d, f)
    shift = rng.integers(0, e)
    # per-expert weights: rows of one random matrix rolled by the expert index (cheap to build, all experts differ)
    codes = np.stack([np.roll(codes1.reshape(d, -1), ex + shift, 0).reshape(-1) for ex in range(e)])
    bc = np.stack([np.roll(bc1, ex + shift, 0) for ex in range(e)])
    ws = np.stack([np.roll(ws1, ex + shift, 0) for ex in range(e)])
    wq = np.stack([np.roll(q1, ex + shift, 0) for ex in range(e)])
    r = tokens * topk
    xq = rng.integers(-127, 128, (r, f)).astype(np.int8)
    pos, tok, es, off, ts, mt = M.route_sort(dev(inds), e, 128)
    acc = host(M.moe_mm(dev(xq), r, dev(codes), dev(bc), dev(ws), off, ts, mt, d, 0, tile=(128, 64, 4)))
    assert np.array_equal(acc, moe.moe_int_gemm(xq, host(es), wq))


def test_config3_pipeline_as_benchmarked(M):
    """BASELINE config 3 at full size through the launches the benchmark times: 4096 tokens, 64 experts, top-8, hidden
    2048, intermediate 1024, row tile 256: act_quant -> route_sort -> grouped gate|up GEMM reading token rows through
    `gather` with the SwiGLU epilogue -> act_quant -> grouped down GEMM -> weighted combine (mirrors
    e2e/fused_olmoe.py:207-245, checked like e2e/sc_moe.py:209-244).  The stages of the busiest, the emptiest non-empty
    and a median expert bit for bit against the oracle; all 32768 rows independent of the row tile (64 vs 256); the
    combine of all 4096 tokens against the oracle's sequential bf16 sum."""
    from mxfp4_int8_m5_amd import sc_kernels as S
    rng = np.random.default_rng(3)
    T, E, topk, D, Fi = 4096, 64, 8, 2048, 1024
    R = T * topk
    inds, scores = skewed_routing(rng, T, E, topk)
    perm = linear.interleave_gate_up(Fi)
    gu, dn = [], []
    for _ in range(E):
        c4 = rng.integers(0, 16, (2 * Fi, D), dtype=np.uint8)
        b = rng.integers(0, 4, (2 * Fi, D // 32), dtype=np.uint8)
        gu.append(layout.pack_rows(c4[perm], b[perm], np.exp2(rng.integers(-12, -6, 2 * Fi)).astype(F32)))
        c4 = rng.integers(0, 16, (D, Fi), dtype=np.uint8)
        b = rng.integers(0, 4, (D, Fi // 32), dtype=np.uint8)
        dn.append(layout.pack_rows(c4, b, np.exp2(rng.integers(-12, -6, D)).astype(F32)))
    gc, gb, gw = (dev(np.stack([p[i] for p in gu])) for i in range(3))
    dc, db, dw = (dev(np.stack([p[i] for p in dn])) for i in range(3))
    xb, x = llm_acts(rng, T, D)
    res = bf16.to_bits(rng.standard_normal((T, D)).astype(F32))
    xq, xs = S.act_quant(dev(xb), Mp=T)
    outs = {}
    for tm in (64, 256):
        pos, tok, es, off, ts, mt = M.route_sort(dev(inds), E, tm)
        moe.check_route_sort(inds, E, tm, host(pos), host(tok), host(es), host(off), host(ts))
        act = M.moe_mm(xq, R, gc, gb, gw, off, ts, mt, 2 * Fi, 3, xs, tile=(tm, 64, 4), gather=tok)
        aq, as_ = S.act_quant(act, Mp=R)
        yd = M.moe_mm(aq, R, dc, db, dw, off, ts, mt, D, 1, as_, tile=(tm, 64, 4))
        h, _, _ = M.moe_combine(yd, pos, dev(scores), dev(res), None, None, T, quant=False)
        outs[tm] = (host(act)[host(pos)], host(yd)[host(pos)], host(h))
    for a, b in zip(outs[64], outs[256]):
        assert np.array_equal(a, b)
    # the last pass is the benchmark's (row tile 256): its stages against the oracle on three experts
    pos_h, off_h, tok_h = host(pos), host(off), host(tok)[:R]
    counts = np.diff(off_h)
    assert counts.sum() == R
    rq, rs = linear.act_quant(x)
    assert np.array_equal(host(xq), rq) and np.array_equal(host(xs), rs)
    act_h, yd_h, aq_h, as_h = host(act), host(yd), host(aq), host(as_)
    order = np.argsort(counts)
    nonempty = order[counts[order] > 0]
    for e in (int(nonempty[-1]), int(nonempty[0]), int(nonempty[len(nonempty) // 2])):
        rows = slice(off_h[e], off_h[e + 1])
        t = tok_h[rows]
        q_gu = layout.decode(gu[e][0], gu[e][1], 2 * Fi, D)
        a_ref = linear.epilogue(linear.int_gemm(rq[t], q_gu), rs[t], gu[e][2], 3)
        assert np.array_equal(act_h[rows], a_ref), e
        q2, s2 = linear.act_quant(bf16.from_bits(a_ref))
        assert np.array_equal(aq_h[rows], q2) and np.array_equal(as_h[rows], s2), e
        q_dn = layout.decode(dn[e][0], dn[e][1], D, Fi)
        assert np.array_equal(yd_h[rows], linear.epilogue(linear.int_gemm(q2, q_dn), s2, dn[e][2], 1)), e
    assert np.array_equal(outs[256][2], moe.combine(yd_h, pos_h, scores, res, T))


def test_config4_sparse_moe_full_size(M):
    """BASELINE config 4 at its real shape: 256 routed experts + one shared expert (index 256), top-8 + shared = 9
    slots per token, hidden 2048, expert intermediate 512, the 16-element-block power-of-two format; 2048-token
    prefill through route_sort -> grouped gate|up GEMM (SwiGLU) -> act_quant -> grouped down GEMM, and the batch-1
    decode as a 9-slot grouped GEMV.  Checks: the sort contract at full size; the grouped outputs of a sample of
    expert segments (busiest, emptiest non-empty, shared) bit-exact against the oracle; and two size-independent
    properties over all 18432 rows: the result does not depend on the row tile (64 vs 256), and every row of the
    grouped GEMM equals the GEMV of that row on its expert."""
    from mxfp4_int8_m5_amd import sc_decode as G, sc_kernels as S
    fmt = layout.Format(block=16)
    pf = product_format(fmt)
    rng = np.random.default_rng(4)
    T, E, topk, D, Fi = 2048, 256, 8, 2048, 512
    E1 = E + 1
    inds8, _ = skewed_routing(rng, T, E, topk)
    inds = np.concatenate([inds8, np.full((T, 1), E, np.int32)], 1)            # shared expert appended for every token
    R = T * (topk + 1)
    perm = linear.interleave_gate_up(Fi)
    gu, dn = [], []
    for _ in range(E1):                                                        # random codes: 257 x (1024x2048 + 2048x512)
        c4 = rng.integers(0, 16, (2 * Fi, D), dtype=np.uint8)
        b = rng.integers(0, 4, (2 * Fi, D // 16), dtype=np.uint8)
        gu.append(layout.pack_rows(c4[perm], b[perm], np.exp2(rng.integers(-12, -6, 2 * Fi)).astype(F32), fmt))
        c4 = rng.integers(0, 16, (D, Fi), dtype=np.uint8)
        b = rng.integers(0, 4, (D, Fi // 16), dtype=np.uint8)
        dn.append(layout.pack_rows(c4, b, np.exp2(rng.integers(-12, -6, D)).astype(F32), fmt))
    gc, gb, gw = (dev(np.stack([p[i] for p in gu])) for i in range(3))
    dc, db, dw = (dev(np.stack([p[i] for p in dn])) for i in range(3))
    xb, x = llm_acts(rng, T, D)
    xq, xs = S.act_quant(dev(xb), Mp=T)
    outs = {}
    for tm in (64, 256):
        pos, tok, es, off, ts, mt = M.route_sort(dev(inds), E1, tm)
        moe.check_route_sort(inds, E1, tm, host(pos), host(tok), host(es), host(off), host(ts))
        act = M.moe_mm(xq, R, gc, gb, gw, off, ts, mt, 2 * Fi, 3, xs, tile=(tm, 64, 4), gather=tok, fmt=pf)
        aq, as_ = S.act_quant(act, Mp=R)
        yd = M.moe_mm(aq, R, dc, db, dw, off, ts, mt, D, 1, as_, tile=(tm, 64, 4), fmt=pf)
        # rows back in assignment order, so that the comparison does not depend on the order inside the segments
        outs[tm] = (host(act)[host(pos)], host(yd)[host(pos)])
    assert np.array_equal(outs[64][0], outs[256][0]) and np.array_equal(outs[64][1], outs[256][1])
    # oracle on a sample of experts
    pos_h, off_h, tok_h = host(pos), host(off), host(tok)[:R]
    counts = np.diff(off_h)
    assert counts[E] == T and counts.sum() == R
    rq, rs = linear.act_quant(x)
    act_h, yd_h, aq_h, as_h = host(act), host(yd), host(aq), host(as_)
    for e in (int(np.argmax(counts[:E])), int(np.argmin(np.where(counts > 0, counts, R))), E):
        rows = slice(off_h[e], off_h[e + 1])
        t = tok_h[rows]
        q_gu = layout.decode(gu[e][0], gu[e][1], 2 * Fi, D, fmt)
        a_ref = linear.epilogue(linear.int_gemm(rq[t], q_gu), rs[t], gu[e][2], 3)
        assert np.array_equal(act_h[rows], a_ref)
        q2, s2 = linear.act_quant(bf16.from_bits(a_ref))
        assert np.array_equal(aq_h[rows], q2) and np.array_equal(as_h[rows], s2)
        q_dn = layout.decode(dn[e][0], dn[e][1], D, Fi, fmt)
        assert np.array_equal(yd_h[rows], linear.epilogue(linear.int_gemm(q2, q_dn), s2, dn[e][2], 1))
    # batch-1 decode of token 0: 8 routed slots + the shared expert, one launch per projection
    eidx = dev(inds8[0].astype(np.int32))
    a1 = G.gemv(xq[:1], gc, gb, xs[:1], gw, 2 * Fi, 3, eidx=eidx, xstride=0, shared=E, fmt=pf)          # [9, 512]
    y1 = G.gemv(a1, dc, db, None, dw, D, 1, eidx=eidx, xstride=1, pro=1, shared=E, fmt=pf)              # [9, 2048]
    mine = pos_h[:topk + 1]                                                    # sorted rows of token 0's assignments
    assert np.array_equal(host(a1), act_h[mine]) and np.array_equal(host(y1), yd_h[mine])


def test_grouped_gemm_random_segments(M):
    """Twenty seeded random expert layouts (1 to 11 experts, segments of 0 to 399 rows, at least one empty, every row
    tile, EPI 0 / 1 / 3): bit-exact against the oracle."""
    rng = np.random.default_rng(2025)
    for case in range(20):
        e, n, k = int(rng.integers(1, 12)), int(rng.integers(1, 80)) * 8, int(rng.integers(1, 5)) * 128
        tm = int(rng.choice([64, 128, 256]))
        counts = rng.integers(0, 400, e)
        counts[rng.integers(0, e)] = 0
        if counts.sum() == 0:
            counts[0] = 5
        ex = np.repeat(np.arange(e), counts).astype(np.int32)
        r = len(ex)
        packs = [random_packed(rng, n, k) for _ in range(e)]
        codes, bc, ws = (np.stack([p[i] for p in packs]) for i in range(3))
        wq = np.stack([p[3] for p in packs])
        xq = rng.integers(-127, 128, (r, k)).astype(np.int8)
        xs = (np.abs(rng.standard_normal(r)) * 1e-2).astype(F32)
        off, tstart, mt = M.segments(dev(ex), e, tm)
        epi = int(rng.choice([0, 1, 3]))
        ref = moe.moe_int_gemm(xq, ex, wq)
        got = host(M.moe_mm(dev(xq), r, dev(codes), dev(bc), dev(ws), off, tstart, mt, n, epi, dev(xs), tile=(tm, 64, 4)))
        want = ref if epi == 0 else moe.moe_epilogue(ref, xs, ws, ex, epi)
        assert np.array_equal(got, want), (case, e, n, k, tm, epi, counts.tolist())


@pytest.mark.parametrize("fi", [0, 1])
def test_packed_weight_tile_of_64_row_passes(M, fi):
    """Row tile 64 with the published codebook (32- and 16-element blocks), N % 256 == 0 and K % 256 == 0 takes the
    kernel that keeps the weights packed in LDS and decodes them per wave after the fragment read, with the block
    codes read by the decoding lanes two K steps at a time.  Segments of 0 / 1 / 31 / 33 / 64 / 65 / 130 / 200 rows,
    every number of K steps from 2 to 14 that the loop structure distinguishes (whole trips of 6 and each tail), a
    gather list, INT32 / scaled / SwiGLU epilogues: bit-exact against the oracle (e2e/sc_moe.py:19-92)."""
    fmt = FORMATS[fi]
    rng = np.random.default_rng(640 + fi)
    counts = np.array([33, 0, 1, 64, 31, 200, 65, 0, 130])
    e = len(counts)
    ex = np.repeat(np.arange(e), counts).astype(np.int32)
    r = len(ex)
    off, tstart, mt = M.segments(dev(ex), e, 64)
    for n, k in [(256, 256), (512, 512), (256, 768), (256, 1024), (512, 1280), (256, 1536), (256, 1792), (768, 2048)]:
        packs = [random_packed(rng, n, k, fmt) for _ in range(e)]
        codes, bc, ws = (np.stack([p[i] for p in packs]) for i in range(3))
        wq = np.stack([p[3] for p in packs])
        src = rng.integers(-127, 128, (r + 40, k)).astype(np.int8)     # the rows are gathered out of a larger matrix
        tok = rng.permutation(r + 40)[:r].astype(np.int32)
        ss = (np.abs(rng.standard_normal(r + 40)) * 1e-2).astype(F32)
        xq, xs = src[tok], ss[tok]
        ref = moe.moe_int_gemm(xq, ex, wq)
        dc, db, dw, pf = dev(codes), dev(bc), dev(ws), product_format(fmt)
        acc = host(M.moe_mm(dev(src), r, dc, db, dw, off, tstart, mt, n, 0, tile=(64, 64, 4), gather=dev(tok), fmt=pf))
        assert np.array_equal(acc, ref), (n, k)
        for epi in (1, 3):
            y = host(M.moe_mm(dev(src), r, dc, db, dw, off, tstart, mt, n, epi, dev(ss), tile=(64, 64, 4), gather=dev(tok), fmt=pf))
            assert np.array_equal(y, moe.moe_epilogue(ref, xs, ws, ex, epi)), (n, k, epi)
        # without the gather list, rows in place
        acc = host(M.moe_mm(dev(xq), r, dc, db, dw, off, tstart, mt, n, 0, tile=(64, 64, 4), fmt=pf))
        assert np.array_equal(acc, ref), (n, k, "in place")
        # block codes at an odd address: the aligned two-step reads of that kernel are not possible, the result is the same
        odd = torch.empty(db.numel() + 1, dtype=torch.uint8, device="cuda")[1:].view(db.shape)
        odd.copy_(db)
        acc = host(M.moe_mm(dev(xq), r, dc, odd, dw, off, tstart, mt, n, 0, tile=(64, 64, 4), fmt=pf))
        assert np.array_equal(acc, ref), (n, k, "odd block-code address")


def test_packed_weight_tile_random_layouts(M):
    """Sixteen seeded random expert layouts at row tile 64 on shapes that take the packed-weight kernel and on neighbours
    that do not (N or K not a multiple of 256): both block sizes, 1 to 23 experts, segments of 0 to 300 rows, gather list
    or rows in place, EPI 0 / 1 / 3: bit-exact against the oracle."""
    rng = np.random.default_rng(6464)
    for case in range(16):
        fmt = FORMATS[int(rng.integers(0, 2))]
        e = int(rng.integers(1, 24))
        n = int(rng.choice([256, 512, 768, 1024, 384, 128]))
        k = int(rng.choice([256, 512, 768, 1280, 2048, 2304, 384, 640]))
        counts = rng.integers(0, 150, e)
        counts[rng.integers(0, e)] = int(rng.choice([0, 1, 64, 65, 300]))
        if counts.sum() == 0:
            counts[0] = 3
        ex = np.repeat(np.arange(e), counts).astype(np.int32)
        r = len(ex)
        packs = [random_packed(rng, n, k, fmt) for _ in range(e)]
        codes, bc, ws = (np.stack([p[i] for p in packs]) for i in range(3))
        wq = np.stack([p[3] for p in packs])
        extra = int(rng.integers(0, 50))
        src = rng.integers(-127, 128, (r + extra, k)).astype(np.int8)
        tok = rng.permutation(r + extra)[:r].astype(np.int32)
        ss = (np.abs(rng.standard_normal(r + extra)) * 1e-2).astype(F32)
        gathered = bool(rng.integers(0, 2))
        xq, xs = (src[tok], ss[tok]) if gathered else (src[:r], ss[:r])
        off, tstart, mt = M.segments(dev(ex), e, 64)
        epi = int(rng.choice([0, 1, 3]))
        ref = moe.moe_int_gemm(xq, ex, wq)
        want = ref if epi == 0 else moe.moe_epilogue(ref, xs, ws, ex, epi)
        got = host(M.moe_mm(dev(src), r, dev(codes), dev(bc), dev(ws), off, tstart, mt, n, epi, dev(ss), tile=(64, 64, 4),
                            gather=dev(tok) if gathered else None, fmt=product_format(fmt)))
        assert np.array_equal(got, want), (case, fmt.block, e, n, k, epi, gathered, counts.tolist())
