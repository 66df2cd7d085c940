"""Mixture-of-experts pieces (numpy; test infrastructure): the router (softmax, top-k, renormalisation, shared-expert
gate), the token sort / expert offsets, the grouped GEMM and the weighted combine."""
import numpy as np

from . import bf16, linear

F32 = np.float32


def route(logit_bits, k, renorm=True, shared_bits=None):
    """Router on bf16 logits [M, E] (uint16 bit patterns): probabilities = bf16(softmax in FP32), the k experts of
    largest probability, their probabilities as scores, divided by their sum when `renorm` (every result rounded to
    bf16, as array ops on bf16 arrays do) -> (inds int32 [M, k], score bits uint16 [M, k]).  With `shared_bits` (bf16
    gate logits [M]) a last slot is appended: expert index E with score bf16(sigmoid(logit)).
    Follows e2e/fused_olmoe.py:183-192 (softmax precise -> argpartition of the k largest -> take_along_axis ->
    optional renormalisation) and e2e/fused_qwen35.py:171-180 (always renormalised, shared expert as slot k with its
    sigmoid gate).  The reference leaves the order of the k slots and the choice among equal probabilities to
    argpartition; this restatement lists them by falling probability, equal ones by rising expert index.
    Arithmetic order (the one the device kernel uses): e_j = 1 / exp(min(max - x_j, 80)) with `linear.exp_f32`; the sum
    of e over lane j % 64 in rising j, then the 64-lane butterfly of `linear._wave_sum`; p_j = bf16(e_j / sum); the
    score total is the FP32 sum in slot order rounded to bf16.  Parity with the MLX ops themselves (softmax rounding at
    a bf16 tie, argpartition's choice among equal probabilities) is unpinned; the restatement is pinned against torch
    CPU ops and a brute-force top-k in tests/test_oracle_router.py."""
    x = bf16.from_bits(np.asarray(logit_bits))
    m, n_e = x.shape
    d = np.minimum(x.max(1, keepdims=True) - x, F32(80.0)).astype(F32)
    e = (F32(1.0) / linear.exp_f32(d)).astype(F32)
    lanes = np.zeros((m, -(-n_e // 64) * 64), F32)
    lanes[:, :n_e] = e
    part = np.zeros((m, 64), F32)
    for c in range(lanes.shape[1] // 64):          # lane l adds its experts l, l + 64, ... in rising order
        part = part + lanes[:, 64 * c:64 * c + 64]
    total = linear._wave_sum(part)
    p_bits = bf16.to_bits((e / total[:, None]).astype(F32))
    # k largest: key = probability bits (non-negative bf16 order like integers), ties to the lower index
    key = p_bits.astype(np.int64) * 65536 + (65535 - np.arange(n_e, dtype=np.int64))[None, :]
    inds = np.argsort(-key, axis=1, kind="stable")[:, :k].astype(np.int32)
    s_bits = np.take_along_axis(p_bits, inds, 1)
    if renorm:
        s = bf16.from_bits(s_bits)
        tot = np.zeros(m, F32)
        for j in range(k):
            tot = tot + s[:, j]
        s_bits = bf16.to_bits((s / bf16.rnd(tot)[:, None]).astype(F32))
    if shared_bits is not None:
        g = bf16.from_bits(np.asarray(shared_bits).reshape(m))
        ex = linear.exp_f32(np.minimum(np.abs(g), F32(80.0)))
        y = (F32(1.0) / (F32(1.0) + ex)).astype(F32)
        sig = np.where(g < 0, y, F32(1.0) - y).astype(F32)
        inds = np.concatenate([inds, np.full((m, 1), n_e, np.int32)], 1)
        s_bits = np.concatenate([s_bits, bf16.to_bits(sig)[:, None]], 1)
    return inds, s_bits


def route_sort(inds, n_experts, tm):
    """inds int [M, topk] -> (pos [R], tok [R+tm], esorted [R], off [E+1], tstart [E+1], max_tiles), R = M*topk.
    Assignments grouped by expert; off = exclusive prefix of the per-expert counts, tstart = exclusive prefix of
    ceil(count / tm), pos[i] = sorted row of assignment i, tok[p] = i // topk of the assignment at row p, padding
    rows tok[R:] = 0, max_tiles = ceil(R / tm) + E.  The order inside a segment is free in the reference
    (e2e/sc_moe.py:110-155); this restatement is the stable one."""
    inds = np.asarray(inds)
    m, topk = inds.shape
    flat = inds.reshape(-1).astype(np.int64)
    r = flat.size
    counts = np.bincount(flat, minlength=n_experts)
    off = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    tstart = np.concatenate([[0], np.cumsum(-(-counts // tm))]).astype(np.int32)
    order = np.argsort(flat, kind="stable")
    pos = np.empty(r, np.int32)
    pos[order] = np.arange(r, dtype=np.int32)
    tok = np.zeros(r + tm, np.int32)
    tok[:r] = order // topk
    return pos, tok, flat[order].astype(np.int32), off, tstart, -(-r // tm) + n_experts


def check_route_sort(inds, n_experts, tm, pos, tok, esorted, off, tstart):
    """The order-free contract of the sort (e2e/sc_moe.py:119-139): raises AssertionError on a violation."""
    inds = np.asarray(inds)
    m, topk = inds.shape
    flat = inds.reshape(-1).astype(np.int64)
    r = flat.size
    counts = np.bincount(flat, minlength=n_experts)
    assert np.array_equal(off, np.concatenate([[0], np.cumsum(counts)])), "off"
    assert np.array_equal(tstart, np.concatenate([[0], np.cumsum(-(-counts // tm))])), "tstart"
    assert np.array_equal(np.sort(pos), np.arange(r)), "pos is not a permutation"
    assert np.array_equal(np.asarray(esorted)[pos], flat), "esorted[pos[i]] != expert of assignment i"
    assert np.array_equal(np.asarray(tok)[pos], np.arange(r) // topk), "tok[pos[i]] != token of assignment i"
    assert not np.asarray(tok)[r:r + tm].any(), "padding rows must gather token 0"
    e = np.asarray(esorted)
    assert np.all(e[1:] >= e[:-1]), "rows are not grouped by expert"


def moe_int_gemm(xq_sorted, esorted, wq_experts):
    """Grouped INT32 GEMM: row r uses expert esorted[r]'s INT8 weights [E, N, K].  Per-expert float64 GEMMs as in
    e2e/sc_moe.py:223-226."""
    r = len(esorted)
    n = wq_experts.shape[1]
    acc = np.zeros((r, n), np.int32)
    for e in np.unique(esorted):
        rows = np.nonzero(np.asarray(esorted) == e)[0]
        acc[rows] = linear.int_gemm(xq_sorted[rows], wq_experts[e])
    return acc


def moe_epilogue(acc, xs, ws_experts, esorted, epi):
    """Row r scales with ws_experts[esorted[r]] (e2e/sc_moe.py:71-91, 234-235)."""
    if epi == 0:
        return acc
    y = bf16.to_bits((acc.astype(F32) * np.asarray(xs, F32)[:, None]) * np.asarray(ws_experts, F32)[esorted])
    if epi == 1:
        return y
    r, n = y.shape
    y4 = y.reshape(r, n // 4, 4)
    return linear.swiglu(y4[:, :, 0:2], y4[:, :, 2:4]).reshape(r, n // 2)


def combine(y_bits, pos, score_bits, res_bits, m):
    """h[t] = bf16(res[t] + acc), acc = 0; for j: acc = bf16(bf16(y[pos[t,j]] * score[t,j]) + acc) — the sequential
    bf16 column sum of e2e/fused_olmoe.py:42-66; rows >= M pass the residual through."""
    res = bf16.from_bits(res_bits)
    y = bf16.from_bits(y_bits)
    sc = bf16.from_bits(score_bits)
    topk = sc.shape[1]
    pos = np.asarray(pos).reshape(m, topk)
    acc = np.zeros((m, res.shape[1]), F32)
    for j in range(topk):
        acc = bf16.rnd(bf16.rnd(y[pos[:, j]] * sc[:m, j:j + 1]) + acc)
    h = res.copy()
    h[:m] = bf16.rnd(res[:m] + acc)
    return bf16.to_bits(h)
