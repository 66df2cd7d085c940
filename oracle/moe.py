"""Mixture-of-experts pieces (numpy; test infrastructure): the token sort / expert offsets, the grouped GEMM and
the weighted combine."""
import numpy as np

from . import bf16, linear

F32 = np.float32


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
