"""Pins of the oracle's router restatement (oracle/moe.route; e2e/fused_olmoe.py:183-192, e2e/fused_qwen35.py:171-180)
without the reference's array library: torch CPU ops as an independent implementation of the same array program, a
brute-force top-k, and closed-form cases."""
import numpy as np
import pytest
import torch

from oracle import bf16, moe

F32 = np.float32


def logits(rng, m, e, bias=1.5):
    return bf16.to_bits((rng.standard_normal((m, e)) + rng.standard_normal(e) * bias).astype(F32))


def as_bf16(bits):
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).view(torch.bfloat16)


def ulps(a_bits, b_bits):
    return np.abs(a_bits.astype(np.int64) - b_bits.astype(np.int64))


@pytest.mark.parametrize("m,e,k", [(512, 64, 8), (300, 256, 8), (64, 257, 9), (100, 8, 2), (50, 1000, 5)])
def test_softmax_and_topk_against_torch_cpu(m, e, k):
    """The same array program in torch on the CPU: softmax in FP32 rounded to bf16, k largest, gather, renormalise.
    Probabilities agree to the bf16 bit except where the FP32 value sits on a rounding boundary (at most one step, in
    under 0.1 % of the entries); the selected sets are equal wherever the k-th and (k+1)-th probabilities differ."""
    rng = np.random.default_rng(m + e)
    lb = logits(rng, m, e)
    x = as_bf16(lb)
    p = torch.softmax(x.float(), dim=1).to(torch.bfloat16)
    inds, s_bits = moe.route(lb, k, renorm=False)
    pb = p.view(torch.int16).numpy().view(np.uint16)
    mine = np.take_along_axis(pb, inds, 1)
    d = ulps(mine, s_bits)
    assert d.max() <= 1 and (d > 0).mean() < 1e-3
    # brute force on torch's probabilities: the k largest values as a multiset
    srt = np.sort(pb.astype(np.int32), axis=1)[:, ::-1]
    clear = srt[:, k - 1] != srt[:, k] if k < e else np.ones(m, bool)
    exact = (d == 0).all(1)
    rows = clear & exact
    assert rows.mean() > 0.7          # bf16 probabilities of neighbouring ranks are often equal when E is large
    assert np.array_equal(np.sort(mine[rows].astype(np.int32), axis=1)[:, ::-1], srt[rows, :k])
    # the slots are listed by falling probability, equal ones by rising index
    assert np.all(np.diff(s_bits.astype(np.int32), axis=1) <= 0)
    tie = np.diff(s_bits.astype(np.int32), axis=1) == 0
    assert np.all(np.diff(inds, axis=1)[tie] > 0)
    # no expert twice
    assert all(len(set(r)) == k for r in inds.tolist())


@pytest.mark.parametrize("m,e,k", [(512, 64, 8), (300, 256, 8)])
def test_renormalisation_against_torch_cpu(m, e, k):
    rng = np.random.default_rng(7 * m + e)
    lb = logits(rng, m, e)
    inds, raw = moe.route(lb, k, renorm=False)
    inds2, s_bits = moe.route(lb, k, renorm=True)
    assert np.array_equal(inds, inds2)
    s = as_bf16(raw)
    ref = (s / s.sum(dim=-1, keepdim=True)).view(torch.int16).numpy().view(np.uint16)
    d = ulps(ref, s_bits)
    assert d.max() <= 1 and (d > 0).mean() < 2e-3
    tot = bf16.from_bits(s_bits).sum(1)
    assert np.all(np.abs(tot - 1) < 0.02)


def test_shared_expert_slot_and_sigmoid_gate():
    rng = np.random.default_rng(11)
    m, e, k = 200, 256, 8
    lb = logits(rng, m, e)
    gl = bf16.to_bits((rng.standard_normal(m) * 3).astype(F32))
    gl[:4] = bf16.to_bits(np.array([0.0, -0.0, 40.0, -40.0], F32))
    inds, s_bits = moe.route(lb, k, renorm=True, shared_bits=gl)
    i8, s8 = moe.route(lb, k, renorm=True)
    assert inds.shape == (m, k + 1) and np.all(inds[:, k] == e)
    assert np.array_equal(inds[:, :k], i8) and np.array_equal(s_bits[:, :k], s8)
    ref = torch.sigmoid(as_bf16(gl).float()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    d = ulps(ref, s_bits[:, k])
    assert d.max() <= 1 and (d > 0).mean() < 0.01
    got = bf16.from_bits(s_bits[:4, k]).tolist()
    assert got[:3] == [0.5, 0.5, 1.0] and abs(got[3] / 4.248354e-18 - 1) < 0.01


def test_closed_forms():
    # equal logits: uniform probabilities, the k lowest indices win, renormalised scores are 1/k
    lb = bf16.to_bits(np.full((3, 64), 1.25, F32))
    inds, s_bits = moe.route(lb, 8, renorm=False)
    assert np.array_equal(inds, np.tile(np.arange(8, dtype=np.int32), (3, 1)))
    assert np.all(bf16.from_bits(s_bits) == F32(1 / 64))
    _, s_bits = moe.route(lb, 8, renorm=True)
    assert np.all(bf16.from_bits(s_bits) == F32(0.125))
    # one dominant logit: probability 1 for it, zeros (after the clamp at 80) elsewhere, picked by rising index
    x = np.zeros((1, 16), F32)
    x[0, 5] = 200.0
    inds, s_bits = moe.route(bf16.to_bits(x), 3, renorm=True)
    assert inds.tolist() == [[5, 0, 1]]
    s = bf16.from_bits(s_bits)[0]
    assert s[0] == 1.0 and 0 <= s[1] < 1e-30 and s[1] == s[2]
    # two-expert softmax equals the sigmoid of the difference
    x = np.array([[0.5, -1.0]], F32)
    _, s_bits = moe.route(bf16.to_bits(x), 2, renorm=False)
    want = bf16.to_bits(np.array([1 / (1 + np.exp(-1.5)), 1 / (1 + np.exp(1.5))], F32))
    assert np.array_equal(s_bits[0], want)


def test_brute_force_tiny():
    """Every token of a tiny case against a plain-Python router in float64."""
    rng = np.random.default_rng(5)
    m, e, k = 40, 12, 3
    lb = logits(rng, m, e, bias=0.5)
    inds, s_bits = moe.route(lb, k, renorm=True)
    x = bf16.from_bits(lb).astype(np.float64)
    for t in range(m):
        p = np.exp(x[t] - x[t].max())
        p /= p.sum()
        pb = bf16.to_bits(p.astype(F32)).astype(int)
        order = sorted(range(e), key=lambda j: (-pb[j], j))[:k]
        if sorted(pb, reverse=True)[k - 1] != sorted(pb, reverse=True)[k]:
            assert set(order) == set(inds[t].tolist())
        s = bf16.from_bits(np.array([pb[j] for j in inds[t]], np.uint16)).astype(np.float64)
        want = s / float(bf16.rnd(np.array([s.sum()], F32))[0])
        got = bf16.from_bits(s_bits[t]).astype(np.float64)
        assert np.all(np.abs(got - want) <= np.abs(want) * 2.0 ** -8)
