"""Pins the oracle's router: logits (R1), softmax (R2), top-k (R3), scores (R4)."""
from fractions import Fraction

import numpy as np
import pytest
import torch

from helpers import f32_of_bits


def rnd_bf16(orc, rng, shape, std):
    return orc.f32_to_bf16(rng.normal(0, std, shape).astype(np.float32))


def test_logits_match_fp64_matmul(orc):
    rng = np.random.default_rng(0)
    x, w = rnd_bf16(orc, rng, (40, 512), 1.0), rnd_bf16(orc, rng, (16, 512), 0.02)
    bias = rng.normal(0, 1, 16).astype(np.float32)
    for b in (None, bias):
        g = orc.router_logits(x, w, b)
        exact = f32_of_bits(x).astype(np.float64) @ f32_of_bits(w).astype(np.float64).T
        if b is not None:
            exact = exact + b.astype(np.float64)
        ref = orc.f32_to_bf16(exact.astype(np.float32))
        assert np.array_equal(g, ref)
        t = (torch.from_numpy(f32_of_bits(x)).double() @ torch.from_numpy(f32_of_bits(w)).double().T)
        if b is not None:
            t = t + torch.from_numpy(b).double()
        assert np.array_equal(g, t.float().to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16))


def test_logits_exact_rational_tiny(orc):
    # brute force with exact rationals: the bf16 logit is the correctly rounded exact dot product
    rng = np.random.default_rng(3)
    x, w = rnd_bf16(orc, rng, (3, 64), 1.0), rnd_bf16(orc, rng, (4, 64), 0.02)
    g = orc.router_logits(x, w)
    xf, wf = f32_of_bits(x), f32_of_bits(w)
    for t in range(3):
        for e in range(4):
            exact = sum(Fraction(float(a)) * Fraction(float(b)) for a, b in zip(xf[t], wf[e]))
            ref = orc.f32_to_bf16(np.array([np.float32(float(exact))]))[0]
            assert g[t, e] == ref


def test_fp32_order_moves_few_logits_by_one_ulp(orc):
    # documents how far an fp32 summation order is from the order-independent definition
    rng = np.random.default_rng(4)
    x, w = rnd_bf16(orc, rng, (64, 2048), 1.0), rnd_bf16(orc, rng, (128, 2048), 0.02)
    a, b = orc.router_logits(x, w), orc.router_logits(x, w, f32seq=True)
    diff = (a != b).mean()
    assert diff < 0.05
    assert np.abs(a.astype(np.int32) - b.astype(np.int32)).max() <= 1


def test_softmax_matches_torch_and_sums_to_one(orc):
    rng = np.random.default_rng(1)
    g = rnd_bf16(orc, rng, (64, 128), 2.0)
    p = orc.softmax(g)
    ref = torch.softmax(torch.from_numpy(f32_of_bits(g)), -1).to(torch.bfloat16)
    ref_bits = ref.view(torch.int16).numpy().view(np.uint16)
    # torch's expf may differ from the oracle's in the last fp32 bit: at most one bf16 ulp, rarely
    d = np.abs(p.astype(np.int32) - ref_bits.astype(np.int32))
    assert d.max() <= 1 and (d != 0).mean() < 0.01
    # rows sum to one (the reference checks the same on [2,8,16], nn/activation.rs:1156-1185)
    s = f32_of_bits(p).astype(np.float64).sum(-1)
    assert np.abs(s - 1).max() < 2.0 ** -7
    # order preserving
    gi, pi = f32_of_bits(g), f32_of_bits(p)
    for t in range(8):
        o = np.argsort(gi[t])
        assert (np.diff(pi[t][o]) >= 0).all()


def test_exp_accuracy_and_range(orc):
    xs = np.linspace(-79.9, 0, 4001).astype(np.float32)
    e = np.array([orc.expf(float(v)) for v in xs], np.float64)
    assert np.abs(e / np.exp(xs.astype(np.float64)) - 1).max() < 3e-7
    assert orc.expf(0.0) == 1.0 and orc.expf(-81.0) == 0.0 and orc.expf(float("-inf")) == 0.0


def brute_topk(vals, k):
    order = sorted(range(len(vals)), key=lambda e: (-vals[e], e))
    return order[:k]


def test_topk_total_order_and_ties(orc):
    rng = np.random.default_rng(2)
    v = rnd_bf16(orc, rng, (200, 32), 1.0)
    v[::3] = orc.f32_to_bf16(np.round(f32_of_bits(v[::3]) * 2) / 2)   # many exact ties
    inds = orc.topk(v, 6)
    f = f32_of_bits(v)
    for t in range(200):
        assert inds[t].tolist() == brute_topk(f[t].tolist(), 6)
    # all equal -> lowest ids in order
    same = np.full((1, 16), orc.f32_to_bf16(np.float32(0.25)), np.uint16)
    assert orc.topk(same, 4)[0].tolist() == [0, 1, 2, 3]
    # a tie that straddles the k-th place: the lower id wins
    row = orc.f32_to_bf16(np.array([[0.1, 0.5, 0.3, 0.3, 0.3, 0.9]], np.float32))
    assert orc.topk(row, 3)[0].tolist() == [5, 1, 2]
    # -0 and +0 tie
    z = orc.f32_to_bf16(np.array([[-0.0, 0.0, -1.0]], np.float32))
    assert orc.topk(z, 2)[0].tolist() == [0, 1]


@pytest.mark.parametrize("mode", [0, 1, 2])
def test_scores_closed_forms(orc, mode):
    rng = np.random.default_rng(10 + mode)
    g = rnd_bf16(orc, rng, (50, 64), 1.5)
    p = orc.softmax(g)
    inds = orc.topk(g if mode == 2 else p, 8)
    sc = f32_of_bits(orc.scores(g, p, inds, mode)).astype(np.float64)
    gf, pf = f32_of_bits(g).astype(np.float64), f32_of_bits(p).astype(np.float64)
    sel_p = np.take_along_axis(pf, inds.astype(np.int64), 1)
    if mode == 1:
        assert np.array_equal(sc, sel_p)
    elif mode == 0:
        ref = sel_p / sel_p.sum(-1, keepdims=True)
        assert np.abs(sc / ref - 1).max() < 2.0 ** -6  # two bf16 roundings
        assert np.abs(sc.sum(-1) - 1).max() < 0.02
    else:
        sel_g = np.take_along_axis(gf, inds.astype(np.int64), 1)
        ref = np.exp(sel_g - sel_g.max(-1, keepdims=True))
        ref /= ref.sum(-1, keepdims=True)
        assert np.abs(sc / ref - 1).max() < 2.0 ** -7
    # slot 0 is the best expert, scores never increase along the slots
    assert (np.diff(sc, axis=1) <= 0).all()
