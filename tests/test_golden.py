"""Frozen vectors of the MoE block (tests/golden/moe_block_*.npz, written by
tests/golden/make_golden.py).  CPU: the oracle still gives these answers, and an independent
fp64 numpy restatement of the block agrees with them.  GPU: the HIP path is checked against
the files alone: routing integers and logits bit for bit, outputs within the stated
tolerance (max-abs 2e-2, relative Frobenius 1e-2 in bf16)."""
import glob
import os

import numpy as np
import pytest

from helpers import assert_close_bf16, bf16_tensor, bits_u16, bits_u32, device_block, f32_of_bits

HERE = os.path.dirname(os.path.abspath(__file__))
FILES = sorted(glob.glob(os.path.join(HERE, "golden", "moe_block_*.npz")))
ROUTING = ("topk_idx", "topk_w", "counts", "offsets", "perm", "inv_perm")


def load(path):
    z = np.load(path, allow_pickle=False)
    H, E, k, I, bits, group, mode, T = (int(v) for v in z["config"])
    W = dict(router_w=z["router_w"], router_bias=z["router_bias"] if "router_bias" in z else None)
    for bank in ("gate", "up", "down"):
        W[bank] = tuple(z[f"{bank}_{s}"] for s in ("w", "scales", "biases"))
    return z, (H, E, k, I, bits, group, mode, T), W


def test_fixtures_exist():
    assert len(FILES) == 3


@pytest.mark.parametrize("path", FILES, ids=[os.path.basename(f)[10:-4] for f in FILES])
def test_oracle_reproduces_the_fixtures(orc, path):
    z, (H, E, k, I, bits, group, mode, T), W = load(path)
    cfg = orc.make_config(H, E, k, I, bits, group, mode)
    for strict, key in ((True, "out_strict"), (False, "out_fused")):
        out, d = orc.moe_forward(cfg, W, z["x"], strict=strict, n_threads=2)
        assert np.array_equal(out, z[key]), key
        for n in ROUTING:
            assert np.array_equal(d[n], z[n]), n
    assert np.array_equal(orc.router_logits(z["x"], W["router_w"], W["router_bias"]), z["logits"])


def _dequant(w, s, b, bits):
    """[E,N,words] packed -> float64 [E,N,K], written from the format's definition."""
    per = 32 // bits
    sh = (np.arange(per, dtype=np.uint32) * bits)[None, None, None, :]
    q = ((w[..., None] >> sh) & ((1 << bits) - 1)).reshape(w.shape[0], w.shape[1], -1).astype(np.float64)
    sc = np.repeat(f32_of_bits(s).astype(np.float64), 64, axis=-1)
    bi = np.repeat(f32_of_bits(b).astype(np.float64), 64, axis=-1)
    return sc * q + bi


@pytest.mark.parametrize("path", FILES, ids=[os.path.basename(f)[10:-4] for f in FILES])
def test_fixtures_agree_with_an_fp64_restatement(path):
    """Takes the routing decision from the file (the tie order is this build's convention) and
    recomputes scores and outputs in float64 from the definitions."""
    z, (H, E, k, I, bits, group, mode, T), W = load(path)
    x = f32_of_bits(z["x"]).astype(np.float64)
    logits = x @ f32_of_bits(W["router_w"]).astype(np.float64).T
    if W["router_bias"] is not None:
        logits = logits + W["router_bias"]
    # the selected experts are the k largest logits (softmax is monotone)
    idx = z["topk_idx"].astype(np.int64)
    kth = np.sort(logits, axis=1)[:, -k]
    picked = np.take_along_axis(logits, idx, 1)
    assert (picked >= kth[:, None] - 4e-3 * np.abs(kth[:, None]) - 1e-6).all()
    p = np.exp(logits - logits.max(1, keepdims=True))
    p /= p.sum(1, keepdims=True)
    ps = np.take_along_axis(p, idx, 1)
    if mode == 0:
        sc = ps / ps.sum(1, keepdims=True)
    elif mode == 1:
        sc = ps
    else:
        e = np.exp(picked - picked.max(1, keepdims=True))
        sc = e / e.sum(1, keepdims=True)
    assert np.abs(f32_of_bits(z["topk_w"]) - sc).max() <= 1e-2
    wg, wu, wd = (_dequant(*W[b], bits) for b in ("gate", "up", "down"))
    out = np.zeros((T, H))
    for t in range(T):
        for s in range(k):
            e = idx[t, s]
            g, u = wg[e] @ x[t], wu[e] @ x[t]
            out[t] += sc[t, s] * (wd[e] @ (g / (1 + np.exp(-g)) * u))
    for key in ("out_strict", "out_fused"):
        got = f32_of_bits(z[key]).astype(np.float64)
        assert np.abs(got - out).max() <= 2e-2
        assert np.linalg.norm(got - out) / np.linalg.norm(out) <= 1e-2
    # integer invariants of the dispatch
    assert np.array_equal(z["counts"], np.bincount(idx.reshape(-1), minlength=E).astype(np.uint32))
    assert np.array_equal(z["perm"], np.argsort(idx.reshape(-1), kind="stable").astype(np.uint32))
    assert np.array_equal(z["inv_perm"][z["perm"]], np.arange(T * k, dtype=np.uint32))


@pytest.mark.gpu
@pytest.mark.parametrize("path", FILES, ids=[os.path.basename(f)[10:-4] for f in FILES])
def test_hip_path_matches_the_fixtures(path):
    import torch

    import mlx_rs_amd as m
    z, (H, E, k, I, bits, group, mode, T), W = load(path)
    blk = device_block(m, m.MoeConfig(H, E, k, I, bits, group, mode), W, "cuda")
    out, dbg = blk.forward(bf16_tensor(z["x"], "cuda"), debug=True)
    torch.cuda.synchronize()
    for n in ("topk_idx", "counts", "offsets", "perm", "inv_perm"):
        assert np.array_equal(bits_u32(dbg[n]).reshape(z[n].shape), z[n]), n
    assert np.array_equal(bits_u16(dbg["topk_w"]), z["topk_w"])
    assert_close_bf16(bits_u16(out), z["out_strict"], what="vs op-by-op rounding")
    assert_close_bf16(bits_u16(out), z["out_fused"], what="vs fused rounding")
