"""Pins of the oracle's RMS normalisation and of the block wrapped in norm + residual
(oracle/moe_oracle.c: orc_rms_norm, orc_moe_forward_residual), independent of the oracle's code."""
import numpy as np
import torch

from helpers import f32_of_bits, host_layer, host_tokens


def test_rms_norm_closed_form_and_torch(orc):
    rng = np.random.default_rng(1)
    x = orc.f32_to_bf16(rng.normal(0, 2.0, (7, 192)).astype(np.float32))
    w = orc.f32_to_bf16(rng.normal(1, 0.2, 192).astype(np.float32))
    got = f32_of_bits(orc.rms_norm(x, w, 1e-5)).astype(np.float64)
    xf, wf = f32_of_bits(x).astype(np.float64), f32_of_bits(w).astype(np.float64)
    ref = wf * xf / np.sqrt((xf ** 2).mean(-1, keepdims=True) + 1e-5)
    assert np.abs(got - ref).max() <= np.abs(ref).max() * 2 ** -8      # one bf16 rounding
    t = torch.nn.functional.rms_norm(torch.from_numpy(f32_of_bits(x)), (192,), torch.from_numpy(f32_of_bits(w)), 1e-5)
    assert np.abs(got - t.numpy().astype(np.float64)).max() <= np.abs(ref).max() * 2 ** -8


def test_rms_norm_special_cases(orc):
    one = orc.f32_to_bf16(np.ones(64, np.float32))
    # a constant row c normalises to sign(c) (eps negligible), zero stays zero
    for c in (3.0, -0.5):
        x = orc.f32_to_bf16(np.full((1, 64), c, np.float32))
        assert np.allclose(f32_of_bits(orc.rms_norm(x, one, 1e-12)), np.sign(c), atol=2 ** -8)
    assert not f32_of_bits(orc.rms_norm(orc.f32_to_bf16(np.zeros((2, 64), np.float32)), one, 1e-5)).any()
    # scale invariance: rms_norm(a x) == rms_norm(x) for a power of two (exact in bf16), eps = 0
    rng = np.random.default_rng(2)
    x = rng.normal(0, 1, (3, 64)).astype(np.float32)
    a, b = orc.rms_norm(orc.f32_to_bf16(x), one, 0.0), orc.rms_norm(orc.f32_to_bf16(4 * x), one, 0.0)
    assert np.array_equal(a, b)
    # the weight multiplies: doubling it doubles the result exactly
    two = orc.f32_to_bf16(np.full(64, 2.0, np.float32))
    assert np.array_equal(f32_of_bits(orc.rms_norm(orc.f32_to_bf16(x), two, 1e-5)),
                          2 * f32_of_bits(orc.rms_norm(orc.f32_to_bf16(x), one, 1e-5)))


def test_rms_norm_statistic_of_the_reference_test(orc):
    """mlx-rs/src/fast.rs:304-324: uniform(0,1) input [2,8,16], unit weight, eps 1e-5: mean
    0.8729 +- 0.0175, sum 223.47 +- 4.47 (the input comes from MLX's generator, which cannot be
    reproduced; any uniform sample of that shape lands inside the stated bands)."""
    rng = np.random.default_rng(103)
    x = orc.f32_to_bf16(rng.uniform(0, 1, (16, 16)).astype(np.float32))
    y = f32_of_bits(orc.rms_norm(x, orc.f32_to_bf16(np.ones(16, np.float32)), 1e-5))
    assert abs(y.mean() - 0.87293875) <= 0.017458774 * 2
    assert abs(y.sum() - 223.47232) <= 4.469446 * 2


def test_block_with_norm_and_residual_is_the_composition(orc):
    H, E, k, I, T = 128, 4, 2, 128, 9
    W = host_layer(orc, H, E, k, I, 4, seed=8)
    x = host_tokens(orc, T, H, seed=8)
    nw = orc.f32_to_bf16(np.random.default_rng(3).normal(1, 0.1, H).astype(np.float32))
    cfg = orc.make_config(H, E, k, I)
    out, d = orc.moe_forward(cfg, W, x, strict=True, n_threads=2, norm_weight=nw, eps=1e-6)
    xn = orc.rms_norm(x, nw, 1e-6)
    y, d2 = orc.moe_forward(cfg, W, xn, strict=True, n_threads=2)
    assert all(np.array_equal(d[n], d2[n]) for n in d)
    want = orc.f32_to_bf16(f32_of_bits(x) + f32_of_bits(y))
    assert np.array_equal(out, want)
    fused, _ = orc.moe_forward(cfg, W, x, strict=False, n_threads=2, norm_weight=nw, eps=1e-6)
    assert np.abs(f32_of_bits(fused) - f32_of_bits(out)).max() <= 2e-2
