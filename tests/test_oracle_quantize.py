"""Pins the oracle's MLX-affine quantize / dequantize (W row of the hot-path table).

Anchors: the reference's own known-answer test mlx-rs/src/ops/quantization.rs:298-315
(arange 128x512, group 128, bits 2/4/8: shapes and max error), the format statement
:31-47,85-87 (codes packed low bits first in uint32), and what the arithmetic fixes."""
import numpy as np
import pytest


def unpack(q, bits):
    """Independent unpacking: code c of a row = bits [(c % per)*bits, +bits) of word c // per."""
    per = 32 // bits
    rows, words = q.shape
    out = np.zeros((rows, words * per), np.uint32)
    for j in range(per):
        out[:, j::per] = (q >> np.uint32(j * bits)) & np.uint32((1 << bits) - 1)
    return out


@pytest.mark.parametrize("bits", [2, 4, 8])
def test_reference_kat_arange(orc, bits):
    # test_quantize_dequantize: x[r, c] = c, group 128
    x = np.tile(np.arange(512, dtype=np.float32), (128, 1))
    q, s, b = orc.quantize(x, bits, 128, "f32")
    assert q.shape == (128, 512 // (32 // bits)) and q.dtype == np.uint32
    assert s.shape == (128, 4) and b.shape == (128, 4)
    xh = orc.dequantize(q, s, b, bits, 128)
    assert np.abs(x - xh).max() <= 127.0 / (1 << bits)
    # every row is the same, and the codes are monotone along a group
    codes = unpack(q, bits)
    assert (codes == codes[0]).all()
    g0 = codes[0, :128].astype(int)
    assert (np.diff(g0) <= 0).all() or (np.diff(g0) >= 0).all()


@pytest.mark.parametrize("bits,group", [(4, 64), (8, 64), (4, 32), (8, 128), (2, 64)])
def test_roundtrip_bound_and_packing(orc, bits, group):
    rng = np.random.default_rng(bits * 100 + group)
    w = rng.normal(0, 0.02, (24, 4 * group)).astype(np.float32)
    q, s, b = orc.quantize(w, bits, group, "f32")
    codes = unpack(q, bits).astype(np.float64)
    assert codes.max() <= (1 << bits) - 1
    sg = np.repeat(s.astype(np.float64), group, axis=1)
    bg = np.repeat(b.astype(np.float64), group, axis=1)
    # the oracle's dequantize is s*q + b on the independently unpacked codes
    wh = orc.dequantize(q, s, b, bits, group)
    assert np.allclose(wh, sg * codes + bg, rtol=0, atol=1e-7)
    # every element got the code that is nearest to it among 0 .. 2^bits-1 (brute force over codes)
    allc = np.arange(1 << bits, dtype=np.float64)
    err_all = np.abs(w.astype(np.float64)[..., None] - (sg[..., None] * allc + bg[..., None]))
    assert (np.abs(w - wh) <= err_all.min(-1) + 1e-7).all()
    # unclamped elements are within half a step
    inner = (codes > 0) & (codes < (1 << bits) - 1)
    assert (np.abs(w - wh)[inner] <= (np.abs(sg) / 2 + 1e-6)[inner]).all()
    # a group that straddles zero represents zero exactly (code -bias/scale is an integer in range)
    wg0 = w.reshape(24, 4, group)
    straddle = (wg0.min(-1) < 0) & (wg0.max(-1) > 0)
    zc = -(b.astype(np.float64) / s.astype(np.float64))
    assert (np.abs(zc - np.rint(zc))[straddle] < 1e-4).all()
    assert ((zc >= -1e-4) & (zc <= (1 << bits) - 1 + 1e-4))[straddle].all()
    # the edge of larger magnitude is represented exactly (it is the bias)
    wg = w.reshape(24, 4, group)
    edge = np.where(np.abs(wg.min(-1)) > np.abs(wg.max(-1)), wg.min(-1), wg.max(-1))
    assert np.array_equal(b, edge.astype(np.float32))


def test_special_groups(orc):
    g = 64
    w = np.zeros((4, g), np.float32)
    w[1] = 0.5                                  # constant group
    w[2] = -np.abs(np.linspace(0.1, 1, g))      # negative-dominant: bias = w_min, scale > 0
    w[3] = np.linspace(-0.2, 1, g)              # positive-dominant: bias = w_max, scale < 0
    q, s, b = orc.quantize(w, 4, g, "f32")
    wh = orc.dequantize(q, s, b, 4, g)
    assert np.array_equal(wh[0], w[0]) and b[0, 0] == 0.0
    assert np.allclose(wh[1], 0.5)
    assert b[2, 0] == w[2].min() and s[2, 0] > 0
    assert b[3, 0] == w[3].max() and s[3, 0] < 0
    assert np.abs(wh - w).max() <= np.abs(s).max() / 2 + 1e-6


def test_bf16_scales_are_rounded_after_the_codes(orc):
    rng = np.random.default_rng(5)
    w = rng.normal(0, 0.02, (8, 256)).astype(np.float32)
    q32, s32, b32 = orc.quantize(w, 4, 64, "f32")
    q16, s16, b16 = orc.quantize(w, 4, 64, "bf16")
    assert np.array_equal(q32, q16)
    assert np.array_equal(s16, orc.f32_to_bf16(s32)) and np.array_equal(b16, orc.f32_to_bf16(b32))


def test_bf16_conversion_is_round_to_nearest_even(orc):
    import torch
    rng = np.random.default_rng(1)
    f = np.concatenate([rng.normal(0, 1, 4000), rng.normal(0, 1e-20, 100), [0.0, -0.0, 1.0, 65280.0, 3.3895314e38]])
    f = f.astype(np.float32)
    ours = orc.f32_to_bf16(f)
    ref = torch.from_numpy(f).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(ours, ref)
    assert np.array_equal(orc.bf16_to_f32(ours), torch.from_numpy(f).to(torch.bfloat16).float().numpy())


def test_error_paths(orc):
    w = np.zeros((2, 100), np.float32)
    with pytest.raises(RuntimeError):
        orc.quantize(w, 4, 64)       # columns not divisible by the group
    with pytest.raises(RuntimeError):
        orc.quantize(np.zeros((2, 128), np.float32), 3, 64)  # unsupported bits
