"""Pins the oracle's dispatch (R5), gather_qmm (R6), SwiGLU (R7), combine (R8) and the block (M)."""
import numpy as np
import pytest
import torch

from helpers import f32_of_bits, host_layer, host_tokens, errors


def test_dispatch_is_a_stable_argsort(orc):
    rng = np.random.default_rng(0)
    for P, E in [(1, 4), (64, 8), (1000, 128), (5000, 7)]:
        flat = rng.integers(0, E, P).astype(np.uint32)
        counts, offsets, perm, inv = orc.dispatch(flat, E)
        assert np.array_equal(counts, np.bincount(flat, minlength=E))
        assert np.array_equal(offsets, np.concatenate([[0], np.cumsum(counts)]))
        assert np.array_equal(perm, np.argsort(flat, kind="stable"))
        assert np.array_equal(inv[perm], np.arange(P))
        assert (np.diff(flat[perm].astype(int)) >= 0).all()
    with pytest.raises(RuntimeError):
        orc.dispatch(np.array([0, 9], np.uint32), 4)


def _qbank(orc, rng, E, N, K, bits, std=0.05):
    w = rng.normal(0, std, (E * N, K)).astype(np.float32)
    q, s, b = orc.quantize(w, bits, 64)
    wh = orc.dequantize(q, s, b, bits, 64).reshape(E, N, K)
    return q.reshape(E, N, -1), s.reshape(E, N, -1), b.reshape(E, N, -1), wh


@pytest.mark.parametrize("bits", [4, 8])
def test_gather_qmm_equals_gather_mm_on_dequantised_weights(orc, bits):
    # the reference's test_gather_qmm (ops/quantization.rs:345-423): batch shapes (1)/(5) x (3),
    # indices [0] / [0,2] x [2,1], M=32, N=K=64
    rng = np.random.default_rng(7)
    q, s, b, wh = _qbank(orc, rng, 3, 64, 64, bits, std=1.0)
    for xb, lhs in [(1, [0, 0]), (5, [0, 2])]:
        x = orc.f32_to_bf16(rng.normal(0, 1, (xb, 32, 64)).astype(np.float32))
        rhs = [2, 1]
        y = orc.gather_qmm(x, q, s, b, lhs, rhs, bits)
        xf = f32_of_bits(x).astype(np.float64)
        ref = np.stack([xf[l] @ wh[r].astype(np.float64).T for l, r in zip(lhs, rhs)])
        assert np.allclose(y, ref, rtol=1e-4, atol=1e-4)
    # lhs = None means batch-aligned (test_gather_mm, ops/arithmetic.rs:3139-3211)
    x = orc.f32_to_bf16(rng.normal(0, 1, (2, 4, 64)).astype(np.float32))
    y = orc.gather_qmm(x, q, s, b, None, [1, 0], bits)
    ref = np.stack([f32_of_bits(x)[j].astype(np.float64) @ wh[r].astype(np.float64).T for j, r in enumerate([1, 0])])
    assert np.allclose(y, ref, rtol=1e-4, atol=1e-4)


def test_gather_qmm_single_expert_is_a_plain_matmul(orc):
    rng = np.random.default_rng(8)
    q, s, b, wh = _qbank(orc, rng, 1, 48, 256, 4)
    x = orc.f32_to_bf16(rng.normal(0, 1, (6, 1, 256)).astype(np.float32))
    y = orc.gather_qmm(x, q, s, b, None, [0] * 6, 4)[:, 0]
    ref = torch.from_numpy(f32_of_bits(x)[:, 0]) @ torch.from_numpy(wh[0]).T
    assert torch.allclose(torch.from_numpy(y), ref, rtol=1e-4, atol=1e-5)


def test_gather_qmm_unit_scale_is_exact_integer_arithmetic(orc):
    # scale 1, bias 0, small integer activations: every partial sum is an exact integer in fp32
    rng = np.random.default_rng(9)
    E, N, K = 2, 8, 128
    codes = rng.integers(0, 16, (E, N, K)).astype(np.uint32)
    q = np.zeros((E, N, K // 8), np.uint32)
    for j in range(8):
        q |= codes[..., j::8] << np.uint32(4 * j)
    one = orc.f32_to_bf16(np.ones((E, N, K // 64), np.float32))
    zero = np.zeros((E, N, K // 64), np.uint16)
    xi = rng.integers(-4, 5, (3, 1, K))
    x = orc.f32_to_bf16(xi.astype(np.float32))
    y = orc.gather_qmm(x, q, one, zero, None, [1, 0, 1], 4)[:, 0]
    ref = np.stack([xi[j, 0] @ codes[e].astype(np.int64).T for j, e in enumerate([1, 0, 1])])
    assert np.array_equal(y.astype(np.int64), ref)
    # a single non-zero code picks one column of x
    q1 = np.zeros((1, 1, K // 8), np.uint32)
    q1[0, 0, 5] = 7 << 12   # code 7 at element 5*8 + 3
    y1 = orc.gather_qmm(x[:1], q1, one[:1, :1], zero[:1, :1], None, [0], 4)
    assert y1[0, 0, 0] == 7 * xi[0, 0, 43]


def test_swiglu_closed_form_and_sigmoid_kats(orc):
    # sigmoid(0) = 0.5, sigmoid(+inf) = 1, sigmoid(-inf) = 0 (ops/arithmetic.rs:2577-2600)
    g = np.array([0.0, 80.0, -80.0, 1.0, -1.0], np.float32)
    u = np.array([2.0, 1.0, 1.0, 3.0, 3.0], np.float32)
    out = f32_of_bits(orc.swiglu_f32(g, u)).astype(np.float64)
    ref = g.astype(np.float64) / (1 + np.exp(-g.astype(np.float64))) * u
    assert out[0] == 0.0 and out[1] == 80.0 and abs(out[2]) < 1e-30
    assert (np.abs(out - ref) <= np.abs(ref) * 2.0 ** -8 + 1e-30).all()
    rng = np.random.default_rng(1)
    gb = orc.f32_to_bf16(rng.normal(0, 2, 1000).astype(np.float32))
    ub = orc.f32_to_bf16(rng.normal(0, 2, 1000).astype(np.float32))
    a = f32_of_bits(orc.swiglu_bf16(gb, ub)).astype(np.float64)
    gf, uf = f32_of_bits(gb).astype(np.float64), f32_of_bits(ub).astype(np.float64)
    r = gf / (1 + np.exp(-gf)) * uf
    assert np.abs(a - r).max() <= np.abs(r).max() * 3 * 2.0 ** -8   # three bf16 roundings


def test_combine_closed_form_and_slot_permutation(orc):
    rng = np.random.default_rng(2)
    T, k, H = 9, 4, 64
    y = orc.f32_to_bf16(rng.normal(0, 1, (T * k, H)).astype(np.float32))
    sc = orc.f32_to_bf16(rng.uniform(0, 1, (T, k)).astype(np.float32))
    inv = rng.permutation(T * k).astype(np.uint32)
    out = f32_of_bits(orc.combine(y, sc, inv)).astype(np.float64)
    yf, sf = f32_of_bits(y).astype(np.float64), f32_of_bits(sc).astype(np.float64)
    ref = np.einsum("tk,tkh->th", sf, yf[inv.reshape(T, k).astype(np.int64)])
    assert np.abs(out - ref).max() <= np.abs(ref).max() * 2.0 ** -7
    # identity map when inv_perm is None
    out2 = f32_of_bits(orc.combine(y, sc, None)).astype(np.float64)
    assert np.abs(out2 - np.einsum("tk,tkh->th", sf, yf.reshape(T, k, H))).max() <= 2.0 ** -6
    # shuffling the slots of a token changes nothing beyond fp32 reassociation
    p = rng.permutation(k)
    out3 = f32_of_bits(orc.combine(y, sc[:, p], inv.reshape(T, k)[:, p].reshape(-1))).astype(np.float64)
    assert np.abs(out3 - out).max() <= np.abs(ref).max() * 2.0 ** -7


def numpy_block(orc, W, x, k, mode, bits):
    """Independent fp64 restatement of the whole block from the oracle's routing primitives."""
    xf = f32_of_bits(x).astype(np.float64)
    g = orc.router_logits(x, W["router_w"], W["router_bias"])
    p = orc.softmax(g)
    inds = orc.topk(g if mode == 2 else p, k)
    sc = f32_of_bits(orc.scores(g, p, inds, mode)).astype(np.float64)

    def deq(t):
        E, N = t[0].shape[:2]
        return orc.dequantize(t[0].reshape(E * N, -1), t[1].reshape(E * N, -1), t[2].reshape(E * N, -1),
                              bits, 64).reshape(E, N, -1).astype(np.float64)
    Wg, Wu, Wd = deq(W["gate"]), deq(W["up"]), deq(W["down"])
    out = np.zeros_like(xf)
    for t in range(xf.shape[0]):
        for s in range(k):
            e = int(inds[t, s])
            G, U = Wg[e] @ xf[t], Wu[e] @ xf[t]
            h = G / (1 + np.exp(-G)) * U
            out[t] += sc[t, s] * (Wd[e] @ h)
    return out, inds


@pytest.mark.parametrize("mode,bits", [(0, 4), (1, 4), (2, 8)])
def test_block_against_fp64_restatement(orc, mode, bits):
    H, E, k, I, T = 256, 8, 2, 512, 32
    W = host_layer(orc, H, E, k, I, bits, seed=mode)
    x = host_tokens(orc, T, H, seed=mode)
    cfg = orc.make_config(H, E, k, I, bits, 64, mode)
    ref, inds = numpy_block(orc, W, x, k, mode, bits)
    scale = np.abs(ref).max()
    for strict in (False, True):
        out, d = orc.moe_forward(cfg, W, x, strict=strict, n_threads=4)
        assert np.array_equal(d["topk_idx"], inds)
        assert np.array_equal(d["counts"], np.bincount(inds.reshape(-1), minlength=E))
        assert np.array_equal(d["perm"], np.argsort(inds.reshape(-1), kind="stable"))
        o = f32_of_bits(out).astype(np.float64)
        rel = np.linalg.norm(o - ref) / np.linalg.norm(ref)
        # bf16 outputs: a few ulp from the exact value; op-by-op rounding costs a little more
        assert np.abs(o - ref).max() <= (0.03 if strict else 0.012) * scale
        assert rel <= (8e-3 if strict else 3e-3), rel


def test_strict_and_fused_rounding_points_stay_within_tolerance(orc):
    H, E, k, I, T = 256, 8, 2, 512, 32
    W = host_layer(orc, H, E, k, I, 4, seed=0)
    x = host_tokens(orc, T, H, seed=0)
    cfg = orc.make_config(H, E, k, I)
    a, da = orc.moe_forward(cfg, W, x, strict=True)
    b, db = orc.moe_forward(cfg, W, x, strict=False)
    m, r = errors(b, a)
    assert m <= 2e-2 and r <= 1e-2
    for key in da:
        assert np.array_equal(da[key], db[key])   # routing does not depend on the mode
    # thread count does not change a bit
    c, _ = orc.moe_forward(cfg, W, x, strict=True, n_threads=1)
    assert np.array_equal(a, c)


def test_untransposed_gather_qmm_is_x_times_dequantized(orc):
    """transpose = false (the layout of the reference's test_quantized_matmul,
    mlx-rs/src/ops/quantization.rs:318-342): out = x @ dequantize(w), checked in float64, and on a
    unit-scale integer case where every product and sum is exact."""
    rng = np.random.default_rng(12)
    M, N, K, E = 3, 128, 64, 2
    for bits in (4, 8):
        ws = [orc.quantize((rng.normal(0, 1, (K, N)) / 8).astype(np.float32), bits, 64) for _ in range(E)]
        W, S, B = (np.stack([t[i] for t in ws]) for i in range(3))
        x = orc.f32_to_bf16(rng.normal(0, 1, (4, M, K)).astype(np.float32))
        lhs, rhs = np.array([3, 1], np.uint32), np.array([1, 0], np.uint32)
        y = orc.gather_qmm(x, W, S, B, lhs, rhs, bits=bits, want="f32", transpose=False)
        assert y.shape == (2, M, N)
        for j in range(2):
            ref = f32_of_bits(x[lhs[j]]).astype(np.float64) @ orc.dequantize(W[rhs[j]], S[rhs[j]], B[rhs[j]], bits, 64).astype(np.float64)
            assert np.abs(y[j] - ref).max() <= 1e-4
    # integers: codes 0..15 with scale 1, bias 0; x small integers: the result is the integer product
    q = rng.integers(0, 16, (K, N)).astype(np.uint32)
    packed = np.zeros((1, K, N // 8), np.uint32)
    for c in range(8):
        packed[0] |= q[:, c::8] << np.uint32(4 * c)
    one, zero = orc.f32_to_bf16(np.ones((1, K, N // 64), np.float32)), orc.f32_to_bf16(np.zeros((1, K, N // 64), np.float32))
    xi = rng.integers(-3, 4, (1, 2, K)).astype(np.float32)
    y = orc.gather_qmm(orc.f32_to_bf16(xi), packed, one, zero, None, np.zeros(1, np.uint32), bits=4, want="f32", transpose=False)
    assert np.array_equal(y[0], xi[0] @ q.astype(np.float32))
