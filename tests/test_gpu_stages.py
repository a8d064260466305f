"""GPU parity of the stage-level entry points (through the C ABI) against the oracle: integer
results bit-exact, floats within max-abs 2e-2 and relative Frobenius 1e-2 (bf16)."""
import numpy as np
import pytest
import torch

from helpers import (assert_close_bf16, bits_u16, bits_u32, bf16_tensor, i32_tensor, f32_of_bits)

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def m():
    import mlx_rs_amd
    mlx_rs_amd.load_library()
    return mlx_rs_amd


@pytest.mark.parametrize("T,H,E,k,mode,bias", [
    (1, 2048, 128, 8, 0, False), (33, 2048, 128, 8, 0, True), (300, 512, 60, 6, 1, False),
    (65, 4096, 8, 2, 2, False), (17, 256, 300, 8, 0, True), (5, 128, 5, 5, 2, False),
    # 256 and more 32 x 32 logit tiles: the larger tile of the fp64 kernel (fewer: 16 x 16 tiles), ragged edges
    (2048, 256, 128, 8, 0, True), (1000, 128, 300, 4, 1, False),
    # a single expert (the block as a dense MLP): every score is 1
    (1, 256, 1, 1, 0, False), (40, 256, 1, 1, 2, False), (300, 256, 1, 1, 1, True),
])
def test_route_bit_exact(orc, m, T, H, E, k, mode, bias):
    print(f"route T={T} H={H} E={E} k={k} mode={mode}", flush=True)
    rng = np.random.default_rng(T + E)
    x = orc.f32_to_bf16(rng.normal(0, 1, (T, H)).astype(np.float32))
    w = orc.f32_to_bf16(rng.normal(0, 0.02, (E, H)).astype(np.float32))
    b = rng.normal(0, 1, E).astype(np.float32) if bias else None
    cfg = orc.make_config(H, E, k, 64, 4, 64, mode)
    inds, sc = orc.route(cfg, w, b, x)
    gi, gs, gl = m.ops.route(bf16_tensor(x, "cuda"), bf16_tensor(w, "cuda"), k, mode,
                             None if b is None else torch.from_numpy(b).cuda(), return_logits=True)
    assert np.array_equal(bits_u16(gl), orc.router_logits(x, w, b)), "logits"
    assert np.array_equal(bits_u32(gi), inds), "top-k indices"
    assert np.array_equal(bits_u16(gs), sc), "scores"


def test_route_ties_go_to_the_lower_expert(orc, m):
    # identical router rows give identical logits: ties everywhere
    H, E, k = 128, 16, 4
    rng = np.random.default_rng(0)
    row = orc.f32_to_bf16(rng.normal(0, 0.02, (1, H)).astype(np.float32))
    w = np.repeat(row, E, 0)
    x = orc.f32_to_bf16(rng.normal(0, 1, (7, H)).astype(np.float32))
    gi, _ = m.ops.route(bf16_tensor(x, "cuda"), bf16_tensor(w, "cuda"), k, 0)
    assert (bits_u32(gi) == np.arange(k)).all()
    # zero activations: all logits +0
    gi, gs = m.ops.route(bf16_tensor(np.zeros((3, H), np.uint16), "cuda"), bf16_tensor(w, "cuda"), k, 2)
    assert (bits_u32(gi) == np.arange(k)).all()
    assert np.array_equal(bits_u16(gs), orc.f32_to_bf16(np.full((3, k), 0.25, np.float32)))


@pytest.mark.parametrize("P,E", [(1, 8), (8, 128), (256, 128), (4096, 8), (4097, 128), (40000, 64), (70000, 500),
                                 (1, 1), (300, 1), (5000, 1),
                                 # several blocks, each summing the others' histograms: expert counts that are
                                 # not powers of two, the largest one, pair counts around the per-block span
                                 (5000, 3), (9000, 33), (8193, 200), (20000, 512), (5120, 16), (5121, 16)])
def test_dispatch_bit_exact(orc, m, P, E):
    print(f"dispatch P={P} E={E}", flush=True)
    rng = np.random.default_rng(P)
    zipf = rng.zipf(1.3, P) % E if P > 1000 else rng.integers(0, E, P)
    flat = zipf.astype(np.uint32)
    counts, offsets, perm, inv = orc.dispatch(flat, E)
    g = m.ops.dispatch(i32_tensor(flat, "cuda"), E)
    for got, ref, name in zip(g, (counts, offsets, perm, inv), ("counts", "offsets", "perm", "inv_perm")):
        assert np.array_equal(bits_u32(got), ref), name
    assert np.array_equal(perm, np.argsort(flat, kind="stable"))


@pytest.mark.parametrize("bits,M,N,K,E,n_idx,xb", [
    (4, 32, 64, 128, 3, 2, 5),      # the reference's test shapes (K raised to a multiple of 128 for 4-bit)
    (8, 32, 64, 64, 3, 2, 1),       # ... and its exact shapes with 8-bit codes
    (4, 1, 768, 2048, 16, 40, 40), (8, 1, 256, 512, 4, 300, 300), (4, 3, 48, 256, 5, 7, 4),
    # 4-bit plain products with two token groups per pass whose rows end up staged in slabs (more blocks than
    # CUs, K = 1536 with a partial last slab and K = 2048): the launch gives up the paired row tiles and must
    # size its LDS for the kernel it then runs
    (4, 1, 512, 1536, 64, 512, 512), (4, 1, 512, 2048, 64, 768, 768), (4, 1, 1024, 2048, 40, 480, 480),
])
def test_gather_qmm_matches_oracle(orc, m, bits, M, N, K, E, n_idx, xb):
    print(f"gather_qmm bits={bits} M={M} N={N} K={K} E={E} n_idx={n_idx}", flush=True)
    rng = np.random.default_rng(N + K)
    w = rng.normal(0, 0.02, (E * N, K)).astype(np.float32)   # outputs stay below 4: one bf16 ulp < 2e-2
    q, s, b = orc.quantize(w, bits, 64)
    q, s, b = q.reshape(E, N, -1), s.reshape(E, N, -1), b.reshape(E, N, -1)
    x = orc.f32_to_bf16(rng.normal(0, 1, (xb, M, K)).astype(np.float32))
    rhs = rng.integers(0, E, n_idx).astype(np.uint32)
    lhs = None if xb == n_idx else rng.integers(0, xb, n_idx).astype(np.uint32)
    ref = orc.gather_qmm(x, q, s, b, lhs, rhs, bits, want="bf16")
    got = m.ops.gather_qmm(bf16_tensor(x, "cuda"), i32_tensor(q, "cuda"), bf16_tensor(s, "cuda"),
                           bf16_tensor(b, "cuda"), None if lhs is None else i32_tensor(lhs, "cuda"),
                           i32_tensor(rhs, "cuda"), True, 64, bits, sorted_indices=False)
    assert_close_bf16(bits_u16(got), ref, what="gather_qmm")
    # the sorted hint changes nothing (test_gather_mm_sorted, ops/arithmetic.rs:3214-3238)
    o = np.argsort(rhs, kind="stable")
    got2 = m.ops.gather_qmm(bf16_tensor(x, "cuda"), i32_tensor(q, "cuda"), bf16_tensor(s, "cuda"),
                            bf16_tensor(b, "cuda"), i32_tensor((np.arange(n_idx) if lhs is None else lhs)[o].astype(np.uint32), "cuda"),
                            i32_tensor(rhs[o], "cuda"), True, 64, bits, sorted_indices=True)
    assert np.array_equal(bits_u16(got2), bits_u16(got)[o])


def test_gather_qmm_unit_scale_is_exact(orc, m):
    rng = np.random.default_rng(9)
    E, N, K = 2, 16, 256
    codes = rng.integers(0, 16, (E, N, K)).astype(np.uint32)
    q = np.zeros((E, N, K // 8), np.uint32)
    for j in range(8):
        q |= codes[..., j::8] << np.uint32(4 * j)
    one = orc.f32_to_bf16(np.ones((E, N, K // 64), np.float32))
    zero = np.zeros((E, N, K // 64), np.uint16)
    xi = np.zeros((5, 1, K), np.int64)   # 8 entries of +-1 per row: |sum| <= 120, exact in bf16
    for j in range(5):
        xi[j, 0, rng.choice(K, 8, replace=False)] = rng.choice([-1, 1], 8)
    got = m.ops.gather_qmm(bf16_tensor(orc.f32_to_bf16(xi.astype(np.float32)), "cuda"), i32_tensor(q, "cuda"),
                           bf16_tensor(one, "cuda"), bf16_tensor(zero, "cuda"), None,
                           i32_tensor(np.array([1, 0, 1, 1, 0], np.uint32), "cuda"))
    ref = np.stack([xi[j, 0] @ codes[e].astype(np.int64).T for j, e in enumerate([1, 0, 1, 1, 0])])
    assert np.array_equal(f32_of_bits(bits_u16(got))[:, 0].astype(np.int64), ref)  # |sum| < 256: exact in bf16


def test_swiglu_and_combine(orc, m):
    rng = np.random.default_rng(3)
    # |gate|, |up| <= 1.9: |silu(gate) * up| < 4, so one bf16 ulp stays below the 2e-2 bound
    g = orc.f32_to_bf16(np.clip(rng.normal(0, 0.9, (77, 96)), -1.9, 1.9).astype(np.float32))
    u = orc.f32_to_bf16(np.clip(rng.normal(0, 0.9, (77, 96)), -1.9, 1.9).astype(np.float32))
    got = m.ops.swiglu(bf16_tensor(g, "cuda"), bf16_tensor(u, "cuda"))
    assert_close_bf16(bits_u16(got), orc.swiglu_bf16(g, u), what="swiglu vs op-by-op oracle")
    assert_close_bf16(bits_u16(got), orc.swiglu_f32(f32_of_bits(g), f32_of_bits(u)), rel_fro=3e-3,
                      what="swiglu vs single-rounding oracle")
    T, k, H = 50, 8, 2048
    y = orc.f32_to_bf16(rng.normal(0, 1, (T * k, H)).astype(np.float32))
    sc = orc.f32_to_bf16(rng.uniform(0, 0.3, (T, k)).astype(np.float32))
    inv = rng.permutation(T * k).astype(np.uint32)
    for ip in (inv, None):
        got = m.ops.combine(bf16_tensor(y, "cuda"), bf16_tensor(sc, "cuda"), None if ip is None else i32_tensor(ip, "cuda"))
        assert np.array_equal(bits_u16(got), orc.combine(y, sc, ip)), "combine is a fixed-order fp32 sum: bit-exact"


@pytest.mark.parametrize("bits,group", [(4, 64), (8, 64), (2, 64), (4, 32), (8, 128)])
def test_quantize_dequantize_bit_exact(orc, m, bits, group):
    rng = np.random.default_rng(bits + group)
    w = rng.normal(0, 0.02, (96, 4 * group)).astype(np.float32)
    w[3] = 0.0
    w[4] = 0.25
    q, s, b = orc.quantize(w, bits, group)
    gq, gs, gb = m.ops.quantize(torch.from_numpy(w).cuda(), group, bits)
    assert np.array_equal(bits_u32(gq), q) and np.array_equal(bits_u16(gs), s) and np.array_equal(bits_u16(gb), b)
    wh = m.ops.dequantize(gq, gs, gb, group, bits, dtype=torch.float32).cpu().numpy()
    assert np.array_equal(wh, orc.dequantize(q, s, b, bits, group))
    # as the reference returns it (ops/quantization.rs:124-158): in the type of the scales, one more rounding
    wn = m.ops.dequantize(gq, gs, gb, group, bits)
    assert wn.dtype == torch.bfloat16
    assert np.array_equal(bits_u16(wn), orc.f32_to_bf16(orc.dequantize(q, s, b, bits, group)))
    # the reference's known-answer case (ops/quantization.rs:298-315) on the device
    x = np.tile(np.arange(512, dtype=np.float32), (128, 1))
    gq, gs, gb = m.ops.quantize(torch.from_numpy(x).cuda(), 128, bits)
    assert tuple(gq.shape) == (128, 512 * bits // 32) and tuple(gs.shape) == (128, 4)
    xh = m.ops.dequantize(gq, gs, gb, 128, bits, dtype=torch.float32).cpu().numpy()
    assert np.abs(x - xh).max() <= 127.0 / (1 << bits) + 2.0   # + bf16 rounding of a bias near 511


def test_errors_reach_the_caller(m):
    x = torch.zeros((4, 100), dtype=torch.bfloat16, device="cuda")
    w = torch.zeros((8, 100), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(m.MoeError, match="hidden"):
        m.ops.route(x, w, 2)
    with pytest.raises(m.MoeError, match="divisible"):
        m.ops.quantize(torch.zeros((4, 100), device="cuda"), 64, 4)
    with pytest.raises(m.MoeError, match="top_k"):
        m.ops.route(torch.zeros((4, 128), dtype=torch.bfloat16, device="cuda"),
                    torch.zeros((8, 128), dtype=torch.bfloat16, device="cuda"), 9)


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("M", [1, 5, 8, 9, 64, 65, 130, 300])
def test_quantized_matmul_equals_matmul_on_dequantized(orc, bits, M):
    """The identity of the reference's test_quantized_matmul (mlx-rs/src/ops/quantization.rs:318-342),
    in the transposed layout QuantizedLinear uses: qmm(x, w_q, s, b) == x @ dequantize(w_q, s, b)^T.
    Up to 8 rows run on the streaming kernel, more on the tiled one (64-, 128- and 256-row tiles)."""
    import mlx_rs_amd as m
    rng = np.random.default_rng(50 + M)
    N, K = 192, 256
    w = (rng.normal(0, 1, (N, K)) / np.sqrt(K)).astype(np.float32)
    q, s, b = orc.quantize(w, bits, 64)
    x = orc.f32_to_bf16((rng.normal(0, 1, (M, K))).astype(np.float32))
    print(f"quantized_matmul bits={bits} M={M}", flush=True)
    y = m.ops.quantized_matmul(bf16_tensor(x, "cuda"), i32_tensor(q, "cuda"), bf16_tensor(s, "cuda"),
                               bf16_tensor(b, "cuda"), True, 64, bits)
    torch.cuda.synchronize()
    w_hat = orc.dequantize(q, s, b, bits, 64).astype(np.float64)
    ref = f32_of_bits(x).astype(np.float64) @ w_hat.T
    got = f32_of_bits(bits_u16(y)).astype(np.float64)
    assert got.shape == ref.shape
    assert np.abs(got - ref).max() <= 2e-2
    assert np.linalg.norm(got - ref) / np.linalg.norm(ref) <= 1e-2
    # and the oracle's gather_qmm with a single matrix agrees with the same identity
    yo = orc.gather_qmm(x.reshape(M, 1, K), q[None], s[None], b[None], None, np.zeros(M, np.uint32),
                        bits=bits, want="f32").reshape(M, N)
    assert np.abs(yo - ref).max() <= 1e-4


@pytest.mark.parametrize("bits", [4, 8])
def test_untransposed_quantized_matmul_and_gather_qmm(orc, bits):
    """transpose = false, the layout of the reference's test_quantized_matmul
    (mlx-rs/src/ops/quantization.rs:318-342: m 32, n 128, k 128, group 64, w = normal * 1/sqrt(k),
    quantised along n): qmm(x, w_q, s, b, false) == x @ dequantize(w_q, s, b).  The reference's bound
    is 1e-3 on float32 inputs; activations are bf16 here, so the bf16 tolerance applies."""
    import mlx_rs_amd as m
    rng = np.random.default_rng(0)
    M, N, K = 32, 128, 128
    scale = 1.0 / np.sqrt(K)
    w = (rng.normal(0, 1, (K, N)) * scale).astype(np.float32)
    x = orc.f32_to_bf16((rng.normal(0, 1, (M, K)) * scale).astype(np.float32))
    q, s, b = orc.quantize(w, bits, 64)
    y = m.ops.quantized_matmul(bf16_tensor(x, "cuda"), i32_tensor(q, "cuda"), bf16_tensor(s, "cuda"),
                               bf16_tensor(b, "cuda"), False, 64, bits)
    torch.cuda.synchronize()
    assert tuple(y.shape) == (M, N)
    ref = f32_of_bits(x).astype(np.float64) @ orc.dequantize(q, s, b, bits, 64).astype(np.float64)
    got = f32_of_bits(bits_u16(y)).astype(np.float64)
    assert np.abs(got - ref).max() <= 2e-2 and np.linalg.norm(got - ref) / np.linalg.norm(ref) <= 1e-2
    # gather form with three matrices and both index arrays; the oracle states the same identity
    E = 3
    wq = [orc.quantize((rng.normal(0, 1, (K, N)) * scale).astype(np.float32), bits, 64) for _ in range(E)]
    W, S, B = (np.stack([t[i] for t in wq]) for i in range(3))
    xs = orc.f32_to_bf16((rng.normal(0, 1, (5, 2, K)) * scale).astype(np.float32))
    lhs, rhs = np.array([4, 0, 2, 2], np.uint32), np.array([2, 1, 0, 2], np.uint32)
    yg = m.ops.gather_qmm(bf16_tensor(xs, "cuda"), i32_tensor(W, "cuda"), bf16_tensor(S, "cuda"), bf16_tensor(B, "cuda"),
                          i32_tensor(lhs, "cuda"), i32_tensor(rhs, "cuda"), transpose=False, group_size=64, bits=bits)
    torch.cuda.synchronize()
    yo = orc.gather_qmm(xs, W, S, B, lhs, rhs, bits=bits, want="f32", transpose=False)
    assert tuple(yg.shape) == yo.shape == (4, 2, N)
    for j in range(4):
        refj = f32_of_bits(xs[lhs[j]]).astype(np.float64) @ orc.dequantize(W[rhs[j]], S[rhs[j]], B[rhs[j]], bits, 64).astype(np.float64)
        assert np.abs(yo[j] - refj).max() <= 1e-4
    assert_close_bf16(bits_u16(yg), orc.f32_to_bf16(yo), what="gather_qmm, transpose = false")


def test_stream_probe_runs_and_rejects_bad_sizes():
    """The measurement aid: a launch over a small buffer succeeds and leaves the sink alone;
    sizes that are not whole 32 KiB tile pairs are refused with a message."""
    import mlx_rs_amd as m
    lib = m.capi.load_library()
    buf = torch.ones(4 * 32768, dtype=torch.uint8, device="cuda")
    sink = torch.zeros(1, dtype=torch.int32, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    m.capi.check(lib.mi_moe_stream_probe(buf.data_ptr(), 4 * 32768, sink.data_ptr(), st))
    torch.cuda.synchronize()
    assert int(sink.item()) == 0
    assert lib.mi_moe_stream_probe(buf.data_ptr(), 1000, sink.data_ptr(), st) != 0
    assert "32768" in m.capi.last_error()
    assert lib.mi_moe_stream_probe(None, 32768, sink.data_ptr(), st) != 0


def _exact_logits_f64(x_bits, w_bits, bias):
    """The definition the oracle and both device routes share, in numpy: exact products, float64 sums,
    float64 -> float32 -> bfloat16 (pins orc.router_logits from outside, on the data of these tests)."""
    from helpers import f32_of_bits
    s = f32_of_bits(x_bits).astype(np.float64) @ f32_of_bits(w_bits).astype(np.float64).T
    if bias is not None:
        s = s + bias.astype(np.float64)
    return s.astype(np.float32)


@pytest.mark.parametrize("T,H,E,bias,kind", [
    (65, 64, 1, False, "normal"), (100, 256, 8, True, "normal"), (128, 2048, 128, False, "normal"),
    (333, 4096, 200, True, "normal"), (4096, 2048, 128, True, "normal"), (97, 1024, 512, False, "normal"),
    # rows whose elements span 40 binades: many elements lose bits in fixed point, the bound sends their logits to fp64
    (200, 512, 64, True, "wide"),
    # rows of zeros, subnormals, values near the ends of the bfloat16 range, logits that cancel to (almost) nothing
    (130, 256, 40, False, "edge"),
    # infinities and NaNs in x and in the router matrix
    (70, 128, 16, False, "nonfinite"),
])
def test_router_logits_on_the_int8_matrix_cores_have_the_fp64_bits(orc, m, T, H, E, bias, kind):
    """mi_moe_router_logits above 64 tokens (integer arithmetic + a checked error bound + fp64 where the bound does
    not decide) against the oracle's fp64 accumulation, bit for bit."""
    print(f"router logits T={T} H={H} E={E} bias={bias} {kind}", flush=True)
    rng = np.random.default_rng(T * 7 + E)
    xf = rng.normal(0, 1, (T, H)).astype(np.float32)
    wf = rng.normal(0, 0.02, (E, H)).astype(np.float32)
    if kind == "wide":
        xf *= np.exp2(rng.integers(-40, 1, (T, H))).astype(np.float32)
        wf *= np.exp2(rng.integers(-30, 1, (E, H))).astype(np.float32)
    if kind == "edge":
        xf[0] = 0.0                                   # a token of zeros
        xf[1] = 1e-40                                 # subnormal bfloat16 values
        xf[2] = rng.normal(0, 1, H) * 1e-30
        xf[3] = rng.normal(0, 1, H) * 1e18
        xf[4, : H // 2] = 1.0
        xf[4, H // 2:] = -1.0                         # against a constant router row: exact cancellation
        xf[5] = xf[4]
        xf[5, 0] = 1.0 + 2.0 ** -7                    # ... and cancellation down to one last place
        wf[0] = 0.5
        wf[1] = 0.0
        wf[2] = rng.normal(0, 1, H) * 1e-25
        wf[3] = rng.normal(0, 1, H) * 1e15
        wf[4, ::2] = 1e-38
    x, w = orc.f32_to_bf16(xf), orc.f32_to_bf16(wf)
    if kind == "nonfinite":
        x[3, 5] = 0x7F80   # +inf
        x[9, 0] = 0x7FC0   # NaN
        w[2, 7] = 0xFF80   # -inf
    b = rng.normal(0, 1, E).astype(np.float32) if bias else None
    got = bits_u16(m.ops.router_logits(bf16_tensor(x, "cuda"), bf16_tensor(w, "cuda"),
                                       None if b is None else torch.from_numpy(b).cuda()))
    torch.cuda.synchronize()
    ref = orc.router_logits(x, w, b)
    if kind == "nonfinite":
        from helpers import f32_of_bits
        g, r = f32_of_bits(got), f32_of_bits(ref)
        assert np.array_equal(np.isnan(g), np.isnan(r)) and np.isnan(r).any()
        ok = ~np.isnan(r)
        assert np.array_equal(got[ok], ref[ok])
        return
    bad = np.argwhere(got != ref)
    assert len(bad) == 0, (f"{len(bad)} of {got.size} logits differ from the fp64 accumulation; first (token, expert, got, oracle): "
                           f"{[(int(t), int(e), hex(got[t, e]), hex(ref[t, e])) for t, e in bad[:8]]}")
    if kind == "normal" and T * E * H <= 2 ** 28:
        assert np.array_equal(orc.f32_to_bf16(_exact_logits_f64(x, w, b)), ref), "the oracle itself against numpy float64"
    # the fp64 route (mi_moe_route's) gives the same bits
    _, _, gl = m.ops.route(bf16_tensor(x, "cuda"), bf16_tensor(w, "cuda"), 1, 0,
                           None if b is None else torch.from_numpy(b).cuda(), return_logits=True)
    assert np.array_equal(bits_u16(gl), ref)
