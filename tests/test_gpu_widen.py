"""The op-level entry points beyond the hot path's own shapes: activations in float32 and float16,
group sizes 32 and 128, 2-bit codes, index arrays of any broadcastable shapes.

The first three tests are the reference's own tests of these ops, run as written (float32 inputs,
its shapes, its bounds): mlx-rs/src/ops/quantization.rs:298-315 (test_quantize_dequantize),
:318-342 (test_quantized_matmul: transpose = false, max difference < 1e-3) and :345-423
(test_gather_qmm: gather_qmm against gather_mm on the dequantised weights, all_close at 1e-4).
The dense side of each identity (matmul of the dequantised weights) is computed here in float64."""
import numpy as np
import pytest
import torch

from helpers import assert_close_bf16, bf16_tensor, bits_u16, bits_u32, device_block, host_layer, host_tokens, i32_tensor

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def m():
    import mlx_rs_amd as mod
    mod.load_library()
    return mod


def test_reference_quantize_dequantize_in_float32(orc, m):
    # x[r, c] = c for 128 rows of 512 columns; group 128; bits 2, 4, 8
    x = (torch.ones(128, 1) * torch.arange(512, dtype=torch.float32)[None, :]).cuda()
    for bits in (2, 4, 8):
        q, s, b = m.ops.quantize(x, 128, bits, dtype=torch.float32)
        assert tuple(q.shape) == (128, 512 * bits // 32) and tuple(s.shape) == (128, 4) and tuple(b.shape) == (128, 4)
        assert s.dtype == torch.float32 and b.dtype == torch.float32
        x_hat = m.ops.dequantize(q, s, b, 128, bits)
        assert (x - x_hat).abs().max().item() <= 127.0 / (1 << bits)
        # and the checker's bits: codes, fp32 scales and biases
        qo, so, bo = orc.quantize(x.cpu().numpy(), bits, 128, scale_dtype="f32")
        assert np.array_equal(bits_u32(q), qo)
        assert np.array_equal(s.cpu().numpy(), so) and np.array_equal(b.cpu().numpy(), bo)


def test_reference_quantized_matmul_in_float32(m):
    torch.manual_seed(0)
    group_size, bits, mm, n, k = 64, 4, 32, 128, 128
    scale = 1.0 / k ** 0.5
    x = (torch.randn(mm, k) * scale).cuda()
    w = (torch.randn(k, n) * scale).cuda()
    w_q, scales, biases = m.ops.quantize(w, group_size, bits, dtype=torch.float32)
    w_hat = m.ops.dequantize(w_q, scales, biases, group_size, bits)
    y_q = m.ops.quantized_matmul(x, w_q, scales, biases, False, group_size, bits)
    y_hat = (x.double() @ w_hat.double()).float()
    assert y_q.shape == y_hat.shape and y_q.dtype == torch.float32
    max_diff = (y_q - y_hat).abs().max().item()
    print(f"  quantized_matmul float32: max difference {max_diff:.2e}", flush=True)
    assert max_diff < 1e-3


def test_reference_gather_qmm_in_float32(m):
    torch.manual_seed(0)
    group_size, bits, mm, n, k = 64, 4, 32, 64, 64
    w = torch.randn(3, n, k).cuda()  # the transpose = true shape
    w_q, scales, biases = m.ops.quantize(w.reshape(3 * n, k), group_size, bits, dtype=torch.float32)
    w_hat = m.ops.dequantize(w_q, scales, biases, group_size, bits).reshape(3, n, k)
    w_q, scales, biases = w_q.reshape(3, n, -1), scales.reshape(3, n, -1), biases.reshape(3, n, -1)
    rhs = torch.tensor([2, 1], dtype=torch.int32).cuda()
    # case 1: x batch (1,), lhs_indices (0,) broadcast against rhs_indices (2, 1); case 2: x batch (5,), lhs (0, 2)
    for xb, lhs_list in ((1, [0]), (5, [0, 2])):
        x = torch.randn(xb, mm, k).cuda()
        lhs = torch.tensor(lhs_list, dtype=torch.int32).cuda()
        c2 = m.ops.gather_qmm(x, w_q, scales, biases, lhs, rhs, True, group_size, bits)
        li = lhs.long().expand(2) if len(lhs_list) == 1 else lhs.long()
        c1 = torch.matmul(x[li].double(), w_hat[rhs.long()].double().transpose(-1, -2)).float()  # gather_mm
        assert c2.shape == c1.shape == (2, mm, n)
        assert torch.allclose(c1, c2, rtol=1e-4, atol=1e-4), f"x batch {xb}: max difference {(c1 - c2).abs().max().item():.2e}"


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-5), (torch.float16, 2e-3)])
@pytest.mark.parametrize("bits,group,transpose", [(4, 64, True), (8, 32, True), (2, 128, True), (4, 32, False), (8, 128, False)])
def test_typed_products_against_float64(m, dtype, tol, bits, group, transpose):
    """Random codes, scales and biases (so nothing depends on a quantizer): every element type, group
    size, bit width and weight layout of the plain kernels against the same sum in float64."""
    g = torch.Generator().manual_seed(bits * 1000 + group)
    E, M, N, K, n_idx = 3, 5, 128, 256, 7
    q_axis, other = (K, N) if transpose else (N, K)
    codes = torch.randint(0, 1 << bits, (E, other, q_axis), generator=g)
    per = 32 // bits
    words = torch.zeros((E, other, q_axis // per), dtype=torch.int64)
    for j in range(per):
        words |= codes[..., j::per] << (j * bits)
    w_q = torch.from_numpy(words.numpy().astype(np.uint32).view(np.int32))
    scales = (torch.rand((E, other, q_axis // group), generator=g) * 0.02 + 0.001).to(dtype)
    biases = (torch.randn((E, other, q_axis // group), generator=g) * 0.05).to(dtype)
    x = torch.randn((4, M, K), generator=g).to(dtype)
    lhs = torch.randint(0, 4, (n_idx,), generator=g, dtype=torch.int32)
    rhs = torch.randint(0, E, (n_idx,), generator=g, dtype=torch.int32)
    w_hat = scales.double().repeat_interleave(group, -1) * codes.double() + biases.double().repeat_interleave(group, -1)
    wm = w_hat[rhs.long()]  # [n_idx, other, q_axis]
    ref = torch.matmul(x[lhs.long()].double(), wm.transpose(-1, -2) if transpose else wm)
    got = m.ops.gather_qmm(x.cuda(), w_q.cuda(), scales.cuda(), biases.cuda(), lhs.cuda(), rhs.cuda(), transpose, group, bits)
    assert got.dtype == dtype and tuple(got.shape) == (n_idx, M, N)
    err = (got.double().cpu() - ref).abs().max().item()
    scale = ref.abs().max().item()
    print(f"  {dtype} bits={bits} group={group} transpose={transpose}: max error {err:.2e} at output scale {scale:.2f}", flush=True)
    assert err <= tol * max(1.0, scale)
    # quantized_matmul is the same product on one matrix
    got1 = m.ops.quantized_matmul(x.cuda(), w_q[1].contiguous().cuda(), scales[1].contiguous().cuda(),
                                  biases[1].contiguous().cuda(), transpose, group, bits)
    ref1 = torch.matmul(x.double(), w_hat[1].transpose(-1, -2) if transpose else w_hat[1])
    assert tuple(got1.shape) == (4, M, N)
    assert (got1.double().cpu() - ref1).abs().max().item() <= tol * max(1.0, ref1.abs().max().item())


@pytest.mark.parametrize("bits,group", [(4, 32), (4, 128), (8, 32), (8, 128), (2, 64), (2, 32)])
def test_other_group_sizes_in_bf16_match_the_oracle(orc, m, bits, group):
    rng = np.random.default_rng(bits * 7 + group)
    E, N, K, M, xb, n_idx = 4, 96, 256, 3, 6, 9
    w = rng.normal(0, 0.02, (E * N, K)).astype(np.float32)
    q, s, b = orc.quantize(w, bits, group)
    q, s, b = q.reshape(E, N, -1), s.reshape(E, N, -1), b.reshape(E, N, -1)
    # the device quantizer gives the checker's bits for these group sizes too
    qd, sd, bd = m.ops.quantize(torch.from_numpy(w).cuda(), group, bits)
    assert np.array_equal(bits_u32(qd).reshape(q.shape), q) and np.array_equal(bits_u16(sd).reshape(s.shape), s)
    assert np.array_equal(bits_u16(bd).reshape(b.shape), b)
    x = orc.f32_to_bf16(rng.normal(0, 1, (xb, M, K)).astype(np.float32))
    lhs = rng.integers(0, xb, n_idx).astype(np.uint32)
    rhs = rng.integers(0, E, n_idx).astype(np.uint32)
    ref = orc.gather_qmm(x, q, s, b, lhs, rhs, bits, group, want="bf16")
    got = m.ops.gather_qmm(bf16_tensor(x, "cuda"), i32_tensor(q, "cuda"), bf16_tensor(s, "cuda"), bf16_tensor(b, "cuda"),
                           i32_tensor(lhs, "cuda"), i32_tensor(rhs, "cuda"), True, group, bits)
    assert_close_bf16(bits_u16(got), ref, what=f"gather_qmm bits {bits} group {group}")


@pytest.mark.parametrize("bits,group,T", [(4, 32, 40), (4, 128, 9), (8, 128, 70), (2, 64, 33)])
def test_block_with_other_group_sizes_matches_the_oracle(orc, m, bits, group, T):
    """The whole block on weights in groups of 32 or 128 (or 2-bit codes): routing bit for bit,
    outputs within the tolerance rule, both through the router's one-launch and separate forms."""
    H, E, k, I = 256, 8, 2, 384
    rng = np.random.default_rng(group + T)

    def bank(N, K):
        w = rng.normal(0.0, 0.02, (E * N, K)).astype(np.float32)
        q, s, b = orc.quantize(w, bits, group)
        return q.reshape(E, N, -1), s.reshape(E, N, -1), b.reshape(E, N, -1)

    W = dict(router_w=orc.f32_to_bf16(rng.normal(0.0, 0.02, (E, H)).astype(np.float32)), router_bias=None,
             gate=bank(I, H), up=bank(I, H), down=bank(H, I))
    x = host_tokens(orc, T, H, seed=T)
    blk = device_block(m, m.MoeConfig(H, E, k, I, bits, group, 0), W)
    out, dbg = blk.forward(bf16_tensor(x, "cuda"), debug=True)
    torch.cuda.synchronize()
    ref, d = orc.moe_forward(orc.make_config(H, E, k, I, bits, group, 0), W, x, strict=True, n_threads=8)
    for name in ("topk_idx", "counts", "perm"):
        assert np.array_equal(bits_u32(dbg[name]).reshape(d[name].shape), d[name]), name
    assert_close_bf16(bits_u16(out), ref, what=f"block bits {bits} group {group} T {T}")


def test_index_arrays_broadcast_and_batches_flatten(m):
    """x [2, 3, M, K] (batch of 6), w [2, 2, N, K/8] (batch of 4): lhs_indices [2, 1] against
    rhs_indices [1, 3] gives [2, 3, M, N]; an absent lhs counts through x's batch."""
    g = torch.Generator().manual_seed(5)
    M, N, K = 2, 32, 128
    x = torch.randn((2, 3, M, K), generator=g).cuda()
    w = (torch.randn((4 * N, K), generator=g) * 0.05).cuda()
    w_q, s, b = m.ops.quantize(w, 64, 4, dtype=torch.float32)
    w_hat = m.ops.dequantize(w_q, s, b, 64, 4).reshape(4, N, K)
    w_q, s, b = (t.reshape(2, 2, N, -1) for t in (w_q, s, b))
    lhs = torch.tensor([[5], [1]], dtype=torch.int32).cuda()
    rhs = torch.tensor([[3, 0, 2]], dtype=torch.int32).cuda()
    y = m.ops.gather_qmm(x, w_q, s, b, lhs, rhs, True, 64, 4)
    assert tuple(y.shape) == (2, 3, M, N)
    xf = x.reshape(6, M, K)
    for i in range(2):
        for j in range(3):
            want = xf[int(lhs[i, 0])].double() @ w_hat[int(rhs[0, j])].double().T
            assert torch.allclose(y[i, j].double(), want, rtol=1e-4, atol=1e-4), (i, j)
    # no lhs_indices: arange over x's batch, in x's batch shape, broadcast against rhs [3]
    rhs3 = torch.tensor([1, 1, 2], dtype=torch.int32).cuda()
    y2 = m.ops.gather_qmm(x, w_q, s, b, None, rhs3, True, 64, 4)
    assert tuple(y2.shape) == (2, 3, M, N)
    for i in range(2):
        for j in range(3):
            want = x[i, j].double() @ w_hat[int(rhs3[j])].double().T
            assert torch.allclose(y2[i, j].double(), want, rtol=1e-4, atol=1e-4), (i, j)
    with pytest.raises(m.MoeError, match="broadcast"):
        m.ops.gather_qmm(x, w_q, s, b, torch.zeros(2, dtype=torch.int32).cuda(), rhs3, True, 64, 4)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_indices_out_of_range_are_clamped_not_followed(m, dtype):
    """Index values live in device memory, so the call cannot check them: an index past the last
    matrix must read the last matrix, never memory beyond the operand.  The operands here are the
    leading parts of larger tensors (4 of 8 weight matrices, 2 of 10 x matrices), so that an index
    that were followed would land in memory the test owns and give a different result."""
    torch.manual_seed(3)
    group_size, bits, M, N, K = 64, 4, 2, 64, 128
    w_big = (torch.randn(8, N, K) * 0.05).cuda()
    q, s, b = m.ops.quantize(w_big.reshape(8 * N, K), group_size, bits, dtype=dtype)
    q, s, b = q.reshape(8, N, -1), s.reshape(8, N, -1), b.reshape(8, N, -1)
    x_big = torch.randn(10, M, K).cuda().to(dtype)
    x, qw, sw, bw = x_big[:2], q[:4], s[:4], b[:4]  # same base pointers, fewer matrices
    lhs = torch.tensor([0, 1, 9, 1, 0, 5], dtype=torch.int32, device="cuda")
    rhs = torch.tensor([3, 7, 1, 4, 2, 6], dtype=torch.int32, device="cuda")
    got = m.ops.gather_qmm(x, qw, sw, bw, lhs, rhs, True, group_size, bits)
    want = m.ops.gather_qmm(x, qw, sw, bw, lhs.clamp(max=1), rhs.clamp(max=3), True, group_size, bits)
    assert torch.equal(got.view(torch.int16 if dtype == torch.bfloat16 else torch.int32),
                       want.view(torch.int16 if dtype == torch.bfloat16 else torch.int32))
    # without lhs_indices every index needs its own matrix in x
    lib = m.capi.load_library()
    y = torch.empty(3, M, N, dtype=torch.bfloat16, device="cuda")
    rc = lib.mi_moe_gather_qmm(x.data_ptr(), qw.data_ptr(), sw.data_ptr(), bw.data_ptr(), None, rhs.data_ptr(), 3, 2, M, N, K,
                               4, 1, group_size, bits, 0, y.data_ptr(), None, 0, None)
    assert rc != 0 and b"need as many matrices in x" in lib.mi_moe_last_error()


@pytest.mark.parametrize("dtype,bits,group,M", [(torch.bfloat16, 4, 64, 3), (torch.bfloat16, 8, 64, 300),
                                                (torch.float32, 4, 128, 5), (torch.float16, 2, 32, 2)])
def test_quantized_linear_adds_its_bias(m, dtype, bits, group, M):
    """QuantizedLinear::forward (mlx-rs/src/nn/quantized.rs:363-386): quantized_matmul(transpose = true), then
    `+ bias`.  Against the two ops done separately (bit for bit: the entry point rounds where they round) and
    against float64."""
    g = torch.Generator().manual_seed(bits * 10 + M)
    N, K = 192, 256
    w = (torch.randn((N, K), generator=g) * 0.05).cuda()
    w_q, s, b = m.ops.quantize(w, group, bits, dtype=dtype)
    x = torch.randn((M, K), generator=g).to(dtype).cuda()
    lb = torch.randn((N,), generator=g).to(dtype).cuda()
    y = m.ops.quantized_linear(x, w_q, s, b, lb, True, group, bits)
    y0 = m.ops.quantized_matmul(x, w_q, s, b, True, group, bits)
    torch.cuda.synchronize()
    assert y.dtype == dtype and tuple(y.shape) == (M, N)
    assert torch.equal(y, (y0.float() + lb.float()).to(dtype)), "not the reference's two ops"
    assert torch.equal(m.ops.quantized_linear(x, w_q, s, b, None, True, group, bits), y0)
    w_hat = m.ops.dequantize(w_q, s, b, group, bits, dtype=torch.float32).double()
    ref = x.double() @ w_hat.T + lb.double()
    tol = 2e-2 if dtype == torch.bfloat16 else (4e-3 if dtype == torch.float16 else 1e-4)
    assert (y.double() - ref).abs().max().item() <= tol * max(1.0, ref.abs().max().item())
    with pytest.raises(m.capi.MoeError):
        m.ops.quantized_linear(x, w_q, s, b, lb[:-1].contiguous(), True, group, bits)


def test_operand_shapes_are_checked_against_each_other(m):
    """A call in the reference's default layout (transpose = false, w [K, N*bits/32]) whose operands belong to
    the other layout is refused by the host layer instead of being read past its ends."""
    g = torch.Generator().manual_seed(1)
    N, K = 64, 256
    w_q, s, b = m.ops.quantize((torch.randn((N, K), generator=g) * 0.05).cuda(), 64, 4)  # [N, K/8]: the transposed layout
    x = torch.randn((2, K), generator=g).to(torch.bfloat16).cuda()
    with pytest.raises(m.capi.MoeError, match="K ="):
        m.ops.quantized_matmul(x, w_q, s, b)               # default transpose = False, as the reference's
    y = m.ops.quantized_matmul(x, w_q, s, b, True)
    assert tuple(y.shape) == (2, N)
    with pytest.raises(m.capi.MoeError, match="scales"):
        m.ops.quantized_matmul(x, w_q, s[:, :-1].contiguous(), b[:, :-1].contiguous(), True)
    with pytest.raises(m.capi.MoeError, match="scales"):
        m.ops.gather_qmm(x.reshape(2, 1, K), w_q.reshape(1, N, -1), s.reshape(1, N, -1)[:, :-1].contiguous(),
                         b.reshape(1, N, -1)[:, :-1].contiguous(), rhs_indices=torch.zeros(2, dtype=torch.int32, device="cuda"))
