"""Seeded random shapes through the operator-level entry points and the whole block.

The launch rules of the kernels switch paths on many thresholds at once (rows per expert, blocks per
CU, row length, LDS per block); hand-picked cases sit on the switches their author thought of.  These
draws are what found a wrong LDS size in a path no hand-picked case reached (a 4-bit plain product with
two token groups per pass whose rows ended up in slabs)."""
import random

import numpy as np
import pytest
import torch

from helpers import assert_close_bf16, bits_u16, bits_u32, bf16_tensor, device_block, host_layer, host_tokens

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def m():
    import mlx_rs_amd as mod
    mod.load_library()
    return mod


@pytest.mark.parametrize("seed", [5, 99])
def test_random_gather_qmm_and_quantized_matmul_against_float64(m, seed):
    """gather_qmm == gather_mm on the dequantised weights (the identity of test_gather_qmm,
    mlx-rs/src/ops/quantization.rs:345-423) and quantized_matmul == matmul on them (:318-342), in bf16 on
    the tuned kernels: 250 draws of (bits, M, N, K, experts, rows per expert, lhs present or not, even or
    skewed expert choice) per seed, each output row within 2e-2 of its scale (at least 1) and 1e-2 in relative
    Frobenius norm of the float64 product."""
    rnd = random.Random(seed)
    done = 0
    for case in range(400):
        bits = rnd.choice([4, 4, 8])
        K = rnd.choice([128, 256, 512, 768, 1024, 1536, 2048, 2560, 3072, 4096, 4608, 6144])
        N = rnd.choice([16, 32, 48, 64, 128, 256, 512, 768, 1024, 2048])
        E = rnd.choice([1, 2, 3, 8, 16, 33, 64, 128])
        M = rnd.choice([1, 1, 1, 2, 3, 8])
        # rows per expert decide most path switches: drawn relative to the number of experts
        n_idx = max(1, int(rnd.choice([0.3, 1, 2, 4, 6, 8, 9, 12, 16, 17, 24, 40, 100]) * E / M))
        use_lhs = rnd.random() < 0.5
        xb = rnd.choice([1, 3, 17]) if use_lhs else n_idx
        skew = rnd.random() < 0.4
        Mq = rnd.choice([1, 5, 16, 33, 100, 300, 1000])
        if n_idx * M * N * K > 3e10 or E * N * K > 2e8 or done >= 250:
            continue
        done += 1
        torch.manual_seed(1000 * seed + case)
        tag = f"draw {case}: bits={bits} M={M} N={N} K={K} E={E} n_idx={n_idx} x batch={xb} skewed={skew}"
        w = torch.randn(E * N, K, device="cuda") * 0.05
        q, s, b = m.ops.quantize(w, 64, bits)
        w_hat = m.ops.dequantize(q, s, b, 64, bits, dtype=torch.float32).reshape(E, N, K)
        q, s, b = q.reshape(E, N, -1), s.reshape(E, N, -1), b.reshape(E, N, -1)
        x = torch.randn(xb, M, K, device="cuda").to(torch.bfloat16)
        if skew:
            rhs = (torch.rand(n_idx, device="cuda").pow(3) * E).long().clamp(max=E - 1).to(torch.int32)
        else:
            rhs = torch.randint(0, E, (n_idx,), device="cuda", dtype=torch.int32)
        lhs = torch.randint(0, xb, (n_idx,), device="cuda", dtype=torch.int32) if use_lhs else None
        y = m.ops.gather_qmm(x, q, s, b, lhs, rhs, True, 64, bits)
        xs = x[lhs.long()] if use_lhs else x
        ref = torch.empty(n_idx, M, N, dtype=torch.float64, device="cuda")
        for j0 in range(0, n_idx, 256):
            sl = slice(j0, min(n_idx, j0 + 256))
            ref[sl] = torch.einsum("jmk,jnk->jmn", xs[sl].double(), w_hat[rhs[sl].long()].double())
        err = (y.double() - ref).abs()
        worst = (err / ref.abs().amax(dim=2, keepdim=True).clamp(min=1.0)).max().item()
        rel = (err.pow(2).sum() / ref.pow(2).sum().clamp(min=1e-30)).sqrt().item()
        assert worst <= 2e-2 and rel <= 1e-2, f"{tag}: worst error {worst:.3e} of the row's scale, relative Frobenius {rel:.3e}"
        if case % 3 == 0:
            xq = torch.randn(Mq, K, device="cuda").to(torch.bfloat16)
            yq = m.ops.quantized_matmul(xq, q[0], s[0], b[0], True, 64, bits)
            rq = xq.double() @ w_hat[0].double().T
            worst = ((yq.double() - rq).abs() / rq.abs().amax(dim=1, keepdim=True).clamp(min=1.0)).max().item()
            assert worst <= 2e-2, f"{tag}: quantized_matmul of {Mq} rows: worst error {worst:.3e} of the row's scale"
    assert done == 250


def test_random_block_shapes_against_the_oracle(orc, m):
    """40 draws of (hidden, intermediate, experts, top-k, bits, score mode, routing skew, tokens) through
    mi_moe_forward against both rounding modes of the oracle: integers and scores bit-exact, outputs under the
    tolerance rule, and mi_moe_forward_static (where the batch fits its scratch) bit-identical."""
    rnd = random.Random(11)
    for case in range(40):
        bits = rnd.choice([4, 8])
        H = rnd.choice([128, 256, 384, 512, 1024, 2048])
        I = rnd.choice([128, 256, 512, 768, 1024, 1536, 2048, 2560, 3072])
        E = rnd.choice([1, 2, 3, 5, 8, 16, 33, 64, 128, 200])
        k = rnd.randint(1, min(E, 8))
        # rows per expert decide most path switches: the batch is drawn relative to experts / top-k
        T = min(600, max(1, int(rnd.choice([0.3, 1, 2, 4, 6, 8, 9, 12, 16, 17, 20, 24, 40, 70, 130]) * E / k)))
        mode = rnd.choice([0, 1, 2])
        zipf = rnd.choice([None, None, 1.2])
        seed = rnd.randint(0, 10000)
        print(f"draw {case}: H={H} E={E} k={k} I={I} bits={bits} T={T} mode={mode} zipf={zipf} seed={seed}", flush=True)
        W = host_layer(orc, H, E, k, I, bits, seed, zipf_s=zipf)
        x = host_tokens(orc, T, H, seed)
        blk = device_block(m, m.MoeConfig(H, E, k, I, bits, 64, mode), W)
        xt = bf16_tensor(x, "cuda")
        out, dbg = blk.forward(xt, debug=True)
        torch.cuda.synchronize()
        ocfg = orc.make_config(H, E, k, I, bits, 64, mode)
        ref_f, d = orc.moe_forward(ocfg, W, x, strict=False, n_threads=16)
        ref_s, _ = orc.moe_forward(ocfg, W, x, strict=True, n_threads=16)
        for name in ("topk_idx", "counts", "offsets", "perm", "inv_perm"):
            assert np.array_equal(bits_u32(dbg[name]).reshape(d[name].shape), d[name]), name
        assert np.array_equal(bits_u16(dbg["topk_w"]), d["topk_w"]), "scores"
        got = bits_u16(out)
        assert_close_bf16(got, ref_f, what="vs oracle (fused rounding points)", quiet=True)
        assert_close_bf16(got, ref_s, what="vs oracle (op-by-op rounding)", quiet=True)
        try:
            out2 = blk.forward_static(xt)
        except m.capi.MoeError:
            continue  # the batch needs more than the built-in scratch
        torch.cuda.synchronize()
        assert torch.equal(out2.view(torch.int16), out.view(torch.int16)), "mi_moe_forward_static differs from mi_moe_forward"
