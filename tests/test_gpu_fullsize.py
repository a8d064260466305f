"""The block at the full sizes of the benchmark configurations, checked through properties that do
not need the CPU checker to run the whole batch:
  * token-permutation equivariance, bit for bit: a token's result depends on the token only,
    not on where it sits in the batch, in a tile or in an expert's segment;
  * the integer invariants of routing and dispatch (what a stable argsort / bincount give);
  * a subsample of tokens against the oracle run on those tokens alone (routing is per token, so
    the oracle selects the same experts), within the stated tolerance: max-abs 2e-2 (at unit
    output scale), relative Frobenius 1e-2 in bf16.
"""
import numpy as np
import pytest
import torch

from helpers import assert_close_bf16, bits_u16, bits_u32, f32_of_bits

pytestmark = pytest.mark.gpu

CASES = [
    # config, tokens, zipf s
    ("qwen3_30b_a3b", 1, None),     # K split over the waves: scale/bias tiles of a wave's K range
    ("qwen3_30b_a3b", 4, None),
    ("qwen3_30b_a3b", 24, None),    # 1.5 rows per expert: short segments, five rows per pass and four blocks per CU
    ("qwen3_30b_a3b", 32, None),
    ("qwen3_30b_a3b", 48, None),    # 3 rows per expert: eight rows per pass
    ("qwen3_30b_a3b", 160, None),   # 10 rows per expert: two token groups per pass, rows staged in slabs of 1024
    ("qwen3_30b_a3b", 200, 1.1),    # light batch, uneven routing: long segments tiled beside the streamed ones
    ("qwen3_30b_a3b", 4096, 1.1),
    ("mixtral_8x7b", 1, None),
    ("mixtral_8x7b", 4, None),    # streamed; the down product's rows (K = 14336) and their scales go through LDS in slabs
    ("mixtral_8x7b", 16, None),
    ("mixtral_8x7b", 64, None),   # streamed, 16 rows per expert
    ("mixtral_8x7b", 96, None),   # 64-row tiles
    ("mixtral_8x7b", 2048, None),
    ("qwen3_235b_a22b", 2, None),   # K split over the waves, rows of 4096 4-bit values
    ("qwen3_235b_a22b", 32, None),  # streamed, 4-bit rows of 4096 values (two blocks per CU)
    ("qwen3_235b_a22b", 8192, 1.3),
]


def _host_weights(blk):
    bank = lambda b: (bits_u32(b.weight), bits_u16(b.scales), bits_u16(b.biases))
    return dict(router_w=bits_u16(blk.gate_weight),
                router_bias=None if blk.router_bias is None else blk.router_bias.cpu().numpy(),
                gate=bank(blk.gate_proj), up=bank(blk.up_proj), down=bank(blk.down_proj))


@pytest.mark.parametrize("name,T,zipf", CASES, ids=[f"{n}-T{t}" for n, t, _ in CASES])
def test_full_size_properties(orc, name, T, zipf):
    import mlx_rs_amd as m
    from mlx_rs_amd import synth
    cfg = synth.CONFIGS[name]
    print(f"full size {name} T={T} zipf={zipf}", flush=True)
    blk = synth.make_block(cfg, seed=3, device="cuda", zipf_s=zipf, gen_device="cuda")
    x = synth.make_tokens(cfg, T, seed=3, device="cuda")
    out, dbg = blk.forward(x, debug=True)
    torch.cuda.synchronize()
    E, k, P = cfg.n_experts, cfg.top_k, T * cfg.top_k

    # integer invariants
    idx = bits_u32(dbg["topk_idx"]).reshape(T, k).astype(np.int64)
    counts, offsets = bits_u32(dbg["counts"]).astype(np.int64), bits_u32(dbg["offsets"]).astype(np.int64)
    perm, inv = bits_u32(dbg["perm"]).astype(np.int64), bits_u32(dbg["inv_perm"]).astype(np.int64)
    assert idx.min() >= 0 and idx.max() < E
    assert (np.sort(idx, axis=1)[:, 1:] != np.sort(idx, axis=1)[:, :-1]).all(), "a token picked an expert twice"
    assert np.array_equal(counts, np.bincount(idx.reshape(-1), minlength=E))
    assert counts.sum() == P and offsets[0] == 0 and np.array_equal(offsets[1:], np.cumsum(counts))
    assert np.array_equal(perm, np.argsort(idx.reshape(-1), kind="stable"))
    assert np.array_equal(inv[perm], np.arange(P))
    sc = bits_u16(dbg["topk_w"]).astype(np.uint32) << 16
    sums = sc.view(np.float32).reshape(T, k).sum(1)
    if cfg.score_mode != m.capi.SCORE_SOFTMAX_THEN_TOPK:
        assert np.abs(sums - 1.0).max() <= 2e-2

    # permutation equivariance, bit for bit
    if T > 1:
        g = torch.Generator().manual_seed(5)
        p = torch.randperm(T, generator=g).cuda()
        out_p = blk.forward(x[p].contiguous())
        torch.cuda.synchronize()
        assert torch.equal(out_p.view(torch.int16), out[p].view(torch.int16)), "result depends on the token's position"

    # a subsample against the oracle
    S = min(T, 12)
    pick = np.linspace(0, T - 1, S).astype(np.int64)
    W = _host_weights(blk)
    xs = np.ascontiguousarray(bits_u16(x)[pick])
    ocfg = orc.make_config(cfg.hidden, E, k, cfg.intermediate, cfg.bits, cfg.group_size, cfg.score_mode)
    ref, d = orc.moe_forward(ocfg, W, xs, strict=True, n_threads=16)
    assert np.array_equal(d["topk_idx"].astype(np.int64), idx[pick]), "selection differs from the oracle"
    assert np.array_equal(d["topk_w"], bits_u16(dbg["topk_w"]).reshape(T, k)[pick]), "scores differ from the oracle"
    # the absolute bound is stated for outputs of unit scale; Mixtral's outputs reach |8|, where one
    # bf16 ulp is already 3e-2, so it scales with the largest reference value (never below 2e-2)
    scale = max(1.0, float(np.abs(f32_of_bits(ref)).max()))
    mx, rel = assert_close_bf16(bits_u16(out)[pick], ref, max_abs=2e-2 * scale, what=f"{name} T={T} subsample vs oracle")
    print(f"  subsample of {S} tokens: max-abs {mx:.2e} rel-fro {rel:.2e}", flush=True)
