"""The block at the full sizes of the benchmark configurations:
  * token-permutation equivariance, bit for bit: a token's result depends on the token only,
    not on where it sits in the batch, in a tile or in an expert's segment;
  * the integer invariants of routing and dispatch (what a stable argsort / bincount give);
  * at least 512 tokens (all of them up to 512) against the oracle run on those tokens alone
    (routing is per token, so the oracle selects the same experts), under the tolerance rule of
    helpers.py.  The tokens are chosen from the realised routing so that every expert that received
    rows, every M tile of every tile class (full 256-row tiles and 256-, 128- and 64-row remainder
    tiles, each with its last row), and the streamed short segments are compared; the test asserts
    that coverage.
"""
import numpy as np
import pytest
import torch

from helpers import assert_close_bf16, bits_u16, bits_u32

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
    ("mixtral_8x7b", 320, None),  # 80 rows per expert: 128-row tiles
    ("mixtral_8x7b", 2048, None),
    ("qwen3_235b_a22b", 2, None),   # K split over the waves, rows of 4096 4-bit values
    ("qwen3_235b_a22b", 32, None),  # streamed, 4-bit rows of 4096 values (two blocks per CU)
    ("qwen3_235b_a22b", 160, None), # 10 rows per expert: two token groups per pass; the down product's rows of 1536 values in slabs of 1024 + 512
    ("qwen3_235b_a22b", 384, 1.3),  # light batch, uneven routing
    ("qwen3_235b_a22b", 8192, 1.3),
]


MIN_ORACLE_TOKENS = 512

# Share of the compared elements that may lie beyond the flat 2e-2 (they are then held by the row-scaled
# rule of helpers.py).  Zero for the shapes whose outputs stay within [-1, 1]; the Mixtral-shaped layer's
# outputs reach |11| (one bf16 ulp of a value in [8, 16) is 6.25e-2), measured share 6.4 %; the
# Qwen3-235B-shaped layer's reach |3.3| with Zipf routing at a few hundred tokens (21 of 1.57 M elements).
OVER_FLAT_CEILING = {"mixtral_8x7b": 0.10, "qwen3_235b_a22b": 1e-4}

# Shapes whose outputs exceed a flat 2e-2 against the op-by-op oracle are also compared with the
# mathematics itself: the block recomputed in float64 from the definitions (no intermediate rounding),
# with the routing and the bf16 scores taken as given.  The HIP result must be as close to that truth as
# the oracle's op-by-op result is (which rounds after every MLX op), in max-abs and in relative
# Frobenius error and in its worst element, and every element must lie within a few bf16 ulps of its row's
# scale of the truth.  Measured at 320 tokens (1.3 M elements, |truth| up to 11.3): HIP max-abs 5.6e-2,
# rel-Frobenius 4.0e-3, worst element 1.73 ulps of its row's scale; op-by-op oracle 6.9e-2, 4.8e-3, 2.19 ulps:
# the excess over a flat 2e-2 is bf16 rounding at this output scale, and the fused kernels carry less of it
# than the op-by-op sequence.
FP64_CHECKED = {"mixtral_8x7b", "qwen3_235b_a22b"}
FP64_ERR_VS_ORACLE = 1.25   # err(HIP, fp64) <= this * err(op-by-op oracle, fp64): max-abs, rel-Frobenius, worst ulps
FP64_ULPS_OF_ROW = 2.5      # |HIP - fp64| <= this many bf16 ulps of the row's largest |fp64| value


def _dequant_fp64(bank, e, bits):
    """float64 [N, K] of expert e, from the format's definition (codes low bits first, one scale and
    bias per 64 codes), on the device."""
    w = bank.weight[e].to(torch.int64) & 0xFFFFFFFF
    per = 32 // bits
    sh = torch.arange(per, device=w.device, dtype=torch.int64) * bits
    q = ((w.unsqueeze(-1) >> sh) & ((1 << bits) - 1)).reshape(w.shape[0], -1).to(torch.float64)
    sc = bank.scales[e].to(torch.float64).repeat_interleave(64, dim=1)
    bi = bank.biases[e].to(torch.float64).repeat_interleave(64, dim=1)
    return sc * q + bi


def _check_against_fp64(blk, cfg, x, dbg, pick, got_bits, oracle_bits, what):
    T, k = dbg["topk_idx"].shape
    pick_t = torch.from_numpy(pick).cuda()
    xs = x[pick_t].to(torch.float64)
    idx = dbg["topk_idx"][pick_t].to(torch.int64)
    sc = dbg["topk_w"][pick_t].to(torch.float64)
    truth = torch.zeros((len(pick), cfg.hidden), dtype=torch.float64, device="cuda")
    for e in range(cfg.n_experts):
        rows, slots = torch.nonzero(idx == e, as_tuple=True)
        if rows.numel() == 0:
            continue
        g = xs[rows] @ _dequant_fp64(blk.gate_proj, e, cfg.bits).T
        u = xs[rows] @ _dequant_fp64(blk.up_proj, e, cfg.bits).T
        h = g / (1.0 + torch.exp(-g)) * u
        y = h @ _dequant_fp64(blk.down_proj, e, cfg.bits).T
        truth.index_add_(0, rows, y * sc[rows, slots].unsqueeze(1))
    truth = truth.cpu().numpy()
    from helpers import f32_of_bits
    got = f32_of_bits(got_bits).astype(np.float64)
    orc_out = f32_of_bits(oracle_bits).astype(np.float64)
    err_got, err_orc = np.abs(got - truth), np.abs(orc_out - truth)
    fro = lambda d: float(np.linalg.norm(d) / np.linalg.norm(truth))
    row_max = np.abs(truth).max(axis=1, keepdims=True)
    ulp_row = 2.0 ** (np.floor(np.log2(np.maximum(row_max, 2.0 ** -126))) - 7)
    ulps = err_got / ulp_row
    print(f"  {what} vs float64: HIP max-abs {err_got.max():.3e} rel-Frobenius {fro(got - truth):.3e}; op-by-op oracle "
          f"max-abs {err_orc.max():.3e} rel-Frobenius {fro(orc_out - truth):.3e}; HIP worst element {ulps.max():.2f} bf16 ulps "
          f"of its row's scale (oracle {(err_orc / ulp_row).max():.2f}); max |truth| {np.abs(truth).max():.2f}", flush=True)
    assert err_got.max() <= FP64_ERR_VS_ORACLE * err_orc.max()
    assert fro(got - truth) <= FP64_ERR_VS_ORACLE * fro(orc_out - truth)
    assert ulps.max() <= FP64_ULPS_OF_ROW
    assert ulps.max() <= FP64_ERR_VS_ORACLE * (err_orc / ulp_row).max()


def _plan(cfg, T):
    """Which segments the block tiles at this batch size: (tile lists built, rows from which a segment
    is tiled): the library's own rule."""
    import mlx_rs_amd as m
    return m.capi.tile_rule(cfg.c_struct(), T)


def _pair_classes(idx, counts, offsets, inv, tiled, tmr):
    """Per pair (token-major): (expert, tile number inside the segment or -1, class name, is the
    segment's last row)."""
    T, k = idx.shape
    e = idx.reshape(-1)
    local = inv - offsets[e]
    c = counts[e]
    tile = local // 256
    full = c // 256
    r = c % 256
    rem_cls = np.where(r > 128, 0, np.where(r > 64, 1, 2))
    cls = np.where(tile < full, 3, rem_cls)  # 3 = full 256-row tile; 0/1/2 = remainder in the 256/128/64-row list
    streamed = (c < tmr) | (not tiled)
    cls = np.where(streamed, 4, cls)
    tile = np.where(streamed, -1, tile)
    return e, tile, cls, local == c - 1


CLASS_NAMES = {0: "256-row remainder tile", 1: "128-row tile", 2: "64-row tile", 3: "full 256-row tile", 4: "streamed"}


def _covering_tokens(idx, counts, offsets, inv, tiled, tmr, want):
    """Token ids, sorted: one token for every (expert, tile) and for every tiled segment's last row,
    then evenly spaced ones up to `want`."""
    T, k = idx.shape
    e, tile, cls, last = _pair_classes(idx, counts, offsets, inv, tiled, tmr)
    tok = np.repeat(np.arange(T), k)
    chosen = set()
    order = np.random.default_rng(11).permutation(T * k)
    seen = set()
    for j in order:  # first pair met of every (expert, tile)
        key = (int(e[j]), int(tile[j]))
        if key not in seen:
            seen.add(key)
            chosen.add(int(tok[j]))
    chosen.update(int(t) for t in tok[last & (cls != 4)])
    for t in np.linspace(0, T - 1, min(T, want)).astype(np.int64):
        if len(chosen) >= want:
            break
        chosen.add(int(t))
    return np.array(sorted(chosen), dtype=np.int64)


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

    # tokens against the oracle: all of them up to 512, beyond that a covering choice
    tiled, tmr = _plan(cfg, T)
    pick = np.arange(T) if T <= MIN_ORACLE_TOKENS else _covering_tokens(idx, counts, offsets, inv, tiled, tmr,
                                                                         MIN_ORACLE_TOKENS)
    S = len(pick)
    assert S >= min(T, MIN_ORACLE_TOKENS)
    e_all, tile_all, cls_all, last_all = _pair_classes(idx, counts, offsets, inv, tiled, tmr)
    sel = np.isin(np.repeat(np.arange(T), k), pick)
    assert set(np.unique(e_all)) == set(np.unique(e_all[sel])), "an expert with rows is not compared"
    assert set(zip(e_all.tolist(), tile_all.tolist())) == set(zip(e_all[sel].tolist(), tile_all[sel].tolist())), \
        "an M tile is not compared"
    assert set(np.unique(cls_all)) == set(np.unique(cls_all[sel])), "a tile class is not compared"
    assert (last_all & (cls_all != 4)).sum() == (last_all & (cls_all != 4) & sel).sum(), "a segment's last row is not compared"
    present = {CLASS_NAMES[int(c)]: int((cls_all[sel] == c).sum()) for c in np.unique(cls_all)}
    print(f"  {S} tokens vs oracle; pairs compared per class: {present}; experts with rows: {len(np.unique(e_all))}",
          flush=True)
    W = _host_weights(blk)
    xs = np.ascontiguousarray(bits_u16(x)[pick])
    ocfg = orc.make_config(cfg.hidden, E, k, cfg.intermediate, cfg.bits, cfg.group_size, cfg.score_mode)
    ref, d = orc.moe_forward(ocfg, W, xs, strict=True, n_threads=16)
    assert np.array_equal(d["topk_idx"].astype(np.int64), idx[pick]), "selection differs from the oracle"
    assert np.array_equal(d["topk_w"], bits_u16(dbg["topk_w"]).reshape(T, k)[pick]), "scores differ from the oracle"
    assert_close_bf16(bits_u16(out)[pick], ref, what=f"{name} T={T}, {S} tokens vs oracle",
                      max_over_flat=OVER_FLAT_CEILING.get(name, 0.0))
    if name in FP64_CHECKED:
        _check_against_fp64(blk, cfg, x, dbg, pick, bits_u16(out)[pick], ref, f"{name} T={T}")
