"""GPU parity of the whole block (mi_moe_forward through the C ABI) against the oracle."""
import numpy as np
import pytest
import torch

from helpers import (assert_close_bf16, bits_u16, bits_u32, bf16_tensor, device_block, errors, f32_of_bits,
                     host_layer, host_tokens, i32_tensor)

pytestmark = pytest.mark.gpu


def _run_case(orc, H, E, k, I, bits, T, score_mode, seed=0, zipf_s=None, threads=16, std=0.02):
    import mlx_rs_amd as m
    print(f"case H={H} E={E} k={k} I={I} bits={bits} T={T} mode={score_mode} seed={seed}", flush=True)
    W = host_layer(orc, H, E, k, I, bits, seed, std=std, zipf_s=zipf_s)
    x = host_tokens(orc, T, H, seed)
    cfg = m.MoeConfig(H, E, k, I, bits, 64, score_mode)
    blk = device_block(m, cfg, W)
    out, dbg = blk.forward(bf16_tensor(x, "cuda"), debug=True)
    torch.cuda.synchronize()
    ocfg = orc.make_config(H, E, k, I, bits, 64, score_mode)
    ref_f, d = orc.moe_forward(ocfg, W, x, strict=False, n_threads=threads)
    ref_s, _ = orc.moe_forward(ocfg, W, x, strict=True, n_threads=threads)
    # integer results: bit-exact
    for name in ("topk_idx", "counts", "offsets", "perm", "inv_perm"):
        got = bits_u32(dbg[name]).reshape(d[name].shape)
        assert np.array_equal(got, d[name]), f"{name} differs from the oracle"
    assert np.array_equal(bits_u16(dbg["topk_w"]), d["topk_w"]), "scores differ from the oracle"
    got = bits_u16(out)
    mf, rf = assert_close_bf16(got, ref_f, what="vs oracle (fused rounding points)")
    ms, rs = assert_close_bf16(got, ref_s, what="vs oracle (op-by-op rounding)")
    return got


def test_tiny_config(orc):
    # H256 E8 k2 I512 4-bit T32, renormalised top-2
    _run_case(orc, 256, 8, 2, 512, 4, 32, 0)


@pytest.mark.parametrize("T", [1, 8, 32])
def test_qwen3_30b_decode(orc, T):
    _run_case(orc, 2048, 128, 8, 768, 4, T, 0)


def test_score_modes(orc):
    _run_case(orc, 256, 8, 2, 512, 4, 17, 1, seed=3)
    _run_case(orc, 256, 8, 2, 512, 4, 17, 2, seed=4)


def test_eight_bit(orc):
    _run_case(orc, 512, 8, 2, 1024, 8, 40, 2, seed=5)


@pytest.mark.parametrize("T,I,bits", [(1, 6144, 4), (20, 6144, 4), (20, 6144, 8), (5, 4608, 8), (70, 8192, 4)])
def test_long_rows_are_staged_in_slabs(orc, T, I, bits):
    # the down product's rows are I long: beyond 4096 values the streaming kernel stages them a
    # slab at a time (whole and partial last slabs, K split over the waves at T = 1, several
    # passes over a segment at T = 70)
    _run_case(orc, 256, 8, 2, I, bits, T, 0, seed=60 + T)


def test_long_segments_and_imbalance(orc):
    # segments longer than one token tile, strongly skewed routing
    _run_case(orc, 256, 16, 4, 256, 4, 300, 0, seed=6, zipf_s=1.3)


def test_prefill_sized_dispatch(orc):
    # P = 6000 pairs > 4096: the multi-block dispatch path
    _run_case(orc, 128, 64, 6, 128, 4, 1000, 0, seed=7, zipf_s=1.1)


def test_run_to_run_identical(orc):
    import mlx_rs_amd as m
    W = host_layer(orc, 256, 8, 2, 512, 4, 11)
    x = bf16_tensor(host_tokens(orc, 64, 256, 11), "cuda")
    blk = device_block(m, m.MoeConfig(256, 8, 2, 512), W)
    outs = [bits_u16(blk.forward(x)) for _ in range(3)]
    assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[0], outs[2])


def test_fused_router_equals_the_separate_kernels(orc):
    """Up to 64 tokens the block runs logits + selection + dispatch as one launch; the stage-level
    entry points run them as separate kernels.  Same integers and scores, call after call (the
    launch leaves its arrival counters at zero), across batch sizes on both sides of the switch, and
    on both sides of the switch between the one-exchange kernel (up to 8 tokens) and the two-exchange
    kernel, which share a counter."""
    import mlx_rs_amd as m
    _fused_vs_separate(orc, m, 256, 128, 8, 128, [1, 64, 3, 64, 17, 65, 2, 40, 1, 8, 9, 8])
    # more pairs than the dispatching workgroup has threads (60 x 20 = 1200), few experts
    _fused_vs_separate(orc, m, 128, 32, 20, 128, [60, 33, 64, 5, 60, 8])


def _fused_vs_separate(orc, m, H, E, k, I, batches):
    W = host_layer(orc, H, E, k, I, 4, 21, zipf_s=0.7)
    blk = device_block(m, m.MoeConfig(H, E, k, I), W)
    rw = bf16_tensor(W["router_w"], "cuda")
    rb = torch.from_numpy(W["router_bias"]).cuda()
    for rep, T in enumerate(batches):
        print(f"fused router H={H} E={E} k={k} T={T}", flush=True)
        x = bf16_tensor(host_tokens(orc, T, H, 100 + rep), "cuda")
        _, dbg = blk.forward(x, debug=True)
        inds, sc = m.ops.route(x, rw, k, 0, router_bias=rb)
        counts, offsets, perm, inv = m.ops.dispatch(inds, E)
        torch.cuda.synchronize()
        for got, want, name in ((dbg["topk_idx"], inds, "topk_idx"), (dbg["counts"], counts, "counts"),
                                (dbg["offsets"], offsets, "offsets"), (dbg["perm"], perm, "perm"),
                                (dbg["inv_perm"], inv, "inv_perm")):
            assert torch.equal(got.reshape(want.shape), want), f"{name} at T={T}"
        assert torch.equal(dbg["topk_w"].view(torch.int16), sc.view(torch.int16)), f"scores at T={T}"


@pytest.mark.parametrize("T,E,k,bits,zipf", [(192, 8, 2, 4, None), (200, 8, 2, 4, 0.8), (700, 8, 2, 8, None),
                                             (333, 16, 4, 4, 1.2), (1100, 4, 1, 4, None)])
def test_tile_classes(orc, T, E, k, bits, zipf):
    # segments of 9 rows and more are cut into 256-, 128- and 64-row tiles, shorter ones stream:
    # these shapes put segments into every class, with remainders on both sides of each boundary
    _run_case(orc, 256, E, k, 384, bits, T, 0, seed=31 + T, zipf_s=zipf)


@pytest.mark.parametrize("bits,zipf", [(4, None), (8, 0.7)])
def test_tile_classes_with_the_chip_full(orc, bits, zipf):
    # narrow layers leave the chip blocks to spare and run their 256- and 128-row tiles with the
    # 64-row kernel (the shapes of test_tile_classes); here both products have more than 256 blocks
    # even with 128-row tiles, so each list is run by the kernel of its own size
    _run_case(orc, 3072, 8, 2, 1536, bits, 1100, 0, seed=17 + bits, zipf_s=zipf)


@pytest.mark.parametrize("T,H,I", [(40, 2048, 768), (44, 1024, 2048), (13, 256, 384), (16, 2048, 256)])
def test_two_token_groups_per_pass(orc, T, H, I):
    # 4-bit segments of 9 to 16 rows take one pass of the streaming kernel (two MFMA tiles of 8
    # tokens against each chunk of weights); rows of 2048 values are staged in slabs of 1024
    _run_case(orc, H, 8, 2, I, 4, T, 0, seed=91 + T)


@pytest.mark.parametrize("T,H,E,k,I", [(64, 512, 64, 8, 1536), (100, 512, 64, 8, 2048), (65, 2048, 33, 6, 1536),
                                       (160, 1024, 128, 8, 1536)])
def test_two_token_groups_with_rows_in_slabs(orc, T, H, E, k, I):
    # the down product of a layer with many experts (more blocks than CUs) and rows of 1536 or 2048 values at 8
    # to 16 rows per expert: two token groups per pass, rows staged in slabs of 1024 (the last one of 512 values
    # for 1536), one row tile per wave
    _run_case(orc, H, E, k, I, 4, T, 0, seed=300 + T)


@pytest.mark.parametrize("T,E,k,zipf", [(100, 16, 2, 1.5), (40, 16, 4, 1.2), (150, 32, 4, 1.0), (150, 32, 4, None)])
def test_light_batches_tile_only_long_segments(orc, T, E, k, zipf):
    # 6 to 20 rows per expert on average (4-bit): the streamed segments lead on the caller's stream,
    # segments of 17 rows and more (uneven routing) are tiled on the side streams; 40 tokens: the
    # one-launch router builds the tile lists
    _run_case(orc, 256, E, k, 384, 4, T, 0, seed=57 + T, zipf_s=zipf)


@pytest.mark.parametrize("T,H,E,k,I,bits,mode,zipf", [(1, 256, 8, 2, 512, 4, 0, None), (32, 2048, 128, 8, 768, 4, 0, None),
                                                      (300, 256, 16, 4, 256, 8, 2, 1.0)])
def test_norm_and_residual_around_the_block(orc, T, H, E, k, I, bits, mode, zipf):
    """mi_moe_forward_residual: x + moe(rms_norm(x)).  The normalised rows carry the selection, so
    routing must still match the oracle bit for bit; rms_norm on its own is bit-exact too."""
    import mlx_rs_amd as m
    print(f"residual case T={T} H={H} E={E} k={k} I={I} bits={bits} mode={mode}", flush=True)
    W = host_layer(orc, H, E, k, I, bits, seed=40 + T, zipf_s=zipf)
    x = host_tokens(orc, T, H, seed=40 + T)
    nw = orc.f32_to_bf16(np.random.default_rng(T).normal(1.0, 0.2, H).astype(np.float32))
    blk = device_block(m, m.MoeConfig(H, E, k, I, bits, 64, mode), W)
    xd, nwd = bf16_tensor(x, "cuda"), bf16_tensor(nw, "cuda")
    out, dbg = blk.forward_residual(xd, nwd, 1e-6, debug=True)
    xn = m.ops.rms_norm(xd, nwd, 1e-6)
    torch.cuda.synchronize()
    assert np.array_equal(bits_u16(xn), orc.rms_norm(x, nw, 1e-6)), "rms_norm differs from the oracle"
    ocfg = orc.make_config(H, E, k, I, bits, 64, mode)
    ref_s, d = orc.moe_forward(ocfg, W, x, strict=True, n_threads=16, norm_weight=nw, eps=1e-6)
    ref_f, _ = orc.moe_forward(ocfg, W, x, strict=False, n_threads=16, norm_weight=nw, eps=1e-6)
    for name in ("topk_idx", "counts", "perm"):
        assert np.array_equal(bits_u32(dbg[name]).reshape(d[name].shape), d[name]), name
    assert np.array_equal(bits_u16(dbg["topk_w"]), d["topk_w"])
    assert_close_bf16(bits_u16(out), ref_f, what="vs oracle (fused rounding points)")
    assert_close_bf16(bits_u16(out), ref_s, what="vs oracle (op-by-op rounding)")
    # and it is the plain forward on rms_norm(x) plus x, up to the one rounding that is saved
    y = blk.forward(xn)
    torch.cuda.synchronize()
    want = (xd.float() + y.float()).bfloat16()
    assert_close_bf16(bits_u16(out), bits_u16(want), what="vs x + forward(rms_norm(x)) in two roundings")
    with pytest.raises(m.MoeError, match="alias"):
        blk.forward_residual(xd, nwd, 1e-6, out=xd)


@pytest.mark.parametrize("T", [4, 70, 300])
def test_graph_replays_equal_eager(orc, T):
    """A forward captured into a HIP graph (decode: the one-launch router with its self-resetting
    arrival counters; 70 tokens: streamed segments first, tiles beside them; prefill: the tiled
    kernels) gives the eager result on every replay, with eager forwards of other sizes and
    synchronisations in between."""
    import mlx_rs_amd as m
    H, E, k, I = 256, 16, 4, 256
    W = host_layer(orc, H, E, k, I, 4, seed=77)
    blk = device_block(m, m.MoeConfig(H, E, k, I), W)
    x = bf16_tensor(host_tokens(orc, T, H, seed=77), "cuda")
    other = bf16_tensor(host_tokens(orc, 7, H, seed=78), "cuda")
    blk.reserve(max(T, 7))
    eager = blk.forward(x).clone()
    out = torch.empty_like(x)
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        blk.forward(x, out=out)
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        blk.forward(x, out=out)
    for rep in range(4):
        out.zero_()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int16), eager.view(torch.int16)), f"replay {rep} differs from the eager result"
        blk.forward(other)  # eager work through the same handle and workspace between the replays
        torch.cuda.synchronize()


@pytest.mark.parametrize("T", [16, 40, 70, 400])
def test_two_handles_on_two_streams(orc, T):
    """Handles are independent: two layers running concurrently on two streams (each with its own
    workspace) give what they give one after the other.  From 40 tokens on each forward also forks
    its kernel chains onto the handle's own streams and joins them back (40 and 70: streamed
    segments first, with the one-launch router and the separate kernels; 400: tiles first)."""
    import mlx_rs_amd as m
    H, E, k, I = 256, 16, 4, 256
    print(f"two handles T={T}", flush=True)
    blks, xs, refs = [], [], []
    for i in range(2):
        W = host_layer(orc, H, E, k, I, 4, seed=90 + i)
        blks.append(device_block(m, m.MoeConfig(H, E, k, I), W))
        xs.append(bf16_tensor(host_tokens(orc, T, H, seed=90 + i), "cuda"))
        refs.append(blks[i].forward(xs[i]).clone())
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    outs = [torch.empty_like(xs[0]), torch.empty_like(xs[1])]
    for rep in range(20):
        for i in range(2):
            with torch.cuda.stream(streams[i]):
                blks[i].forward(xs[i], out=outs[i])
    torch.cuda.synchronize()
    for i in range(2):
        assert torch.equal(outs[i].view(torch.int16), refs[i].view(torch.int16)), f"handle {i}"


def test_empty_batch_and_leading_axes(orc):
    """[B, L, H] goes through as B*L rows (the Module contract, mlx-rs/src/module/module.rs:28-50,
    as the dense Mlp is called with [B, L, H], mlx-lm/src/models/qwen3.rs:321-324); an empty batch
    succeeds and touches nothing."""
    import mlx_rs_amd as m
    H, E, k, I = 256, 8, 2, 512
    W = host_layer(orc, H, E, k, I, 4, seed=5)
    blk = device_block(m, m.MoeConfig(H, E, k, I), W)
    x = bf16_tensor(host_tokens(orc, 6, H, seed=6), "cuda")
    flat = blk.forward(x).clone()
    cube = blk.forward(x.reshape(2, 3, H))
    torch.cuda.synchronize()
    assert cube.shape == (2, 3, H)
    assert torch.equal(cube.reshape(6, H).view(torch.int16), flat.view(torch.int16))
    empty = blk.forward(x[:0])
    torch.cuda.synchronize()
    assert empty.shape == (0, H)
    out, dbg = blk.forward(x[:0].reshape(0, 1, H), debug=True)
    assert out.shape == (0, 1, H) and dbg["perm"].numel() == 0


@pytest.mark.parametrize("T,zipf", [(16, None), (60, 1.3), (200, 1.3)])
def test_widest_outputs_of_the_shape_sweep(orc, T, zipf):
    # the shape whose outputs are the largest of those swept (rows of 4096 values, two experts per
    # token: |out| reaches 2.7, where a bf16 ulp is 1.6e-2), under the one tolerance rule
    _run_case(orc, 4096, 8, 2, 1024, 4, T, 0, seed=200 + T, zipf_s=zipf)


@pytest.mark.parametrize("bits,T", [(4, 1), (4, 7), (4, 40), (4, 300), (8, 1), (8, 40), (8, 300)])
def test_one_expert_is_the_dense_quantized_mlp(orc, bits, T):
    """n_experts = 1, top_k = 1: the router can only pick the one expert with score 1, and the block is
    the dense quantized MLP down(silu(gate(x)) * up(x)) of mlx-lm/src/models/qwen3.rs:204-255 with
    QuantizedLinear layers (mlx-rs/src/nn/quantized.rs:363-386).  Checked against the oracle like any
    block, and against the chain of the op-level entry points (three quantized_matmul and a swiglu)."""
    import mlx_rs_amd as m
    H, I = 1024, 3072
    got = _run_case(orc, H, 1, 1, I, bits, T, 0, seed=90 + T)
    W = host_layer(orc, H, 1, 1, I, bits, 90 + T)
    x = bf16_tensor(host_tokens(orc, T, H, 90 + T), "cuda")
    mats = {n: (i32_tensor(W[n][0][0], "cuda"), bf16_tensor(W[n][1][0], "cuda"), bf16_tensor(W[n][2][0], "cuda"))
            for n in ("gate", "up", "down")}
    g = m.ops.quantized_matmul(x, *mats["gate"], True, 64, bits)
    u = m.ops.quantized_matmul(x, *mats["up"], True, 64, bits)
    h = m.ops.swiglu(g, u)
    y = m.ops.quantized_matmul(h, *mats["down"], True, 64, bits)
    assert_close_bf16(got, bits_u16(y), what="block vs the chain of quantized_matmul and swiglu")


def test_side_streams_belong_to_the_gpu_not_to_a_handle():
    """A hundred handles on one GPU: no stream is created after the first handle's three, and a
    prefill-sized forward through the last handle gives the first one's result."""
    import mlx_rs_amd as m
    from mlx_rs_amd import synth
    lib = m.load_library()
    cfg = m.MoeConfig(256, 8, 2, 512)
    first = synth.make_block(cfg, seed=2, device="cuda", gen_device="cuda")
    created = lib.mi_moe_debug_side_streams_created()
    assert created >= 3 and created % 3 == 0
    blocks = [m.SparseMoeBlock(cfg, first.gate_weight, first.gate_proj, first.up_proj, first.down_proj) for _ in range(100)]
    assert lib.mi_moe_debug_side_streams_created() == created
    x = synth.make_tokens(cfg, 512, seed=2, device="cuda")   # 128 rows per expert: tile classes on the side streams
    a, b = first.forward(x), blocks[-1].forward(x)
    torch.cuda.synchronize()
    assert torch.equal(a, b)
    assert lib.mi_moe_debug_side_streams_created() == created
