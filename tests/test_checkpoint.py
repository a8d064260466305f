"""safetensors ingestion of a quantized MoE layer in the mlx-community layout
(mlx-rs_amd/checkpoint.py).  No real checkpoint can be fetched here, so the files are written by
the test in that layout: dtype tags U32 / BF16 (mlx-rs/src/dtype.rs:206-256), key names of
mlx-lm's switch layers, and the `inner.weight` spelling of mlx-rs's QuantizedLinear
(mlx-rs/src/nn/quantized.rs:325-327)."""
import json
import struct

import numpy as np
import pytest
import torch

from helpers import assert_close_bf16, bf16_tensor, bits_u16, bits_u32, host_layer, host_tokens, i32_tensor


def _write(tmp_path, W, nested=False, prefix=None, layer=3):
    from mlx_rs_amd import checkpoint
    bank = lambda t: (i32_tensor(t[0]), bf16_tensor(t[1]), bf16_tensor(t[2]))
    path = str(tmp_path / "model.safetensors")
    keys = checkpoint.save_moe_layer(path, bf16_tensor(W["router_w"]), bank(W["gate"]), bank(W["up"]),
                                     bank(W["down"]), layer=layer, prefix=prefix, nested_inner=nested)
    return path, keys


@pytest.mark.parametrize("nested,prefix", [(False, None), (True, None), (False, "model.layers.3.block_sparse_moe")])
def test_layout_and_round_trip_on_the_host(orc, tmp_path, nested, prefix):
    from mlx_rs_amd import checkpoint
    H, E, k, I = 128, 4, 2, 256
    W = host_layer(orc, H, E, k, I, 4, seed=3)
    path, keys = _write(tmp_path, W, nested, prefix)
    with open(path, "rb") as f:  # the container format itself: 8-byte length + JSON header
        n = struct.unpack("<Q", f.read(8))[0]
        header = json.loads(f.read(n))
    p = prefix or "model.layers.3.mlp"
    wkey = f"{p}.switch_mlp.gate_proj." + ("inner.weight" if nested else "weight")
    assert header[wkey]["dtype"] == "U32" and header[wkey]["shape"] == [E, I, H * 4 // 32]
    assert header[f"{p}.switch_mlp.down_proj.scales"]["dtype"] == "BF16"
    assert header[f"{p}.switch_mlp.down_proj.scales"]["shape"] == [E, H, I // 64]
    assert header[f"{p}.gate.weight"] == {"dtype": "BF16", "shape": [E, H], "data_offsets": header[f"{p}.gate.weight"]["data_offsets"]}
    tensors, shp = checkpoint.read_moe_layer(path, layer=3)
    assert shp == dict(hidden=H, n_experts=E, intermediate=I, bits=4, group_size=64)
    assert np.array_equal(bits_u16(tensors["gate.weight"]), W["router_w"])
    for name, bank in (("gate_proj", "gate"), ("up_proj", "up"), ("down_proj", "down")):
        assert np.array_equal(bits_u32(tensors[f"{name}.weight"]), W[bank][0])
        assert np.array_equal(bits_u16(tensors[f"{name}.scales"]), W[bank][1])
        assert np.array_equal(bits_u16(tensors[f"{name}.biases"]), W[bank][2])


def test_errors_and_config(orc, tmp_path):
    import mlx_rs_amd as m
    from mlx_rs_amd import checkpoint
    W = host_layer(orc, 128, 4, 2, 128, 8, seed=4)
    path, _ = _write(tmp_path, W)
    with pytest.raises(m.MoeError, match="no MoE layer 0"):
        checkpoint.read_moe_layer(path, layer=0)
    _, shp = checkpoint.read_moe_layer(str(tmp_path), layer=3)  # a directory of shards works too
    assert shp["bits"] == 8
    assert checkpoint.routing_from_config({"model_type": "mixtral", "num_experts_per_tok": 2}) == (2, m.capi.SCORE_TOPK_THEN_SOFTMAX)
    assert checkpoint.routing_from_config({"model_type": "qwen3_moe", "num_experts_per_tok": 8, "norm_topk_prob": True}) == (8, 0)
    assert checkpoint.routing_from_config({"model_type": "qwen3_moe", "num_experts_per_tok": 8, "norm_topk_prob": False}) == (8, 1)
    with pytest.raises(m.MoeError, match="top_k"):
        checkpoint.load_moe_block(path, layer=3, device="cpu")


@pytest.mark.gpu
def test_block_from_a_checkpoint_matches_the_oracle(orc, tmp_path):
    import mlx_rs_amd as m
    from mlx_rs_amd import checkpoint
    H, E, k, I, T = 256, 8, 2, 512, 20
    W = host_layer(orc, H, E, k, I, 4, seed=6)
    path, _ = _write(tmp_path, W, nested=True)
    (tmp_path / "config.json").write_text(json.dumps({"model_type": "qwen3_moe", "num_experts_per_tok": k,
                                                      "norm_topk_prob": True}))
    blk = checkpoint.load_moe_block(path, layer=3, device="cuda")
    assert (blk.config.hidden, blk.config.n_experts, blk.config.top_k, blk.config.intermediate) == (H, E, k, I)
    x = host_tokens(orc, T, H, seed=6)
    out, dbg = blk.forward(bf16_tensor(x, "cuda"), debug=True)
    torch.cuda.synchronize()
    ref, d = orc.moe_forward(orc.make_config(H, E, k, I), W, x, strict=True, n_threads=4)
    assert np.array_equal(bits_u32(dbg["topk_idx"]).reshape(d["topk_idx"].shape), d["topk_idx"])
    assert_close_bf16(bits_u16(out), ref, what="block loaded from safetensors")
