"""Reading and writing the MoE layer of a quantized mlx-community checkpoint (safetensors).

What `mlx_lm.convert -q` writes for a sparse MoE layer, and what mlx-rs would load through
``Array::load_safetensors`` / ``ModuleParametersExt::load_safetensors``
(mlx-rs/src/ops/io.rs:50-76, module/module.rs:260-283; dtype tags U32 / BF16 from
mlx-rs/src/dtype.rs:206-256):

    <prefix>.gate.weight                                 BF16 [E, H]        the router
    <prefix>.switch_mlp.{gate,up,down}_proj.weight       U32  [E, N, K*bits/32]
    <prefix>.switch_mlp.{gate,up,down}_proj.scales       BF16 [E, N, K/group]
    <prefix>.switch_mlp.{gate,up,down}_proj.biases       BF16 [E, N, K/group]

with ``<prefix> = model.layers.<i>.mlp`` (Mixtral: ``model.layers.<i>.block_sparse_moe``).
mlx-rs's own QuantizedLinear nests the packed matrix one level deeper, under ``inner.weight``
(mlx-rs/src/nn/quantized.rs:254-279,325-327), so that spelling is accepted too.  The tensors are
used as they are stored: no repacking.
"""
import json
import os

import torch
from safetensors import safe_open
from safetensors.torch import save_file

from . import capi
from .moe import MoeConfig, QuantizedSwitchLinear, SparseMoeBlock

PROJECTIONS = ("gate_proj", "up_proj", "down_proj")


def _find_prefix(keys, layer):
    for p in (f"model.layers.{layer}.mlp", f"model.layers.{layer}.block_sparse_moe",
              f"layers.{layer}.mlp", f"layers.{layer}.block_sparse_moe"):
        if f"{p}.gate.weight" in keys:
            return p
    raise capi.MoeError(f"no MoE layer {layer} in the checkpoint (looked for model.layers.{layer}.mlp.gate.weight "
                        f"and model.layers.{layer}.block_sparse_moe.gate.weight)")


def _files(path):
    if os.path.isdir(path):
        fs = sorted(os.path.join(path, f) for f in os.listdir(path) if f.endswith(".safetensors"))
        if not fs:
            raise capi.MoeError(f"no .safetensors file in {path}")
        return fs
    return [path]


def read_moe_layer(path, layer=0, device="cpu"):
    """Returns (tensors, shapes): tensors = {"gate.weight": bf16 [E,H], "<proj>.weight": int32
    (the U32 bits), "<proj>.scales" / "<proj>.biases": bf16}, shapes = dict(hidden, n_experts,
    intermediate, bits, group_size) read off the tensor shapes."""
    index = {}
    for f in _files(path):
        with safe_open(f, "pt") as sf:
            for k in sf.keys():
                index[k] = f
    prefix = _find_prefix(index, layer)
    want = {"gate.weight": [f"{prefix}.gate.weight"]}
    for p in PROJECTIONS:
        want[f"{p}.weight"] = [f"{prefix}.switch_mlp.{p}.weight", f"{prefix}.switch_mlp.{p}.inner.weight"]
        want[f"{p}.scales"] = [f"{prefix}.switch_mlp.{p}.scales"]
        want[f"{p}.biases"] = [f"{prefix}.switch_mlp.{p}.biases"]
    out = {}
    for name, candidates in want.items():
        key = next((c for c in candidates if c in index), None)
        if key is None:
            raise capi.MoeError(f"checkpoint has no tensor {candidates[0]}")
        with safe_open(index[key], "pt") as sf:
            t = sf.get_tensor(key)
        if name.endswith(".weight") and name != "gate.weight":
            if t.dtype not in (torch.uint32, torch.int32):
                raise capi.MoeError(f"{key}: expected U32 packed codes, got {t.dtype}")
            t = t.view(torch.int32)
        elif t.dtype != torch.bfloat16:
            raise capi.MoeError(f"{key}: expected BF16, got {t.dtype} (convert the checkpoint with a bf16 dtype)")
        out[name] = t.contiguous().to(device)
    E, H = out["gate.weight"].shape
    s = out["gate_proj.scales"]
    I = s.shape[1]
    group = H // s.shape[2]
    bits = out["gate_proj.weight"].shape[2] * 32 // H
    for p, (N, K) in zip(PROJECTIONS, ((I, H), (I, H), (H, I))):
        exp_w, exp_s = (E, N, K * bits // 32), (E, N, K // group)
        if tuple(out[f"{p}.weight"].shape) != exp_w or tuple(out[f"{p}.scales"].shape) != exp_s \
                or tuple(out[f"{p}.biases"].shape) != exp_s:
            raise capi.MoeError(f"{p}: shapes {tuple(out[f'{p}.weight'].shape)}, {tuple(out[f'{p}.scales'].shape)} "
                                f"do not fit E={E} H={H} I={I} bits={bits} group={group}")
    return out, dict(hidden=H, n_experts=E, intermediate=I, bits=bits, group_size=group)


def routing_from_config(config_json):
    """top_k and score mode from a Hugging Face / mlx-lm config.json (dict or path)."""
    cfg = config_json
    if isinstance(cfg, (str, os.PathLike)):
        with open(cfg) as f:
            cfg = json.load(f)
    top_k = int(cfg.get("num_experts_per_tok", cfg.get("num_experts_per_token", 2)))
    if cfg.get("model_type", "").startswith("mixtral"):
        mode = capi.SCORE_TOPK_THEN_SOFTMAX
    elif cfg.get("norm_topk_prob", True):
        mode = capi.SCORE_SOFTMAX_THEN_TOPK_RENORM
    else:
        mode = capi.SCORE_SOFTMAX_THEN_TOPK
    return top_k, mode


def load_moe_block(path, layer=0, top_k=None, score_mode=None, device="cuda"):
    """A SparseMoeBlock over the tensors of one checkpoint layer.  top_k / score_mode come from
    the arguments or from config.json beside the weights."""
    tensors, shp = read_moe_layer(path, layer, device)
    if top_k is None or score_mode is None:
        cfg_path = os.path.join(path if os.path.isdir(path) else os.path.dirname(path), "config.json")
        if not os.path.exists(cfg_path):
            raise capi.MoeError("top_k and score_mode must be given when there is no config.json beside the weights")
        k2, m2 = routing_from_config(cfg_path)
        top_k = k2 if top_k is None else top_k
        score_mode = m2 if score_mode is None else score_mode
    cfg = MoeConfig(shp["hidden"], shp["n_experts"], top_k, shp["intermediate"], shp["bits"], shp["group_size"],
                    score_mode)
    banks = [QuantizedSwitchLinear(tensors[f"{p}.weight"], tensors[f"{p}.scales"], tensors[f"{p}.biases"])
             for p in PROJECTIONS]
    return SparseMoeBlock(cfg, tensors["gate.weight"], *banks)


def save_moe_layer(path, gate_weight, gate_proj, up_proj, down_proj, layer=0, prefix=None, nested_inner=False):
    """Writes one layer in the layout above.  Each projection is a (weight int32/uint32, scales bf16,
    biases bf16) triple or a QuantizedSwitchLinear."""
    prefix = prefix or f"model.layers.{layer}.mlp"
    out = {f"{prefix}.gate.weight": gate_weight.detach().cpu().contiguous()}
    for name, bank in zip(PROJECTIONS, (gate_proj, up_proj, down_proj)):
        w, s, b = (bank.weight, bank.scales, bank.biases) if hasattr(bank, "weight") else bank
        wkey = "inner.weight" if nested_inner else "weight"
        out[f"{prefix}.switch_mlp.{name}.{wkey}"] = w.detach().cpu().contiguous().view(torch.uint32)
        out[f"{prefix}.switch_mlp.{name}.scales"] = s.detach().cpu().contiguous()
        out[f"{prefix}.switch_mlp.{name}.biases"] = b.detach().cpu().contiguous()
    save_file(out, path)
    return sorted(out)
