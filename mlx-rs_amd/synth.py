"""Synthetic, seeded MoE layers of the shapes the benchmark and the parity tests use.

Dense fp32 weights ~N(0, 0.02) are drawn with a CPU torch.Generator (so the bytes do not
depend on the GPU), moved to the device and quantised there with ``ops.quantize``
(MLX-affine, group 64, bf16 scales/biases).  The router is bf16 ~N(0, 0.02), unquantised.
A Zipf router bias ``-s * ln(rank_e)`` (rank = seeded permutation of 1..E) gives the load
imbalance of the prefill configurations.
"""
import math

import torch

from . import capi, ops
from .moe import MoeConfig, QuantizedSwitchLinear, SparseMoeBlock

CONFIGS = {
    # hidden, experts, top_k, intermediate, bits
    "tiny": MoeConfig(256, 8, 2, 512, 4, 64, capi.SCORE_SOFTMAX_THEN_TOPK_RENORM),
    "qwen3_30b_a3b": MoeConfig(2048, 128, 8, 768, 4, 64, capi.SCORE_SOFTMAX_THEN_TOPK_RENORM),
    "mixtral_8x7b": MoeConfig(4096, 8, 2, 14336, 8, 64, capi.SCORE_TOPK_THEN_SOFTMAX),
    "qwen3_235b_a22b": MoeConfig(4096, 128, 8, 1536, 4, 64, capi.SCORE_SOFTMAX_THEN_TOPK_RENORM),
}


def _randn(shape, gen, device):
    """Standard normal fp32 on `device`; drawn where the generator lives (CPU by default)."""
    return torch.randn(shape, generator=gen, dtype=torch.float32, device=gen.device).to(device)


def _bank(cfg, n_out, n_in, gen, device, std=0.02):
    E = cfg.n_experts
    w = torch.empty((E, n_out, n_in * cfg.bits // 32), dtype=torch.int32, device=device)
    s = torch.empty((E, n_out, n_in // cfg.group_size), dtype=torch.bfloat16, device=device)
    b = torch.empty_like(s)
    for e in range(E):
        dense = _randn((n_out, n_in), gen, device) * std
        q, sc, bi = ops.quantize(dense, cfg.group_size, cfg.bits)
        w[e], s[e], b[e] = q, sc, bi
    return QuantizedSwitchLinear(w, s, b)


def zipf_bias(n_experts, s, seed):
    gen = torch.Generator().manual_seed(seed + 7919)
    rank = torch.randperm(n_experts, generator=gen).to(torch.float32) + 1.0
    return (-s * torch.log(rank)).to(torch.float32)


def make_block(cfg, seed=0, device="cuda", zipf_s=None, gen_device="cpu"):
    """A SparseMoeBlock with seeded synthetic weights on ``device``.  gen_device="cuda" draws
    the dense weights on the GPU (fast; the bytes then depend on the GPU's generator)."""
    gen = torch.Generator(device=gen_device).manual_seed(seed)
    router = (_randn((cfg.n_experts, cfg.hidden), gen, device) * 0.02).to(torch.bfloat16)
    gate = _bank(cfg, cfg.intermediate, cfg.hidden, gen, device)
    up = _bank(cfg, cfg.intermediate, cfg.hidden, gen, device)
    down = _bank(cfg, cfg.hidden, cfg.intermediate, gen, device)
    bias = None if zipf_s is None else zipf_bias(cfg.n_experts, zipf_s, seed).to(device)
    return SparseMoeBlock(cfg, router, gate, up, down, router_bias=bias)


def make_tokens(cfg, tokens, seed=0, device="cuda"):
    gen = torch.Generator().manual_seed(seed + 104729)
    x = torch.randn((tokens, cfg.hidden), generator=gen, dtype=torch.float32)
    return x.to(torch.bfloat16).to(device)


def layer_bytes_per_expert(cfg):
    """codes + bf16 scales + bf16 biases of the gate, up and down matrices of one expert."""
    n_k = cfg.intermediate * cfg.hidden
    return 3 * (n_k * cfg.bits // 8) + 3 * (n_k // cfg.group_size) * 4


def decode_algorithmic_bytes(cfg, tokens, n_active):
    """HBM bytes one forward has to move: the active experts' weights, the router matrix,
    x in and out.  Indices, scores and workspace traffic are not counted."""
    return (n_active * layer_bytes_per_expert(cfg) + cfg.n_experts * cfg.hidden * 2
            + 2 * tokens * cfg.hidden * 2)


def prefill_flops(cfg, tokens):
    return tokens * cfg.top_k * 2 * 3 * cfg.hidden * cfg.intermediate + tokens * 2 * cfg.hidden * cfg.n_experts


def expected_active(cfg, tokens):
    e, p = cfg.n_experts, tokens * cfg.top_k
    return e * (1.0 - math.pow(1.0 - 1.0 / e, p))
