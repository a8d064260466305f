"""Shared helpers of the parity tests: tensors <-> raw-bit numpy arrays, error metrics,
and a CPU-side builder of synthetic quantized layers that uses the oracle's quantizer."""
import numpy as np
import torch

# tolerances stated by the task for float outputs in bf16
MAX_ABS_TOL = 2e-2
REL_FRO_TOL = 1e-2


def bits_u16(t):
    """bf16 torch tensor (any device) -> numpy uint16 of the raw bits."""
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def bits_u32(t):
    return t.detach().cpu().contiguous().numpy().view(np.uint32)


def bf16_tensor(bits, device="cpu"):
    """numpy uint16 raw bits -> bf16 torch tensor."""
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).view(torch.bfloat16).to(device)


def i32_tensor(u32, device="cpu"):
    return torch.from_numpy(np.ascontiguousarray(u32).view(np.int32)).to(device)


def f32_of_bits(bits):
    return (bits.astype(np.uint32) << 16).view(np.float32)


def errors(got_bits, ref_bits):
    a, b = f32_of_bits(got_bits).astype(np.float64), f32_of_bits(ref_bits).astype(np.float64)
    max_abs = float(np.abs(a - b).max()) if a.size else 0.0
    rel = float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30)) if a.size else 0.0
    return max_abs, rel


def assert_close_bf16(got_bits, ref_bits, max_abs=MAX_ABS_TOL, rel_fro=REL_FRO_TOL, what=""):
    m, r = errors(got_bits, ref_bits)
    assert m <= max_abs and r <= rel_fro, f"{what}: max-abs {m:.3e} (tol {max_abs}), rel-Frobenius {r:.3e} (tol {rel_fro})"
    return m, r


def host_layer(orc, H, E, k, I, bits=4, seed=0, std=0.02, zipf_s=None):
    """Synthetic layer on the host, quantised by the oracle: dict usable by oracle.moe_forward."""
    rng = np.random.default_rng(seed)

    def bank(N, K):
        w = rng.normal(0.0, std, (E * N, K)).astype(np.float32)
        q, s, b = orc.quantize(w, bits, 64)
        return q.reshape(E, N, -1), s.reshape(E, N, -1), b.reshape(E, N, -1)

    W = dict(router_w=orc.f32_to_bf16(rng.normal(0.0, std, (E, H)).astype(np.float32)),
             router_bias=None, gate=bank(I, H), up=bank(I, H), down=bank(H, I))
    if zipf_s is not None:
        rank = rng.permutation(E).astype(np.float32) + 1.0
        W["router_bias"] = (-zipf_s * np.log(rank)).astype(np.float32)
    return W


def host_tokens(orc, T, H, seed=0):
    rng = np.random.default_rng(seed + 1000)
    return orc.f32_to_bf16(rng.normal(0.0, 1.0, (T, H)).astype(np.float32))


def device_block(mod, cfg, W, device="cuda"):
    """Upload a host layer (host_layer) and wrap it in the product's SparseMoeBlock."""
    def bank(t):
        return mod.QuantizedSwitchLinear(i32_tensor(t[0], device), bf16_tensor(t[1], device), bf16_tensor(t[2], device))
    bias = None if W.get("router_bias") is None else torch.from_numpy(W["router_bias"]).to(device)
    return mod.SparseMoeBlock(cfg, bf16_tensor(W["router_w"], device), bank(W["gate"]), bank(W["up"]),
                              bank(W["down"]), router_bias=bias)
