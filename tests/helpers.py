"""Shared helpers of the parity tests: tensors <-> raw-bit numpy arrays, error metrics,
and a CPU-side builder of synthetic quantized layers that uses the oracle's quantizer."""
import numpy as np
import torch

# The one tolerance rule of every float comparison in these tests.
#
# Stated for the path: bf16 outputs within max-abs 2e-2 and relative Frobenius error 1e-2 of the
# reference.  The absolute figure is a figure at unit output scale: bf16 keeps 8 significant bits, so
# from |value| = 4 on a single ulp (2^-5 = 3.1e-2) is already more than 2e-2 and no bf16 result could
# meet a flat bar.  An output element is a sum of products whose rounding errors follow the size of
# the terms, not of the sum (an output of 0.1 in a row whose values reach 8 carries the rounding of
# terms of that size), so the scale is the row's, not the element's.  The rule, row by row:
#     |got - ref| <= 2e-2 * max(1, max |ref| over the row)
# and always, over the whole array, relative Frobenius error <= 1e-2.  Rows that stay within [-1, 1]
# are held to the flat bar.  For scale: 2e-2 * 2^k is 2.56 bf16 ulps of values in [2^k, 2^(k+1));
# the oracle's own two rounding modes (one bf16 rounding where the library has one / one after every
# MLX op) lie up to 2 such ulps apart on the same inputs.
# assert_close_bf16 prints the unscaled max-abs error and the number of elements beyond the flat bar
# on every call, so the flat figure is always on record.
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
    """(unscaled max-abs error, relative Frobenius error) of two arrays of bf16 bits."""
    a, b = f32_of_bits(got_bits).astype(np.float64), f32_of_bits(ref_bits).astype(np.float64)
    max_abs = float(np.abs(a - b).max()) if a.size else 0.0
    rel = float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30)) if a.size else 0.0
    return max_abs, rel


def row_tolerance(ref):
    """The absolute tolerance of every element of `ref` (float array, rows along the last axis)."""
    ref = np.asarray(ref, dtype=np.float64)
    if ref.ndim == 0:
        return MAX_ABS_TOL * max(1.0, abs(float(ref)))
    row_max = np.abs(ref).max(axis=-1, keepdims=True) if ref.shape[-1] else np.zeros(ref.shape[:-1] + (1,))
    return np.broadcast_to(MAX_ABS_TOL * np.maximum(1.0, row_max), ref.shape)


def assert_close_bf16(got_bits, ref_bits, what="", rel_fro=REL_FRO_TOL, quiet=False, max_over_flat=None):
    """The tolerance rule above.  Returns (unscaled max-abs, rel-Frobenius) and prints them together
    with the worst error in units of its row's tolerance.  max_over_flat (optional): the largest share
    of the elements that may lie beyond the flat 2e-2 (0.0: none; they can only sit in rows whose
    reference reaches beyond 1, where the row-scaled allowance applies)."""
    a, b = f32_of_bits(got_bits).astype(np.float64), f32_of_bits(ref_bits).astype(np.float64)
    assert a.shape == b.shape, f"{what}: shapes {a.shape} vs {b.shape}"
    m, r = errors(got_bits, ref_bits)
    if a.size == 0:
        return m, r
    assert np.isfinite(a).all() and np.isfinite(b).all(), f"{what}: non-finite values"
    tol = row_tolerance(b)
    ratio = np.abs(a - b) / tol
    worst = int(np.argmax(ratio))
    over_flat = int((np.abs(a - b) > MAX_ABS_TOL).sum())
    if not quiet:
        print(f"  {what}: max-abs {m:.3e} unscaled ({over_flat} of {a.size} elements beyond the flat {MAX_ABS_TOL}; "
              f"max |ref| {np.abs(b).max():.2f}); worst element at {ratio.flat[worst]:.2f} of its row's tolerance "
              f"{tol.flat[worst]:.3e}; rel-Frobenius {r:.3e}", flush=True)
    if max_over_flat is not None:
        assert over_flat <= max_over_flat * a.size, (
            f"{what}: {over_flat} of {a.size} elements beyond the flat {MAX_ABS_TOL} (ceiling {max_over_flat:.3f} of them)")
    assert ratio.flat[worst] <= 1.0 and r <= rel_fro, (
        f"{what}: element {worst}: got {a.flat[worst]!r}, reference {b.flat[worst]!r}, error "
        f"{abs(a.flat[worst] - b.flat[worst]):.3e} > tolerance {tol.flat[worst]:.3e} of its row; "
        f"unscaled max-abs {m:.3e}; rel-Frobenius {r:.3e} (tol {rel_fro})")
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
