"""Writes tests/golden/moe_block_*.npz: frozen inputs and expected outputs of the MoE block
on small layers, produced by the CPU oracle (oracle/moe_oracle.c).

The reference repository holds no output vectors for this path (its tests check identities,
mlx-rs/src/ops/quantization.rs:298-423), so these files freeze the oracle's answers: the CPU
suite checks that the oracle still reproduces them, the GPU suite checks the HIP path against
them without running the oracle.  Re-run only when the oracle's definition changes:
    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
sys.path.insert(0, os.path.dirname(HERE))

CASES = {
    # name: (H, E, k, I, bits, score_mode, T, seed, zipf_s)
    "q4_renorm": (128, 4, 2, 128, 4, 0, 8, 11, None),
    "q4_plain_skewed": (256, 8, 3, 128, 4, 1, 12, 12, 1.1),
    "q8_topk_softmax": (128, 8, 2, 192, 8, 2, 10, 13, None),
}


def main():
    import oracle
    from helpers import host_layer, host_tokens
    for name, (H, E, k, I, bits, mode, T, seed, zipf) in CASES.items():
        W = host_layer(oracle, H, E, k, I, bits, seed=seed, zipf_s=zipf)
        x = host_tokens(oracle, T, H, seed=seed)
        cfg = oracle.make_config(H, E, k, I, bits, 64, mode)
        strict, d = oracle.moe_forward(cfg, W, x, strict=True, n_threads=1)
        fused, d2 = oracle.moe_forward(cfg, W, x, strict=False, n_threads=1)
        assert all(np.array_equal(d[n], d2[n]) for n in d)
        arrays = dict(config=np.array([H, E, k, I, bits, 64, mode, T], np.int32), x=x,
                      router_w=W["router_w"], out_strict=strict, out_fused=fused,
                      logits=oracle.router_logits(x, W["router_w"], W["router_bias"]), **d)
        if W["router_bias"] is not None:
            arrays["router_bias"] = W["router_bias"]
        for bank in ("gate", "up", "down"):
            for suffix, a in zip(("w", "scales", "biases"), W[bank]):
                arrays[f"{bank}_{suffix}"] = a
        path = os.path.join(HERE, f"moe_block_{name}.npz")
        np.savez_compressed(path, **arrays)
        print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
