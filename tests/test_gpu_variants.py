"""Every compiled variant of the two grouped-product kernels is launched at least once on rows whose
results are compared with the oracle.

The cases come from tests/variant_cases.py (one block shape per variant, found with the launch planner).
Each case: the planner says which variants the forward launches; the realised routing (rows per expert,
from the forward's own debug outputs) says which of them find rows; the forward is compared with the
oracle under the tolerance rule of helpers.py, routing bit for bit.  The last test of the file asserts
that the variants so checked are all the variants the library holds, and that the library's own launch
counters agree."""
import numpy as np
import pytest
import torch

from helpers import assert_close_bf16, bits_u16, bits_u32, f32_of_bits
from variant_cases import BLOCK_CASES, OP_CASE, kernels_with_rows, rules

pytestmark = pytest.mark.gpu

CHECKED = set()      # variants that ran on oracle-compared rows
LAUNCHES_BEFORE = {}


def _host_weights(blk):
    bank = lambda b: (bits_u32(b.weight), bits_u16(b.scales), bits_u16(b.biases))
    return dict(router_w=bits_u16(blk.gate_weight), router_bias=None,
                gate=bank(blk.gate_proj), up=bank(blk.up_proj), down=bank(blk.down_proj))


@pytest.mark.parametrize("shape,names", BLOCK_CASES, ids=["H%d-I%d-E%d-k%d-T%d-b%d" % c for c, _ in BLOCK_CASES])
def test_variant_on_checked_rows(orc, shape, names):
    import mlx_rs_amd as m
    from mlx_rs_amd import synth
    H, I, E, k, T, bits = shape
    print(f"variant case H={H} I={I} E={E} k={k} T={T} bits={bits}: {names}", flush=True)
    if not LAUNCHES_BEFORE:
        LAUNCHES_BEFORE.update(m.capi.kernel_launches())
    cfg = m.MoeConfig(H, E, k, I, bits)
    plan = [n for n, _ in m.capi.plan_forward(cfg.c_struct(), T)]
    before = m.capi.kernel_launches()
    blk = synth.make_block(cfg, seed=17, device="cuda", gen_device="cuda")
    x = synth.make_tokens(cfg, T, seed=17, device="cuda")
    out, dbg = blk.forward(x, debug=True)
    torch.cuda.synchronize()
    after = m.capi.kernel_launches()
    launched = {n for n in after if after[n] > before[n]}
    assert launched == set(plan), "the planner and the forward disagree"
    counts = bits_u32(dbg["counts"])
    tiled, tmr = rules(H, I, E, k, T, bits)
    worked = kernels_with_rows(plan, counts, T, tiled, tmr)
    for n in names:
        assert n in worked, f"{n} was launched but the routing gave it no rows (rows per expert: {counts.tolist()})"
    ocfg = orc.make_config(H, E, k, I, bits, 64, cfg.score_mode)
    ref, d = orc.moe_forward(ocfg, _host_weights(blk), bits_u16(x), strict=True, n_threads=16)
    assert np.array_equal(d["topk_idx"], bits_u32(dbg["topk_idx"]).reshape(T, k))
    assert np.array_equal(d["perm"], bits_u32(dbg["perm"]))
    assert_close_bf16(bits_u16(out), ref, what=f"H={H} I={I} E={E} k={k} T={T} {bits}-bit")
    CHECKED.update(worked)


def test_variant_reached_by_the_operator_only(orc):
    import mlx_rs_amd as m
    c = OP_CASE
    rng = np.random.default_rng(3)
    N, K, rows = c["N"], c["K"], c["rows"]
    q, s, b = orc.quantize(rng.normal(0, 0.02, (N, K)).astype(np.float32), c["bits"], 64)
    x = orc.f32_to_bf16(rng.normal(0, 1, (rows, 1, K)).astype(np.float32))
    from helpers import bf16_tensor, i32_tensor
    before = m.capi.kernel_launches()
    y = m.ops.gather_qmm(bf16_tensor(x, "cuda"), i32_tensor(q.reshape(1, N, -1), "cuda"), bf16_tensor(s.reshape(1, N, -1), "cuda"),
                         bf16_tensor(b.reshape(1, N, -1), "cuda"), rhs_indices=torch.zeros(rows, dtype=torch.int32, device="cuda"),
                         transpose=True, group_size=64, bits=c["bits"])
    torch.cuda.synchronize()
    after = m.capi.kernel_launches()
    assert {n for n in after if after[n] > before[n]} == {c["variant"]}
    ref = f32_of_bits(x).astype(np.float64).reshape(rows, K) @ orc.dequantize(q, s, b, c["bits"], 64).astype(np.float64).T
    assert_close_bf16(bits_u16(y).reshape(rows, N), orc.f32_to_bf16(ref.astype(np.float32)), what="operator-only variant")
    CHECKED.add(c["variant"])


def test_zz_every_variant_ran_on_checked_rows():
    import mlx_rs_amd as m
    now = m.capi.kernel_launches()
    missing = sorted(set(now) - CHECKED)
    assert not missing, f"variants without a parity-checked launch: {missing}"
    assert all(now[n] > LAUNCHES_BEFORE.get(n, 0) for n in now), "the library's own counters disagree"
