"""The C++ host layer (mlx-rs_amd/host/mi_moe.hpp) driven through its test program
tests/cpp/host_mirror: error values on the CPU, and on the GPU the block, gather_qmm and
quantize/dequantize against the oracle on the same inputs (the C++ counterpart of what
test_gpu_block.py / test_gpu_stages.py check through the Python host layer)."""
import os
import subprocess

import numpy as np
import pytest

from helpers import assert_close_bf16, host_layer, host_tokens

HERE = os.path.dirname(os.path.abspath(__file__))
EXE = os.path.join(HERE, "cpp", "host_mirror")


@pytest.fixture(scope="module")
def exe():
    import mlx_rs_amd as m
    m.load_library()
    if not os.path.exists(EXE):
        subprocess.run(["make", "-C", os.path.join(HERE, "cpp")], check=True)
    return EXE


def test_error_values_without_a_gpu(exe):
    r = subprocess.run([exe, "errors"], capture_output=True, text=True, timeout=60)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "errors: ok" in r.stdout


@pytest.mark.gpu
@pytest.mark.parametrize("bits,mode", [(4, 0), (8, 2)])
def test_cpp_block_and_ops_match_the_oracle(exe, orc, tmp_path, bits, mode):
    H, E, k, I, T = 256, 8, 2, 512, 24
    W = host_layer(orc, H, E, k, I, bits, seed=5)
    x = host_tokens(orc, T, H, seed=5)
    rng = np.random.default_rng(9)
    wf = rng.normal(0, 0.05, (48, 256)).astype(np.float32)
    cfg = orc.make_config(H, E, k, I, bits, 64, mode)
    ref, d = orc.moe_forward(cfg, W, x, strict=False, n_threads=4)
    ref_half, _ = orc.moe_forward(cfg, W, x[:T // 2], strict=False, n_threads=4)
    lhs = np.repeat(np.arange(T, dtype=np.uint32), k)
    rhs = d["topk_idx"].reshape(-1).astype(np.uint32)
    for name, a in [("x", x), ("router_w", W["router_w"]), ("lhs", lhs), ("rhs", rhs), ("wf", wf)]:
        np.ascontiguousarray(a).tofile(tmp_path / f"{name}.bin")
    for bank in ("gate", "up", "down"):
        for suffix, a in zip("wsb", W[bank]):
            np.ascontiguousarray(a).tofile(tmp_path / f"{bank}_{suffix}.bin")
    (tmp_path / "cfg.txt").write_text(f"{H} {E} {k} {I} {bits} {mode} {T} {wf.shape[0]} {wf.shape[1]}\n")
    print(f"host_mirror forward bits={bits} mode={mode}", flush=True)
    r = subprocess.run([exe, "forward", str(tmp_path)], capture_output=True, text=True, timeout=100)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "forward: ok" in r.stdout

    out = np.fromfile(tmp_path / "out.bin", np.uint16).reshape(T, H)
    assert_close_bf16(out, ref, what="block")
    out2 = np.fromfile(tmp_path / "out2.bin", np.uint16).reshape(T // 2, H)
    assert_close_bf16(out2, ref_half, what="block, shorter second call")
    gq = np.fromfile(tmp_path / "gq.bin", np.uint16).reshape(T * k, 1, I)
    gref = orc.gather_qmm(x.reshape(T, 1, H), *W["gate"], lhs, rhs, bits=bits, want="bf16")
    assert_close_bf16(gq, gref, what="gather_qmm")
    q, s, b = orc.quantize(wf, 4, 64)
    assert np.array_equal(np.fromfile(tmp_path / "q.bin", np.uint32).reshape(q.shape), q)
    assert np.array_equal(np.fromfile(tmp_path / "s.bin", np.uint16).reshape(s.shape), s)
    assert np.array_equal(np.fromfile(tmp_path / "b.bin", np.uint16).reshape(b.shape), b)
    dq = np.fromfile(tmp_path / "dq.bin", np.float32).reshape(wf.shape)
    assert np.array_equal(dq, orc.dequantize(q, s, b, 4, 64))
