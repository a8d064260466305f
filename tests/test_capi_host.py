"""Host-side checks of the C ABI that need no GPU: the library loads, exports every symbol the
header declares, and rejects bad arguments with a status and a message (never a crash), the way
mlx-sys calls report errors to mlx-rs (mlx-rs/src/utils/guard.rs:20-49, error.rs:226-280;
error-path tests ops/sort.rs:266-298)."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    import mlx_rs_amd as m
    return m.load_library()


def header_symbols():
    text = open(os.path.join(ROOT, "include", "mi_moe.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mi_moe_[a-z_0-9]+)\s*\(", text)))


def test_every_declared_symbol_is_exported(lib):
    import mlx_rs_amd as m
    syms = header_symbols()
    assert len(syms) >= 17
    for s in syms:
        assert hasattr(lib, s), f"{s} is declared in include/mi_moe.h but not exported"
    assert sorted(m.capi.EXPORTS) == syms
    assert lib.mi_moe_version().startswith(b"mi_moe")


def cfg(**kw):
    import mlx_rs_amd as m
    base = dict(hidden=256, n_experts=8, top_k=2, intermediate=512, bits=4, group_size=64, score_mode=0)
    base.update(kw)
    return m.capi.Config(**base)


@pytest.mark.parametrize("kw,needle", [
    (dict(hidden=100), "hidden"), (dict(bits=3), "bits"), (dict(group_size=48), "group_size"), (dict(group_size=128, hidden=192), "group_size"),
    (dict(top_k=9), "top_k"), (dict(top_k=0), "top_k"), (dict(n_experts=0), "n_experts"),
    (dict(intermediate=96), "intermediate"), (dict(score_mode=7), "score_mode"),
    (dict(hidden=192), "128"),
])
def test_bad_config_is_rejected_with_a_message(lib, kw, needle):
    import mlx_rs_amd as m
    n = C.c_size_t(12345)
    c = cfg(**kw)
    assert lib.mi_moe_workspace_size(C.byref(c), 4, C.byref(n)) != 0
    assert needle in m.capi.last_error()
    assert n.value == 12345                     # outputs untouched on failure
    with pytest.raises(m.MoeError):
        m.capi.check(1)


def test_null_and_range_checks(lib):
    import mlx_rs_amd as m
    c = cfg()
    n = C.c_size_t()
    assert lib.mi_moe_workspace_size(C.byref(c), 32, C.byref(n)) == 0 and n.value > 0
    assert lib.mi_moe_workspace_size(C.byref(c), -1, C.byref(n)) != 0
    assert lib.mi_moe_workspace_size(None, 1, C.byref(n)) != 0
    h = C.c_void_p()
    assert lib.mi_moe_create(C.byref(c), None, C.byref(h)) != 0 and "weights" in m.capi.last_error()
    w = m.capi.Weights()                          # all NULL
    assert lib.mi_moe_create(C.byref(c), C.byref(w), C.byref(h)) != 0 and not h.value
    assert lib.mi_moe_forward(None, None, 1, None, None, 0, None, None) != 0
    assert lib.mi_moe_forward(None, None, -1, None, None, 0, None, None) != 0
    assert lib.mi_moe_destroy(None) == 0
    # stage level
    assert lib.mi_moe_route(None, None, None, 4, 256, 8, 2, 0, None, None, None, None, 0, None) != 0
    assert lib.mi_moe_route(None, None, None, 4, 250, 8, 2, 0, None, None, None, None, 0, None) != 0
    assert "hidden" in m.capi.last_error()
    assert lib.mi_moe_dispatch(None, 8, 4, None, None, None, None, None, 0, None) != 0
    assert lib.mi_moe_gather_qmm(None, None, None, None, None, None, 2, 2, 1, 96, 64, 3, 0, 64, 4, 0,
                                 None, None, 0, None) != 0
    assert "group_size" in m.capi.last_error()     # untransposed weights are quantised along N: N % group_size
    assert lib.mi_moe_gather_qmm(None, None, None, None, None, None, 2, 2, 1, 64, 64, 3, 1, 64, 5, 0,
                                 None, None, 0, None) != 0
    assert "bits" in m.capi.last_error()
    # without lhs_indices index j reads x[j]: three indices need three matrices in x (checked before anything
    # is launched or any pointer followed: host memory stands in for the operands here)
    host = (C.c_char * 64)()
    fake = C.cast(host, C.c_void_p)
    assert lib.mi_moe_gather_qmm(fake, fake, fake, fake, None, fake, 3, 2, 1, 64, 128, 4, 1, 64, 4, 0,
                                 fake, None, 0, None) != 0
    assert "as many matrices in x" in m.capi.last_error()
    assert lib.mi_moe_combine(None, None, None, 4, 2, 64, None, None) != 0
    assert lib.mi_moe_swiglu(None, None, 8, None, None) != 0
    assert lib.mi_moe_stream_probe(None, 1000, None, None) != 0
    assert "32768" in m.capi.last_error()
    assert lib.mi_moe_stream_probe(None, 32768, None, None) != 0
    assert lib.mi_moe_quantize(None, 2, 100, 64, 4, None, None, None, None) != 0
    assert "divisible" in m.capi.last_error()
    assert lib.mi_moe_dequantize(None, None, None, 2, 128, 64, 3, None, None) != 0
    # entry points next to the path
    n2 = C.c_size_t(7)
    assert lib.mi_moe_quantized_matmul_workspace_size(-1, 128, 4, C.byref(n2)) != 0 and n2.value == 7
    assert lib.mi_moe_quantized_matmul_workspace_size(300, 256, 4, C.byref(n2)) == 0 and n2.value > 300 * 256 * 2
    assert lib.mi_moe_quantized_matmul(None, None, None, None, 4, 96, 128, 0, 64, 4, None, None, 0, None) != 0
    assert "group_size" in m.capi.last_error()
    assert lib.mi_moe_quantized_matmul(None, None, None, None, 4, 64, 100, 1, 32, 4, None, None, 0, None) != 0
    assert "K (100)" in m.capi.last_error()
    assert lib.mi_moe_quantized_matmul_typed(None, None, None, None, 4, 64, 128, 1, 64, 4, 3, None, None, 0, None) != 0
    assert "dtype" in m.capi.last_error()
    assert lib.mi_moe_quantize_typed(None, 2, 128, 64, 4, 9, None, None, None, None) != 0 and "dtype" in m.capi.last_error()
    assert lib.mi_moe_quantized_matmul(None, None, None, None, 0, 64, 128, 1, 64, 4, None, None, 0, None) == 0
    assert lib.mi_moe_rms_norm(None, None, 1e-5, 4, 100, None, None) != 0 and "hidden" in m.capi.last_error()
    assert lib.mi_moe_rms_norm(None, None, -1.0, 4, 128, None, None) != 0 and "eps" in m.capi.last_error()
    assert lib.mi_moe_rms_norm(None, None, 1e-5, 4, 128, None, None) != 0
    assert lib.mi_moe_rms_norm(None, None, 1e-5, 0, 128, None, None) == 0
    assert lib.mi_moe_forward_residual(None, None, None, 1e-5, 1, None, None, 0, None, None) != 0
    assert "norm_weight" in m.capi.last_error()
    # empty inputs succeed without touching memory
    assert lib.mi_moe_swiglu(None, None, 0, None, None) == 0
    assert lib.mi_moe_stream_probe(None, 0, None, None) == 0
    assert lib.mi_moe_combine(None, None, None, 0, 2, 64, None, None) == 0


def test_error_handler_receives_the_message(lib):
    import mlx_rs_amd as m
    seen = []
    cb = m.capi.ERROR_HANDLER(lambda msg, data: seen.append(msg.decode()))
    lib.mi_moe_set_error_handler(cb, None, C.cast(None, m.capi.ERROR_DTOR))
    try:
        assert lib.mi_moe_workspace_size(None, 1, None) != 0
        assert seen and "NULL" in seen[-1]
    finally:
        lib.mi_moe_set_error_handler(C.cast(None, m.capi.ERROR_HANDLER), None, C.cast(None, m.capi.ERROR_DTOR))


def test_missing_library_fails_loudly(monkeypatch):
    import mlx_rs_amd as m
    monkeypatch.setattr(m.capi, "_lib", None)
    monkeypatch.setattr(m.capi, "_SO", "/nonexistent/libmi_moe.so")
    with pytest.raises(m.MoeError):
        m.capi.load_library()


def test_operand_shapes_of_a_quantized_product_are_checked_on_the_host():
    """The shape check of ops.quantized_matmul / gather_qmm (no GPU needed: shapes only).  The reference's
    default is transpose = false (mlx-rs/src/ops/quantization.rs:101): a [N, K*bits/32] matrix handed over
    without transpose = true is refused, not read as [K, N'*bits/32]."""
    import inspect

    import torch

    from mlx_rs_amd import capi, ops
    assert inspect.signature(ops.quantized_matmul).parameters["transpose"].default is False
    assert inspect.signature(ops.gather_qmm).parameters["transpose"].default is True   # ops/quantization.rs:193
    N, K = 64, 256
    w = torch.empty((N, K // 8), dtype=torch.int32, device="meta")
    s = torch.empty((N, K // 64), dtype=torch.bfloat16, device="meta")
    assert ops._check_qmat("quantized_matmul", w, s, s, K, True, 64, 4) == N
    with pytest.raises(capi.MoeError, match="K = 256, w has K = 64"):
        ops._check_qmat("quantized_matmul", w, s, s, K, False, 64, 4)
    with pytest.raises(capi.MoeError, match="scales must be"):
        ops._check_qmat("quantized_matmul", w, s[:, :-1], s, K, True, 64, 4)
    wn = torch.empty((K, N // 8), dtype=torch.int32, device="meta")
    sn = torch.empty((K, N // 64), dtype=torch.bfloat16, device="meta")
    assert ops._check_qmat("quantized_matmul", wn, sn, sn, K, False, 64, 4) == N
    with pytest.raises(capi.MoeError, match="biases must be"):
        ops._check_qmat("quantized_matmul", wn, sn, s, K, False, 64, 4)
