"""Operator-level host API on torch tensors, named after the mlx-rs functions whose MLX
dispatch each one replaces.  torch supplies device memory and the current stream; all
arithmetic happens in libmi_moe.so.

dtypes: activations/scales/biases ``torch.bfloat16`` on the hot path (the op-level functions also
take float16 and float32); packed weights and indices ``torch.int32`` holding the uint32 bit
patterns (torch has no arithmetic on uint32).
"""
import ctypes as C

import torch

from . import capi
from .capi import check, load_library


def _ptr(t):
    return None if t is None else C.c_void_p(t.data_ptr())


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _need(t, dtype, name):
    if t.dtype != dtype:
        raise capi.MoeError(f"{name}: expected dtype {dtype}, got {t.dtype}")
    if not t.is_cuda:
        raise capi.MoeError(f"{name}: expected a device tensor")
    if not t.is_contiguous():
        raise capi.MoeError(f"{name}: expected a contiguous tensor")
    return t


def _workspace(nbytes, device):
    return torch.empty(int(nbytes) + 256, dtype=torch.uint8, device=device)


_DTYPES = {torch.bfloat16: capi.DTYPE_BF16, torch.float16: capi.DTYPE_F16, torch.float32: capi.DTYPE_F32}


def _float_dtype(t, name):
    if t.dtype not in _DTYPES:
        raise capi.MoeError(f"{name}: expected bfloat16, float16 or float32, got {t.dtype}")
    if not t.is_cuda:
        raise capi.MoeError(f"{name}: expected a device tensor")
    if not t.is_contiguous():
        raise capi.MoeError(f"{name}: expected a contiguous tensor")
    return _DTYPES[t.dtype]


def quantize(w, group_size=64, bits=4, dtype=torch.bfloat16):
    """ops::quantize (mlx-rs/src/ops/quantization.rs:50-83): returns (w_q, scales, biases).
    w: float32 [rows, cols]; scales and biases come out in ``dtype`` (MLX gives them the type of its
    input: pass torch.float32 for the reference's float32 flows)."""
    lib = load_library()
    _need(w, torch.float32, "w")
    if dtype not in _DTYPES:
        raise capi.MoeError(f"quantize: dtype must be bfloat16, float16 or float32, got {dtype}")
    rows, cols = w.shape
    if cols % max(group_size, 1) or group_size not in (32, 64, 128) or bits not in (2, 4, 8):
        check(lib.mi_moe_quantize(None, rows, cols, group_size, bits, None, None, None, None))
    q = torch.empty((rows, cols * bits // 32), dtype=torch.int32, device=w.device)
    s = torch.empty((rows, cols // group_size), dtype=dtype, device=w.device)
    b = torch.empty_like(s)
    check(lib.mi_moe_quantize_typed(_ptr(w), rows, cols, group_size, bits, _DTYPES[dtype], _ptr(q), _ptr(s), _ptr(b),
                                    _stream()))
    return q, s, b


def dequantize(w_q, scales, biases, group_size=64, bits=4, dtype=None):
    """ops::dequantize (mlx-rs/src/ops/quantization.rs:124-158); scales and biases in bfloat16,
    float16 or float32.  The result has their element type, as the reference's has; ``dtype=torch.float32``
    asks for the fp32 values before that last rounding."""
    lib = load_library()
    _need(w_q, torch.int32, "w_q")
    dt = _float_dtype(scales, "scales")
    _need(biases, scales.dtype, "biases")
    if dtype is None:
        dtype = scales.dtype
    if dtype not in (scales.dtype, torch.float32):
        raise capi.MoeError(f"dequantize: dtype must be that of the scales ({scales.dtype}) or float32, got {dtype}")
    if w_q.dim() != 2:
        raise capi.MoeError("dequantize: w_q must be a matrix")
    rows = w_q.shape[0]
    cols = w_q.shape[1] * 32 // bits
    if group_size > 0 and cols % group_size == 0 and tuple(scales.shape) != (rows, cols // group_size):
        raise capi.MoeError(f"dequantize: scales must be [{rows}, {cols // group_size}], got {tuple(scales.shape)}")
    if biases.shape != scales.shape:
        raise capi.MoeError("dequantize: biases must have the shape of scales")
    out = torch.empty((rows, cols), dtype=dtype, device=w_q.device)
    fn = lib.mi_moe_dequantize_typed if dtype == torch.float32 else lib.mi_moe_dequantize_native
    check(fn(_ptr(w_q), _ptr(scales), _ptr(biases), rows, cols, group_size, bits, dt, _ptr(out), _stream()))
    return out


def _prod(shape):
    n = 1
    for d in shape:
        n *= int(d)
    return n


def gather_qmm(x, w, scales, biases, lhs_indices=None, rhs_indices=None, transpose=True,
               group_size=64, bits=4, sorted_indices=False):
    """ops::gather_qmm (mlx-rs/src/ops/quantization.rs:160-230), same argument order and defaults.
    x: [..., M, K] in bfloat16, float16 or float32 (scales and biases in the same type); w: int32
    [..., N, K*bits/32] (transpose = False: [..., K, N*bits/32]).  The leading axes of x and of w are
    batch axes; ``lhs_indices`` / ``rhs_indices`` (int32, any shapes) index the flattened batches and
    are broadcast against each other; an absent one counts through its batch.  Returns
    [*broadcast shape, M, N]."""
    lib = load_library()
    dt = _float_dtype(x, "x")
    _need(w, torch.int32, "w")
    _need(scales, x.dtype, "scales")
    if biases is None:
        raise capi.MoeError("gather_qmm: biases are required (affine quantisation)")
    _need(biases, x.dtype, "biases")
    if x.dim() < 2 or w.dim() < 2:
        raise capi.MoeError("gather_qmm: x must be [..., M, K] and w [..., N, K*bits/32]")
    M, K = x.shape[-2:]
    xb_shape, wb_shape = tuple(x.shape[:-2]), tuple(w.shape[:-2])
    xb, E = _prod(xb_shape), _prod(wb_shape)
    N = w.shape[-2] if transpose else w.shape[-1] * 32 // bits
    kw = w.shape[-1] * 32 // bits if transpose else w.shape[-2]
    if kw != K:
        raise capi.MoeError(f"gather_qmm: x has K = {K}, w has K = {kw}")
    if scales.dim() != w.dim() or biases.dim() != w.dim():
        raise capi.MoeError("gather_qmm: scales and biases must have as many axes as w")
    _check_qmat("gather_qmm", w, scales, biases, K, transpose, group_size, bits)
    dev = x.device

    def counted(shape):
        return torch.arange(_prod(shape), dtype=torch.int32, device=dev).reshape(shape)

    lhs = counted(xb_shape) if lhs_indices is None else lhs_indices
    rhs = counted(wb_shape) if rhs_indices is None else rhs_indices
    for t, name in ((lhs, "lhs_indices"), (rhs, "rhs_indices")):
        if t.dtype != torch.int32 or not t.is_cuda:
            raise capi.MoeError(f"gather_qmm: {name} must be an int32 device tensor")
    try:
        lhs_b, rhs_b = torch.broadcast_tensors(lhs, rhs)
    except RuntimeError as err:
        raise capi.MoeError(f"gather_qmm: index shapes {tuple(lhs.shape)} and {tuple(rhs.shape)} do not broadcast") from err
    out_batch = tuple(lhs_b.shape)
    lhs_f, rhs_f = lhs_b.reshape(-1).contiguous(), rhs_b.reshape(-1).contiguous()
    n_idx = rhs_f.numel()
    y = torch.empty((n_idx, M, N), dtype=x.dtype, device=dev)
    need = C.c_size_t()
    check(lib.mi_moe_gather_qmm_workspace_size(min(max(E, 1), 512), n_idx, M, C.byref(need)))
    ws = _workspace(need.value, dev)
    check(lib.mi_moe_gather_qmm_typed(
        _ptr(x), _ptr(w), _ptr(scales), _ptr(biases), _ptr(lhs_f), _ptr(rhs_f), n_idx, xb, M, N, K, E, int(transpose),
        group_size, bits, int(sorted_indices), dt, _ptr(y), _ptr(ws), ws.numel(), _stream()))
    return y.reshape(*out_batch, M, N)


def _check_qmat(who, w, scales, biases, K, transpose, group_size, bits):
    """Shapes of one quantized matrix against x's K: returns N.  w [N, K*bits/32] and scales / biases
    [N, K/group_size] with transpose, w [K, N*bits/32] and scales / biases [K, N/group_size] without."""
    if bits not in (2, 4, 8) or group_size not in (32, 64, 128):
        return None  # the library words the refusal
    per = 32 // bits
    if transpose:
        N, kw = w.shape[-2], w.shape[-1] * per
    else:
        N, kw = w.shape[-1] * per, w.shape[-2]
    if kw != K:
        raise capi.MoeError(f"{who}: x has K = {K}, w has K = {kw} (transpose = {bool(transpose)}, w {tuple(w.shape)})")
    rows, q_axis = (N, K) if transpose else (K, N)
    if q_axis % group_size == 0:
        want = (rows, q_axis // group_size)
        for t, name in ((scales, "scales"), (biases, "biases")):
            if tuple(t.shape[-2:]) != want or tuple(t.shape[:-2]) != tuple(w.shape[:-2]):
                raise capi.MoeError(f"{who}: {name} must be {tuple(w.shape[:-2]) + want}, got {tuple(t.shape)}")
    return N


def quantized_matmul(x, w, scales, biases, transpose=False, group_size=64, bits=4):
    """ops::quantized_matmul (mlx-rs/src/ops/quantization.rs:91-122), same argument order and defaults
    (``transpose`` defaults to False as there; QuantizedLinear passes True, mlx-rs/src/nn/quantized.rs:363-386).
    x: [..., K] in bfloat16, float16 or float32 (scales and biases in the same type).
    transpose = True: w int32 [N, K*bits/32], scales/biases [N, K/group_size];
    transpose = False: w int32 [K, N*bits/32], scales/biases [K, N/group_size].  Returns [..., N]."""
    return quantized_linear(x, w, scales, biases, None, transpose, group_size, bits, _who="quantized_matmul")


def quantized_linear(x, w, scales, biases, linear_bias=None, transpose=True, group_size=64, bits=4,
                     _who="quantized_linear"):
    """QuantizedLinear::forward (mlx-rs/src/nn/quantized.rs:363-386): quantized_matmul with
    transpose = True, then ``+ linear_bias`` ([N], x's type) when the layer has one; each of the two
    ops rounds to x's type, as the reference's."""
    lib = load_library()
    dt = _float_dtype(x, "x")
    _need(w, torch.int32, "w")
    _need(scales, x.dtype, "scales")
    _need(biases, x.dtype, "biases")
    if w.dim() != 2 or x.dim() < 1 or scales.dim() != 2 or biases.dim() != 2:
        raise capi.MoeError(f"{_who}: x must be [..., K], w, scales and biases matrices")
    K = x.shape[-1]
    N = _check_qmat(_who, w, scales, biases, K, transpose, group_size, bits)
    if N is None:
        N = w.shape[0] if transpose else w.shape[1] * 32 // max(bits, 1)
    if linear_bias is not None:
        if not transpose:
            raise capi.MoeError(f"{_who}: a linear bias goes with transpose = True (the layout of QuantizedLinear)")
        _need(linear_bias, x.dtype, "linear_bias")
        if linear_bias.numel() != N:
            raise capi.MoeError(f"{_who}: linear_bias must have {N} elements, got {linear_bias.numel()}")
    x2 = x.reshape(-1, K)
    M = x2.shape[0]
    y = torch.empty((M, N), dtype=x.dtype, device=x.device)
    need = C.c_size_t()
    check(lib.mi_moe_quantized_matmul_workspace_size(M, K, bits, C.byref(need)))
    ws = _workspace(need.value, x.device)
    if linear_bias is None:
        check(lib.mi_moe_quantized_matmul_typed(_ptr(x2), _ptr(w), _ptr(scales), _ptr(biases), M, N, K,
                                                1 if transpose else 0, group_size, bits, dt, _ptr(y), _ptr(ws),
                                                ws.numel(), _stream()))
    else:
        check(lib.mi_moe_quantized_linear_typed(_ptr(x2), _ptr(w), _ptr(scales), _ptr(biases), _ptr(linear_bias), M, N, K,
                                                group_size, bits, dt, _ptr(y), _ptr(ws), ws.numel(), _stream()))
    return y.reshape(*x.shape[:-1], N)


def rms_norm(x, weight, eps=1e-5):
    """fast::rms_norm (mlx-rs/src/fast.rs:190-207): weight * x * rsqrt(mean(x^2) + eps) over the last
    axis.  x: bf16 [..., H]; weight: bf16 [H]."""
    lib = load_library()
    _need(x, torch.bfloat16, "x")
    _need(weight, torch.bfloat16, "weight")
    H = x.shape[-1]
    if weight.numel() != H:
        raise capi.MoeError(f"rms_norm: weight must have {H} elements, got {weight.numel()}")
    x2 = x.reshape(-1, H)
    out = torch.empty_like(x2)
    check(lib.mi_moe_rms_norm(_ptr(x2), _ptr(weight), float(eps), x2.shape[0], H, _ptr(out), _stream()))
    return out.reshape(x.shape)


def router_logits(x, router_w, router_bias=None):
    """The gate Linear alone: bf16 logits [T, E] = x . router_w^T (+ router_bias), the way the block computes
    them (mi_moe_router_logits: above 64 tokens on the int8 matrix cores, with the bits of the fp64 route)."""
    lib = load_library()
    _need(x, torch.bfloat16, "x")
    _need(router_w, torch.bfloat16, "router_w")
    T, H = x.shape
    E = router_w.shape[0]
    if router_w.shape[1] != H:
        raise capi.MoeError(f"router_logits: x has {H} columns, router_w {router_w.shape[1]}")
    logits = torch.empty((T, E), dtype=torch.bfloat16, device=x.device)
    need = C.c_size_t()
    check(lib.mi_moe_router_logits_workspace_size(T, H, E, C.byref(need)))
    ws = _workspace(need.value, x.device)
    check(lib.mi_moe_router_logits(_ptr(x), _ptr(router_w),
                                   _ptr(None if router_bias is None else _need(router_bias, torch.float32, "router_bias")),
                                   T, H, E, _ptr(logits), _ptr(ws), ws.numel(), _stream()))
    return logits


def route(x, router_w, top_k, score_mode=capi.SCORE_SOFTMAX_THEN_TOPK_RENORM, router_bias=None,
          return_logits=False):
    """Gate Linear + softmax(precise) + top-k + scores in one call (what an mlx-lm MoE block
    does with matmul / softmax_axis / argpartition_axis / take_along_axis / sum_axis / divide).
    Returns (inds int32 [T,k], scores bf16 [T,k][, logits bf16 [T,E]])."""
    lib = load_library()
    _need(x, torch.bfloat16, "x")
    _need(router_w, torch.bfloat16, "router_w")
    T, H = x.shape
    E = router_w.shape[0]
    inds = torch.empty((T, top_k), dtype=torch.int32, device=x.device)
    sc = torch.empty((T, top_k), dtype=torch.bfloat16, device=x.device)
    logits = torch.empty((T, E), dtype=torch.bfloat16, device=x.device)
    need = C.c_size_t()
    check(lib.mi_moe_router_logits_workspace_size(T, H, E, C.byref(need)))  # room for the integer route's byte planes
    ws = _workspace(need.value + 256, x.device)
    check(lib.mi_moe_route(_ptr(x), _ptr(router_w),
                           _ptr(None if router_bias is None else _need(router_bias, torch.float32, "router_bias")),
                           T, H, E, top_k, score_mode, _ptr(inds), _ptr(sc), _ptr(logits), _ptr(ws), ws.numel(), _stream()))
    return (inds, sc, logits) if return_logits else (inds, sc)


def dispatch(expert_of_pair, n_experts):
    """Stable sort of the pairs by expert: returns (counts, offsets, perm, inv_perm), the
    results of mlx-lm's argsort / argsort / floor_divide sequence plus the histogram."""
    lib = load_library()
    flat = _need(expert_of_pair, torch.int32, "expert_of_pair").reshape(-1)
    P = flat.numel()
    dev = flat.device
    counts = torch.empty(n_experts, dtype=torch.int32, device=dev)
    offsets = torch.empty(n_experts + 1, dtype=torch.int32, device=dev)
    perm = torch.empty(P, dtype=torch.int32, device=dev)
    inv = torch.empty(P, dtype=torch.int32, device=dev)
    need = C.c_size_t()
    check(lib.mi_moe_dispatch_workspace_size(n_experts, P, C.byref(need)))
    ws = _workspace(need.value, dev)
    check(lib.mi_moe_dispatch(_ptr(flat), P, n_experts, _ptr(counts), _ptr(offsets), _ptr(perm), _ptr(inv),
                              _ptr(ws), ws.numel(), _stream()))
    return counts, offsets, perm, inv


def swiglu(gate, up):
    """nn::silu(gate) * up on bf16 tensors (mlx-rs/src/nn/activation.rs:142-144)."""
    lib = load_library()
    _need(gate, torch.bfloat16, "gate")
    _need(up, torch.bfloat16, "up")
    if gate.shape != up.shape:
        raise capi.MoeError("swiglu: gate and up must have the same shape")
    out = torch.empty_like(gate)
    check(lib.mi_moe_swiglu(_ptr(gate), _ptr(up), gate.numel(), _ptr(out), _stream()))
    return out


def combine(y, scores, inv_perm=None):
    """(y[inv] * scores[..., None]).sum(-2): y bf16 [P, H], scores bf16 [T, k] -> bf16 [T, H]."""
    lib = load_library()
    _need(y, torch.bfloat16, "y")
    _need(scores, torch.bfloat16, "scores")
    T, k = scores.shape
    H = y.shape[-1]
    out = torch.empty((T, H), dtype=torch.bfloat16, device=y.device)
    check(lib.mi_moe_combine(_ptr(y), _ptr(scores),
                             _ptr(None if inv_perm is None else _need(inv_perm, torch.int32, "inv_perm")),
                             T, k, H, _ptr(out), _stream()))
    return out
