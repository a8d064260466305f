"""The sparse MoE block, shaped like an mlx-rs ``Module<&Array>``:
``forward(x) -> Array`` and ``training_mode(bool)`` (mlx-rs/src/module/module.rs:28-50);
it stands where the dense ``Mlp`` stands in mlx-lm/src/models/qwen3.rs:204-255,321-324.

Parameters keep the names and layouts of an mlx-community quantized checkpoint:
``gate.weight`` bf16 [E,H]; ``switch_mlp.{gate_proj,up_proj,down_proj}.{weight u32
[E,N,K*bits/32], scales bf16 [E,N,K/64], biases bf16 [E,N,K/64]}``.
"""
import ctypes as C
from dataclasses import dataclass

import torch

from . import capi
from .capi import check, load_library
from .ops import _need, _ptr, _stream


@dataclass
class MoeConfig:
    hidden: int
    n_experts: int
    top_k: int
    intermediate: int
    bits: int = 4
    group_size: int = 64
    score_mode: int = capi.SCORE_SOFTMAX_THEN_TOPK_RENORM

    def c_struct(self):
        return capi.Config(self.hidden, self.n_experts, self.top_k, self.intermediate, self.bits,
                           self.group_size, self.score_mode)


@dataclass
class QuantizedSwitchLinear:
    """A bank of E quantized matrices (QuantizedLinear's fields, mlx-rs/src/nn/quantized.rs:
    254-279, with a leading expert axis)."""
    weight: torch.Tensor  # int32 [E, N, K*bits/32]
    scales: torch.Tensor  # bf16 [E, N, K/64]
    biases: torch.Tensor  # bf16 [E, N, K/64]

    def c_struct(self):
        _need(self.weight, torch.int32, "weight")
        _need(self.scales, torch.bfloat16, "scales")
        _need(self.biases, torch.bfloat16, "biases")
        return capi.QMat(self.weight.data_ptr(), self.scales.data_ptr(), self.biases.data_ptr())


class SparseMoeBlock:
    def __init__(self, config, gate_weight, gate_proj, up_proj, down_proj, router_bias=None):
        self.config = config
        self.gate_weight = _need(gate_weight, torch.bfloat16, "gate.weight")
        self.router_bias = router_bias
        self.gate_proj, self.up_proj, self.down_proj = gate_proj, up_proj, down_proj
        self._lib = load_library()
        self._handle = C.c_void_p()
        self._cfg = config.c_struct()
        w = capi.Weights(self.gate_weight.data_ptr(),
                         None if router_bias is None else _need(router_bias, torch.float32, "router_bias").data_ptr(),
                         gate_proj.c_struct(), up_proj.c_struct(), down_proj.c_struct())
        check(self._lib.mi_moe_create(C.byref(self._cfg), C.byref(w), C.byref(self._handle)))
        self._ws = None
        self._ws_tokens = -1
        self.training = False

    def __del__(self):
        h = getattr(self, "_handle", None)
        if h is not None and h.value:
            self._lib.mi_moe_destroy(h)
            self._handle = C.c_void_p()

    def training_mode(self, mode):
        """No layer of the block behaves differently in training (module.rs:44-50)."""
        self.training = bool(mode)

    def workspace_bytes(self, tokens):
        need = C.c_size_t()
        check(self._lib.mi_moe_workspace_size(C.byref(self._cfg), tokens, C.byref(need)))
        return need.value

    def reserve(self, tokens):
        if tokens > self._ws_tokens:
            self._ws = torch.empty(self.workspace_bytes(tokens) + 256, dtype=torch.uint8,
                                   device=self.gate_weight.device)
            self._ws_tokens = tokens
        return self._ws

    def forward_residual(self, x, norm_weight, eps=1e-5, debug=False, out=None):
        """x + self(rms_norm(x, norm_weight, eps)): the block with the layer norm in front of it and
        the residual add behind it (mlx-lm/src/models/qwen3.rs:310-325) in one call."""
        return self.forward(x, debug=debug, out=out, _norm=(_need(norm_weight, torch.bfloat16, "norm_weight"), eps))

    @staticmethod
    def _check_out(out, x2, who):
        """`out` is written through its raw pointer: it must be what the kernels assume."""
        _need(out, torch.bfloat16, "out")
        if out.device != x2.device:
            raise capi.MoeError(f"{who}: out is on {out.device}, x on {x2.device}")
        if out.numel() != x2.numel():
            raise capi.MoeError(f"{who}: out must hold {x2.numel()} elements, got {out.numel()}")
        return out

    def forward_static(self, x, out=None):
        """forward() on the library's built-in scratch instead of a workspace tensor
        (mi_moe_forward_static): nothing is allocated by the call when ``out`` is given.  Raises
        when the batch needs more workspace than the scratch holds.  Every call on one GPU, through
        whatever block, uses the same scratch array: calls that overlap on a GPU (two streams, two
        threads) race, so keep them on one stream or order them with events."""
        _need(x, torch.bfloat16, "x")
        c = self.config
        if x.shape[-1] != c.hidden:
            raise capi.MoeError(f"forward_static: last dimension must be {c.hidden}, got {x.shape[-1]}")
        x2 = x.reshape(-1, c.hidden)
        if out is None:
            out = torch.empty_like(x2)
        else:
            self._check_out(out, x2, "forward_static")
        check(self._lib.mi_moe_forward_static(self._handle, _ptr(x2), x2.shape[0], _ptr(out), None, _stream()))
        return out.reshape(x.shape)

    def forward(self, x, debug=False, out=None, _norm=None):
        """x: bf16 [..., H] -> bf16 [..., H].  With debug=True also returns the routing
        arrays (topk_idx, topk_w, counts, offsets, perm, inv_perm)."""
        _need(x, torch.bfloat16, "x")
        c = self.config
        if x.shape[-1] != c.hidden:
            raise capi.MoeError(f"forward: last dimension must be {c.hidden}, got {x.shape[-1]}")
        x2 = x.reshape(-1, c.hidden)
        T = x2.shape[0]
        if out is None:
            out = torch.empty_like(x2)
        else:
            self._check_out(out, x2, "forward")
        ws = self.reserve(max(T, 1))
        dbg_struct, dbg = None, None
        if debug:
            dev, P = x.device, T * c.top_k
            dbg = dict(topk_idx=torch.empty((T, c.top_k), dtype=torch.int32, device=dev),
                       topk_w=torch.empty((T, c.top_k), dtype=torch.bfloat16, device=dev),
                       counts=torch.empty(c.n_experts, dtype=torch.int32, device=dev),
                       offsets=torch.empty(c.n_experts + 1, dtype=torch.int32, device=dev),
                       perm=torch.empty(P, dtype=torch.int32, device=dev),
                       inv_perm=torch.empty(P, dtype=torch.int32, device=dev))
            dbg_struct = capi.DebugOut(*[dbg[n].data_ptr() for n in
                                         ("topk_idx", "topk_w", "counts", "offsets", "perm", "inv_perm")])
        dbg_arg = None if dbg_struct is None else C.byref(dbg_struct)
        if _norm is None:
            check(self._lib.mi_moe_forward(self._handle, _ptr(x2), T, _ptr(out), _ptr(ws), ws.numel(), dbg_arg,
                                           _stream()))
        else:
            if _norm[0].numel() != c.hidden:
                raise capi.MoeError(f"forward_residual: norm_weight must have {c.hidden} elements")
            check(self._lib.mi_moe_forward_residual(self._handle, _ptr(x2), _ptr(_norm[0]), float(_norm[1]), T,
                                                    _ptr(out), _ptr(ws), ws.numel(), dbg_arg, _stream()))
        out = out.reshape(x.shape)
        return (out, dbg) if debug else out

    __call__ = forward

    def forward_timed(self, x, out=None, kernels=False):
        """One forward with HIP events between the stages; returns (out, stage_ms list) and, with
        kernels=True, the grouped-product kernels' own durations (capi.KERNEL_NAMES) as well."""
        _need(x, torch.bfloat16, "x")
        x2 = x.reshape(-1, self.config.hidden)
        T = x2.shape[0]
        if out is None:
            out = torch.empty_like(x2)
        else:
            self._check_out(out, x2, "forward_timed")
        ws = self.reserve(max(T, 1))
        ms = (C.c_float * capi.N_STAGES)()
        kms = (C.c_float * capi.N_KERNEL_TIMES)()
        check(self._lib.mi_moe_forward_timed(self._handle, _ptr(x2), T, _ptr(out), _ptr(ws), ws.numel(),
                                             _stream(), ms, kms))
        if kernels:
            return out.reshape(x.shape), list(ms), list(kms)
        return out.reshape(x.shape), list(ms)
