"""mlx-rs_amd: MI355X-native quantized mixture-of-experts block with mlx-rs semantics.

The product is ``libmi_moe.so`` (hand-written HIP kernels for gfx950 behind the C ABI of
``include/mi_moe.h``).  This Python package is the thin host side used by the tests and
the benchmark: ``capi`` binds the C ABI with ctypes, ``ops`` mirrors the mlx-rs operator
names on torch tensors (torch is used for device memory and streams only), ``moe`` holds
the block with the ``forward`` / ``training_mode`` shape of an mlx-rs ``Module``.
There is no CPU fallback: every call fails loudly when the library is missing.
"""
from . import capi  # noqa: F401
from .capi import MoeError, library_path, load_library  # noqa: F401
from . import ops  # noqa: F401
from .moe import MoeConfig, QuantizedSwitchLinear, SparseMoeBlock  # noqa: F401
from . import synth  # noqa: F401

__all__ = ["capi", "ops", "synth", "MoeError", "MoeConfig", "QuantizedSwitchLinear",
           "SparseMoeBlock", "load_library", "library_path"]
