"""ctypes binding of include/mi_moe.h (one function per exported symbol)."""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libmi_moe.so")

SCORE_SOFTMAX_THEN_TOPK_RENORM = 0
SCORE_SOFTMAX_THEN_TOPK = 1
SCORE_TOPK_THEN_SOFTMAX = 2
DTYPE_BF16, DTYPE_F16, DTYPE_F32 = 0, 1, 2
N_STAGES = 6
N_KERNEL_TIMES = 8
KERNEL_NAMES = ("gate_up_tiles256", "gate_up_tiles128", "gate_up_tiles64", "gate_up_streamed",
                "down_tiles256", "down_tiles128", "down_tiles64", "down_streamed")
STATIC_SCRATCH_BYTES = 8388608
STAGE_NAMES = ("router_logits", "router_select", "dispatch", "gate_up_swiglu", "down", "combine")

# every symbol include/mi_moe.h declares
EXPORTS = (
    "mi_moe_last_error", "mi_moe_set_error_handler", "mi_moe_version", "mi_moe_create",
    "mi_moe_destroy", "mi_moe_workspace_size", "mi_moe_forward", "mi_moe_forward_static", "mi_moe_forward_residual",
    "mi_moe_rms_norm", "mi_moe_forward_timed",
    "mi_moe_route_workspace_size",
    "mi_moe_route", "mi_moe_dispatch_workspace_size", "mi_moe_dispatch",
    "mi_moe_gather_qmm_workspace_size", "mi_moe_gather_qmm",
    "mi_moe_quantized_matmul_workspace_size", "mi_moe_quantized_matmul", "mi_moe_swiglu", "mi_moe_combine",
    "mi_moe_quantize", "mi_moe_dequantize", "mi_moe_stream_probe",
    "mi_moe_gather_qmm_typed", "mi_moe_quantized_matmul_typed", "mi_moe_quantize_typed", "mi_moe_dequantize_typed",
    "mi_moe_quantized_linear_typed", "mi_moe_dequantize_native",
    "mi_moe_debug_kernel_count", "mi_moe_debug_kernel_name", "mi_moe_debug_kernel_launches", "mi_moe_debug_plan_forward", "mi_moe_debug_plan_grouped",
    "mi_moe_debug_side_streams_created", "mi_moe_debug_tile_rule",
    "mi_moe_router_logits_workspace_size", "mi_moe_router_logits",
)


class MoeError(RuntimeError):
    """A non-zero status from the library; ``what`` is the library's message
    (the role of mlx-rs's ``Exception { what }``, mlx-rs/src/error.rs:162-192)."""

    def __init__(self, what):
        super().__init__(what)
        self.what = what


class Config(C.Structure):
    _fields_ = [(n, C.c_int32) for n in
                ("hidden", "n_experts", "top_k", "intermediate", "bits", "group_size", "score_mode")]


class QMat(C.Structure):
    _fields_ = [("w", C.c_void_p), ("scales", C.c_void_p), ("biases", C.c_void_p)]


class Weights(C.Structure):
    _fields_ = [("router_w", C.c_void_p), ("router_bias", C.c_void_p),
                ("gate", QMat), ("up", QMat), ("down", QMat)]


class DebugOut(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in
                ("topk_idx", "topk_w", "counts", "offsets", "perm", "inv_perm")]


ERROR_HANDLER = C.CFUNCTYPE(None, C.c_char_p, C.c_void_p)
ERROR_DTOR = C.CFUNCTYPE(None, C.c_void_p)

_lib = None


def library_path():
    return _SO


def load_library():
    """Load libmi_moe.so built in-tree by ``__graft_entry__.build()`` (or the Makefile in
    csrc/).  Raises if it is missing: there is no other code path."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_SO):
        raise MoeError(f"{_SO} is missing: build it with `make -C {_HERE}/csrc` "
                       "(or __graft_entry__.build()); there is no fallback path")
    lib = C.CDLL(_SO)
    vp, i32, i64, sz = C.c_void_p, C.c_int32, C.c_int64, C.c_size_t
    lib.mi_moe_last_error.restype = C.c_char_p
    lib.mi_moe_last_error.argtypes = []
    lib.mi_moe_version.restype = C.c_char_p
    lib.mi_moe_version.argtypes = []
    lib.mi_moe_set_error_handler.restype = None
    lib.mi_moe_set_error_handler.argtypes = [ERROR_HANDLER, vp, ERROR_DTOR]
    sigs = {
        "mi_moe_create": [C.POINTER(Config), C.POINTER(Weights), C.POINTER(vp)],
        "mi_moe_destroy": [vp],
        "mi_moe_workspace_size": [C.POINTER(Config), i64, C.POINTER(sz)],
        "mi_moe_forward": [vp, vp, i64, vp, vp, sz, C.POINTER(DebugOut), vp],
        "mi_moe_forward_static": [vp, vp, i64, vp, C.POINTER(DebugOut), vp],
        "mi_moe_forward_timed": [vp, vp, i64, vp, vp, sz, vp, C.POINTER(C.c_float), C.POINTER(C.c_float)],
        "mi_moe_forward_residual": [vp, vp, vp, C.c_float, i64, vp, vp, sz, C.POINTER(DebugOut), vp],
        "mi_moe_rms_norm": [vp, vp, C.c_float, i64, i32, vp, vp],
        "mi_moe_route_workspace_size": [i32, i64, C.POINTER(sz)],
        "mi_moe_route": [vp, vp, vp, i64, i32, i32, i32, i32, vp, vp, vp, vp, sz, vp],
        "mi_moe_router_logits_workspace_size": [i64, i32, i32, C.POINTER(sz)],
        "mi_moe_router_logits": [vp, vp, vp, i64, i32, i32, vp, vp, sz, vp],
        "mi_moe_dispatch_workspace_size": [i32, i64, C.POINTER(sz)],
        "mi_moe_dispatch": [vp, i64, i32, vp, vp, vp, vp, vp, sz, vp],
        "mi_moe_gather_qmm_workspace_size": [i32, i64, i32, C.POINTER(sz)],
        "mi_moe_gather_qmm": [vp, vp, vp, vp, vp, vp, i64, i64, i32, i32, i32, i32, i32, i32, i32,
                              i32, vp, vp, sz, vp],
        "mi_moe_quantized_matmul_workspace_size": [i64, i32, i32, C.POINTER(sz)],
        "mi_moe_quantized_matmul": [vp, vp, vp, vp, i64, i32, i32, i32, i32, i32, vp, vp, sz, vp],
        "mi_moe_swiglu": [vp, vp, i64, vp, vp],
        "mi_moe_combine": [vp, vp, vp, i64, i32, i32, vp, vp],
        "mi_moe_quantize": [vp, i64, i64, i32, i32, vp, vp, vp, vp],
        "mi_moe_dequantize": [vp, vp, vp, i64, i64, i32, i32, vp, vp],
        "mi_moe_stream_probe": [vp, sz, vp, vp],
        "mi_moe_gather_qmm_typed": [vp, vp, vp, vp, vp, vp, i64, i64, i32, i32, i32, i32, i32, i32, i32,
                                    i32, i32, vp, vp, sz, vp],
        "mi_moe_quantized_matmul_typed": [vp, vp, vp, vp, i64, i32, i32, i32, i32, i32, i32, vp, vp, sz, vp],
        "mi_moe_quantize_typed": [vp, i64, i64, i32, i32, i32, vp, vp, vp, vp],
        "mi_moe_dequantize_typed": [vp, vp, vp, i64, i64, i32, i32, i32, vp, vp],
        "mi_moe_dequantize_native": [vp, vp, vp, i64, i64, i32, i32, i32, vp, vp],
        "mi_moe_quantized_linear_typed": [vp, vp, vp, vp, vp, i64, i32, i32, i32, i32, i32, vp, vp, sz, vp],
        "mi_moe_debug_plan_forward": [C.POINTER(Config), i64, C.c_char_p, sz],
        "mi_moe_debug_tile_rule": [C.POINTER(Config), i64, C.POINTER(i32), C.POINTER(i32)],
        "mi_moe_debug_plan_grouped": [i32, i32, i32, i32, i64, i32, i64, i64, i32, i32, C.c_char_p, sz],
    }
    for name, args in sigs.items():
        fn = getattr(lib, name)
        fn.restype = C.c_int
        fn.argtypes = args
    for name in ("mi_moe_debug_kernel_count", "mi_moe_debug_side_streams_created"):
        getattr(lib, name).restype = C.c_int32
        getattr(lib, name).argtypes = []
    lib.mi_moe_debug_kernel_name.restype = C.c_char_p
    lib.mi_moe_debug_kernel_name.argtypes = [i32]
    lib.mi_moe_debug_kernel_launches.restype = i64
    lib.mi_moe_debug_kernel_launches.argtypes = [i32]
    _lib = lib
    return lib


def kernel_launches():
    """{variant name: launches in this process} for every grouped-product kernel variant the library holds."""
    lib = load_library()
    out = {}
    for i in range(lib.mi_moe_debug_kernel_count()):
        out[lib.mi_moe_debug_kernel_name(i).decode()] = lib.mi_moe_debug_kernel_launches(i)
    return out


def _plan_entries(buf):
    out = []
    for item in buf.value.decode().split(";"):
        if item:
            name, *rest = item.split(" ")
            out.append((name, {k: v for k, v in (r.split("=") for r in rest)}))
    return out


def tile_rule(cfg, tokens):
    """(tile lists are built, rows from which a segment is tiled) for a forward of `tokens` tokens: the
    library's own rule (needs no GPU)."""
    tiled, tmr = C.c_int32(), C.c_int32()
    check(load_library().mi_moe_debug_tile_rule(C.byref(cfg), tokens, C.byref(tiled), C.byref(tmr)))
    return bool(tiled.value), tmr.value


def segment_rows_by_kernel(count, tiled, tmr):
    """Rows of a segment of `count` rows that each grouped-product kernel takes:
    [256-row tiles, 128-row tiles, 64-row tiles, streamed] (see tile_rule)."""
    count = int(count)
    if not tiled or count < tmr:
        return [0, 0, 0, count]
    full, r = divmod(count, 256)
    rows = [full * 256, 0, 0, 0]
    if r > 128:
        rows[0] += r
    elif r > 64:
        rows[1] = r
    else:
        rows[2] = r
    return rows


def plan_forward(cfg, tokens):
    """The grouped-product kernel variants a forward of `tokens` tokens would launch, as
    [(name, {"grid": "AxB", "block": "256", "lds": bytes})]; launches nothing and needs no GPU."""
    lib = load_library()
    buf = C.create_string_buffer(4096)
    check(lib.mi_moe_debug_plan_forward(C.byref(cfg), tokens, buf, len(buf)))
    return _plan_entries(buf)


def plan_grouped(N, K, bits, glu, total_rows, max_active, max_rows_per_expert, max_streamed_rows=0, tile_lists=False,
                 paired_out=False):
    lib = load_library()
    buf = C.create_string_buffer(4096)
    check(lib.mi_moe_debug_plan_grouped(N, K, bits, int(glu), total_rows, max_active, max_rows_per_expert,
                                        max_streamed_rows, int(tile_lists), int(paired_out), buf, len(buf)))
    return _plan_entries(buf)


def last_error():
    return load_library().mi_moe_last_error().decode()


def check(status):
    """Turn a status into an exception the way mlx-rs's Guarded::try_from_op does
    (mlx-rs/src/utils/guard.rs:20-49)."""
    if status != 0:
        raise MoeError(last_error())
