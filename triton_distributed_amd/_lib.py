"""ctypes binding of libfdk.so (declarations: include/fdk.h, measurement aids: include/fdk_measure.h).

The library is loaded from ``triton_distributed_amd/lib/libfdk.so``.  There is no fallback: if the file
is missing or a symbol is absent, importing the decode entry points raises.
"""
from __future__ import annotations

import ctypes as C
import os
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "lib" / "libfdk.so"

FDK_ABI_VERSION = 8
FDK_ABI_REVISION = 2      # the library may be newer (its structs only grow at the end), never older

# fdk_dtype
FDK_BF16, FDK_FP16, FDK_FP8_E4M3, FDK_FP32 = 0, 1, 2, 3
# fdk_status
FDK_OK, FDK_ENULL, FDK_EALIGN, FDK_ESHAPE, FDK_EUNSUPPORTED, FDK_EWORKSPACE, FDK_EABI = 0, -1, -2, -3, -4, -5, -6
# fdk_algo
FDK_ALGO_AUTO, FDK_ALGO_VALU, FDK_ALGO_MFMA = 0, 1, 2
# flags
FDK_FLAG_PACK_LSE, FDK_FLAG_DRY_RUN, FDK_FLAG_SINGLE_LAUNCH, FDK_FLAG_FP8_FOLD_K_SCALE = 1, 2, 8, 16
FDK_STATIC_SCRATCH_BYTES = 32 << 20

# declared in include/fdk.h
EXPORTS = (
    "fdk_abi_version", "fdk_abi_revision", "fdk_last_error", "fdk_device_cus", "fdk_plan", "fdk_workspace_bytes",
    "fdk_decode", "fdk_decode_splitkv", "fdk_combine", "fdk_combine_ranks", "fdk_counters_len", "fdk_kv_append",
    "fdk_decode_static", "fdk_length_feedback_alloc", "fdk_length_feedback_free",
)
# declared in include/fdk_measure.h
MEASURE_EXPORTS = ("fdk_probe_linear_read",)


class FdkPlan(C.Structure):
    _fields_ = [("num_splits", C.c_int32), ("chunk_tokens", C.c_int32), ("algo", C.c_int32),
                ("kv_heads_per_wg", C.c_int32), ("balanced", C.c_int32), ("workgroups", C.c_int32),
                ("chunk_floor", C.c_int32), ("reserved", C.c_int32)]


class FdkDecodeArgs(C.Structure):
    _fields_ = [
        ("struct_size", C.c_uint32), ("flags", C.c_uint32),
        ("q", C.c_void_p), ("q_stride_b", C.c_int64), ("q_stride_h", C.c_int64), ("q_dtype", C.c_int32),
        ("kv_dtype", C.c_int32), ("k_cache", C.c_void_p), ("v_cache", C.c_void_p),
        ("k_stride_page", C.c_int64), ("k_stride_tok", C.c_int64), ("k_stride_head", C.c_int64),
        ("v_stride_page", C.c_int64), ("v_stride_tok", C.c_int64), ("v_stride_head", C.c_int64),
        ("k_scale", C.c_void_p), ("v_scale", C.c_void_p),
        ("block_table", C.c_void_p), ("table_stride_b", C.c_int64), ("kv_lens", C.c_void_p),
        ("batch", C.c_int32), ("num_q_heads", C.c_int32), ("num_kv_heads", C.c_int32), ("head_dim", C.c_int32),
        ("page_size", C.c_int32), ("max_pages", C.c_int32), ("max_kv_len", C.c_int32),
        ("min_kv_len", C.c_int32), ("num_splits", C.c_int32),
        ("sm_scale", C.c_float), ("soft_cap", C.c_float),
        ("out", C.c_void_p), ("out_stride_b", C.c_int64), ("out_stride_h", C.c_int64),
        ("out_dtype", C.c_int32), ("algo", C.c_int32),
        ("lse", C.c_void_p), ("lse_stride_b", C.c_int64),
        ("workspace", C.c_void_p), ("workspace_bytes", C.c_size_t),
        ("counters", C.c_void_p), ("counters_len", C.c_int64),
        ("reserved0", C.c_int32 * 4),
        ("length_feedback", C.c_void_p),
        ("reserved1", C.c_void_p), ("reserved2", C.c_int64),
        ("measure", C.c_void_p),           # FdkMeasureArgs*, null in product use
        ("v_head_dim", C.c_int32), ("reserved3", C.c_int32),     # (revision 2) 0: V rows as long as q / K rows
    ]


class FdkMeasureArgs(C.Structure):
    """include/fdk_measure.h: overrides and probes of the benchmark; never changes a result."""
    _fields_ = [
        ("struct_size", C.c_uint32), ("probe_loads", C.c_uint32),
        ("wavefronts", C.c_int32), ("buffers", C.c_int32), ("shares_per_cu", C.c_int32), ("rotate_heads", C.c_int32),
        ("timeline", C.c_void_p), ("timeline_len", C.c_int64),
        ("force_balanced", C.c_int32), ("reserved", C.c_int32),
    ]


class FdkCombineRanksArgs(C.Structure):
    _fields_ = [
        ("struct_size", C.c_uint32), ("flags", C.c_uint32),
        ("partial", C.c_void_p), ("stride_r", C.c_int64), ("stride_b", C.c_int64), ("stride_h", C.c_int64),
        ("partial_dtype", C.c_int32), ("out_dtype", C.c_int32),
        ("partial_lse", C.c_void_p), ("lse_stride_r", C.c_int64), ("lse_stride_b", C.c_int64),
        ("kv_lens", C.c_void_p),
        ("num_ranks", C.c_int32), ("batch", C.c_int32), ("num_q_heads", C.c_int32), ("head_dim", C.c_int32),
        ("out", C.c_void_p), ("out_stride_b", C.c_int64), ("out_stride_h", C.c_int64),
        ("lse", C.c_void_p), ("lse_stride_b_out", C.c_int64),
    ]


class FdkKvAppendArgs(C.Structure):
    _fields_ = [
        ("struct_size", C.c_uint32), ("flags", C.c_uint32),
        ("qkv", C.c_void_p), ("qkv_stride_b", C.c_int64), ("qkv_stride_t", C.c_int64), ("qkv_stride_h", C.c_int64),
        ("qkv_dtype", C.c_int32), ("kv_dtype", C.c_int32),
        ("q_weight", C.c_void_p), ("k_weight", C.c_void_p), ("q_eps", C.c_float), ("k_eps", C.c_float),
        ("cos", C.c_void_p), ("sin", C.c_void_p), ("cs_stride_b", C.c_int64), ("cs_stride_pos", C.c_int64),
        ("max_positions", C.c_int32),
        ("batch", C.c_int32), ("new_tokens", C.c_int32), ("num_q_heads", C.c_int32), ("num_kv_heads", C.c_int32),
        ("head_dim", C.c_int32),
        ("block_table", C.c_void_p), ("table_stride_b", C.c_int64), ("kv_lens", C.c_void_p),
        ("page_size", C.c_int32), ("max_pages", C.c_int32), ("num_pages", C.c_int32),
        ("k_cache", C.c_void_p), ("v_cache", C.c_void_p),
        ("k_stride_page", C.c_int64), ("k_stride_tok", C.c_int64), ("k_stride_head", C.c_int64),
        ("v_stride_page", C.c_int64), ("v_stride_tok", C.c_int64), ("v_stride_head", C.c_int64),
        ("k_scale", C.c_void_p), ("v_scale", C.c_void_p),
        ("q_out", C.c_void_p), ("q_out_stride_b", C.c_int64), ("q_out_stride_t", C.c_int64),
        ("q_out_stride_h", C.c_int64),
    ]


class FdkError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(f"fdk error {code}: {message}")
        self.code = code
        self.message = message


_lib = None


def load() -> C.CDLL:
    """Load libfdk.so once and type its entry points.  Raises if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    path = os.environ.get("FDK_LIBRARY", str(LIB_PATH))
    if not os.path.exists(path):
        raise ImportError(
            f"{path} not found: build it with `python -m triton_distributed_amd.build` (hipcc, gfx950). "
            "There is no fallback implementation.")
    lib = C.CDLL(path)
    for name in EXPORTS + MEASURE_EXPORTS:
        if not hasattr(lib, name):
            raise ImportError(f"{path} does not export {name}")
    lib.fdk_abi_version.restype = C.c_int
    lib.fdk_abi_version.argtypes = []
    lib.fdk_abi_revision.restype = C.c_int
    lib.fdk_abi_revision.argtypes = []
    lib.fdk_last_error.restype = C.c_char_p
    lib.fdk_last_error.argtypes = []
    lib.fdk_device_cus.restype = C.c_int
    lib.fdk_device_cus.argtypes = []
    lib.fdk_plan.restype = C.c_int
    lib.fdk_plan.argtypes = [C.POINTER(FdkDecodeArgs), C.c_int, C.POINTER(FdkPlan)]
    lib.fdk_workspace_bytes.restype = C.c_size_t
    lib.fdk_workspace_bytes.argtypes = [C.c_int32, C.c_int32, C.c_int32, C.c_int32]
    for name in ("fdk_decode", "fdk_decode_static", "fdk_decode_splitkv", "fdk_combine"):
        fn = getattr(lib, name)
        fn.restype = C.c_int
        fn.argtypes = [C.POINTER(FdkDecodeArgs), C.c_void_p]
    lib.fdk_counters_len.restype = C.c_int64
    lib.fdk_counters_len.argtypes = [C.POINTER(FdkDecodeArgs)]
    lib.fdk_combine_ranks.restype = C.c_int
    lib.fdk_combine_ranks.argtypes = [C.POINTER(FdkCombineRanksArgs), C.c_void_p]
    lib.fdk_probe_linear_read.restype = C.c_int
    lib.fdk_probe_linear_read.argtypes = [C.c_void_p, C.c_size_t, C.c_int, C.c_int, C.c_void_p]
    lib.fdk_length_feedback_alloc.restype = C.c_int
    lib.fdk_length_feedback_alloc.argtypes = [C.POINTER(C.c_void_p), C.POINTER(C.c_void_p)]
    lib.fdk_length_feedback_free.restype = C.c_int
    lib.fdk_length_feedback_free.argtypes = [C.c_void_p]
    lib.fdk_kv_append.restype = C.c_int
    lib.fdk_kv_append.argtypes = [C.POINTER(FdkKvAppendArgs), C.c_void_p]
    if lib.fdk_abi_version() != FDK_ABI_VERSION or lib.fdk_abi_revision() < FDK_ABI_REVISION:
        raise ImportError(f"{path}: ABI {lib.fdk_abi_version()}.{lib.fdk_abi_revision()}, this package needs "
                          f"{FDK_ABI_VERSION}.{FDK_ABI_REVISION} or a later revision")
    _lib = lib
    return lib


def check(rc: int) -> None:
    """Turn a non-zero return code into an exception carrying fdk_last_error()."""
    if rc == 0:
        return
    msg = load().fdk_last_error().decode("utf-8", "replace")
    if rc in (FDK_ENULL, FDK_EALIGN, FDK_ESHAPE, FDK_EUNSUPPORTED, FDK_EABI):
        raise ValueError(f"fdk: {msg} (code {rc})")
    raise FdkError(rc, msg)
