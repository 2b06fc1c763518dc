"""MI355X-native flash-decode: split-KV paged GQA decode attention + LSE combine (gfx950 HIP kernels).

The entry points live in ``flash_decode`` and are loaded on first use; that loads ``lib/libfdk.so`` and raises
ImportError if the library has not been built (``python -m triton_distributed_amd.build``) or does not match
this package's ABI version.  There is no CPU or eager fallback.  ``triton_distributed_amd.build`` itself
imports without the library.
"""
import importlib

__all__ = [
    "LengthFeedback", "PreparedDecode", "SplitKvPlan", "flash_decode", "flash_decode_bsnh", "get_split_kv_plan", "gqa_fwd_batch_decode",
    "gqa_fwd_batch_decode_aot", "gqa_fwd_batch_decode_intra_rank", "gqa_fwd_batch_decode_intra_rank_aot",
    "gqa_fwd_batch_decode_persistent", "gqa_fwd_batch_decode_persistent_aot",
    "inter_rank_combine", "pack_out_lse", "prepare_decode", "probe_linear_read", "qk_norm_rope_update_kvcache",
    "unpack_out_lse",
]


_LAYERS = ("SpGQAFlashDecodeAttention",)
_HOST_ONLY = {"PagedKVCache": ".paged_kv_cache", "alloc_kv_pools": ".paged_kv_cache"}      # importable without the library


def _bind():
    """Import the entry points (loads libfdk.so; raises if it is missing) and bind them on the package: the
    function ``flash_decode`` takes the place of the submodule attribute of the same name that the import sets."""
    mod = importlib.import_module(".flash_decode", __name__)
    globals().update({n: getattr(mod, n) for n in __all__})


def __getattr__(name):
    if name in _HOST_ONLY:
        globals()[name] = getattr(importlib.import_module(_HOST_ONLY[name], __name__), name)
        return globals()[name]
    if name in _LAYERS:
        _bind()
        mod = importlib.import_module(".sp_flash_decode_layer", __name__)
        _bind()                                   # the layer module imports the submodule again
        globals()[name] = getattr(mod, name)
        return globals()[name]
    if name in __all__:
        _bind()
        return globals()[name]
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")


def __dir__():
    return sorted(list(globals()) + __all__ + list(_LAYERS) + list(_HOST_ONLY))
