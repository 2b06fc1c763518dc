"""MI355X-native flash-decode: split-KV paged GQA decode attention + LSE combine (gfx950 HIP kernels).

Importing this package loads ``lib/libfdk.so``; it raises ImportError if the library has not been built
(``python -m triton_distributed_amd.build``).  There is no CPU or eager fallback.
"""
from .flash_decode import (  # noqa: F401
    PreparedDecode,
    SplitKvPlan,
    flash_decode,
    get_split_kv_plan,
    gqa_fwd_batch_decode,
    gqa_fwd_batch_decode_aot,
    gqa_fwd_batch_decode_intra_rank,
    gqa_fwd_batch_decode_intra_rank_aot,
    inter_rank_combine,
    pack_out_lse,
    prepare_decode,
    unpack_out_lse,
)

__all__ = [
    "PreparedDecode", "SplitKvPlan", "flash_decode", "get_split_kv_plan", "gqa_fwd_batch_decode",
    "gqa_fwd_batch_decode_aot", "gqa_fwd_batch_decode_intra_rank", "gqa_fwd_batch_decode_intra_rank_aot",
    "inter_rank_combine", "pack_out_lse", "prepare_decode", "unpack_out_lse",
]
