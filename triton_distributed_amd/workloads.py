"""Seeded synthetic inputs for the five benchmark configurations of the decode path.

Everything is generated on the CPU with a seeded ``torch.Generator`` (so a CPU baseline and the GPU
kernels see identical bits) and moved to the requested device afterwards.  Page tables are drawn
without replacement from a shuffled pool, like the reference's ``PagedKVCache``
(mega_triton_kernel/models/paged_kv_cache.py:46-48).
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import Dict, List, Optional

import torch

E4M3_MAX = 448.0


@dataclass
class DecodeConfig:
    name: str
    seed: int
    batch: int
    q_heads: int
    kv_heads: int
    head_dim: int
    page_size: int
    kv_len: Optional[int] = None         # uniform length, or
    kv_len_range: Optional[tuple] = None  # (lo, hi) inclusive, drawn per sequence
    q_scale: float = 1.0
    kv_dtype: str = "bf16"               # "bf16" | "fp16" | "fp8_e4m3"; a 16-bit cache has q's dtype
    q_dtype: str = "bf16"                # "bf16" | "fp16"
    spare_pages: int = 64
    description: str = ""
    v_head_dim: int = 0                  # values per V / output row where they differ from head_dim (q and K rows)

    @property
    def dv(self) -> int:
        return self.v_head_dim or self.head_dim


CONFIGS: Dict[str, DecodeConfig] = {
    "tiny": DecodeConfig("tiny", 1001, 2, 8, 2, 128, 1, kv_len=512, spare_pages=0,
                         description="B2 8q/2kv D128 N512 P1, block_table = permutation of a 1024-slot pool"),
    "llama3_8b_b32": DecodeConfig("llama3_8b_b32", 1002, 32, 32, 8, 128, 16, kv_len=4096,
                                  description="B32 32q/8kv D128 N4096 P16 bf16 (headline)"),
    "ragged_g8": DecodeConfig("ragged_g8", 1003, 64, 8, 1, 128, 16, kv_len_range=(1, 32768),
                              description="B64 8q/1kv D128 N~U[1,32768] P16 bf16"),
    "long_131k": DecodeConfig("long_131k", 1004, 4, 64, 8, 128, 64, kv_len=131072, q_scale=0.5,
                              description="B4 64q/8kv D128 N131072 P64 bf16, q*0.5"),
    "fp8_70b_b128": DecodeConfig("fp8_70b_b128", 1005, 128, 64, 8, 128, 16, kv_len=8192, kv_dtype="fp8_e4m3",
                                 description="B128 64q/8kv D128 N8192 P16, e4m3 KV with per-kv-head scales"),
}
CONFIG_ORDER: List[str] = ["tiny", "llama3_8b_b32", "ragged_g8", "long_131k", "fp8_70b_b128"]

# Two more shapes for the measurements behind the plan choices (not benchmark configurations): a ragged batch whose
# (sequence, kv head) units would fill the GPU as a single pass, and the headline shape with an fp8 cache.
CONFIGS["ragged_b64_8kv"] = DecodeConfig("ragged_b64_8kv", 1201, 64, 32, 8, 128, 16, kv_len_range=(1, 8192),
                                         description="B64 32q/8kv D128 N~U[1,8192] P16 bf16")
CONFIGS["fp8_8b_b32"] = DecodeConfig("fp8_8b_b32", 1202, 32, 32, 8, 128, 16, kv_len=4096, kv_dtype="fp8_e4m3",
                                     description="B32 32q/8kv D128 N4096 P16, e4m3 KV with per-kv-head scales")

# q / K rows of two segments and V rows of their own length (the reference's BLOCK_HEAD_DIM + BLOCK_DPE and V_DIM,
# flash_decode.py:103-109): the headline shape with 192-value rows, with V rows of 128, and a latent-attention decode
# shape (one shared kv head of 512 + 64 values, 128 q heads, V = 512 values).
CONFIGS["d192_b32"] = DecodeConfig("d192_b32", 1301, 32, 32, 8, 192, 16, kv_len=4096,
                                   description="B32 32q/8kv Dk192 Dv192 N4096 P16 bf16")
CONFIGS["d192v128_b32"] = DecodeConfig("d192v128_b32", 1302, 32, 32, 8, 192, 16, kv_len=4096, v_head_dim=128,
                                       description="B32 32q/8kv Dk192 Dv128 N4096 P16 bf16")
CONFIGS["d576v512_b32"] = DecodeConfig("d576v512_b32", 1303, 32, 128, 1, 576, 64, kv_len=4096, v_head_dim=512,
                                       description="B32 128q/1kv Dk576 Dv512 N4096 P64 bf16")
CONFIGS["d192_fp8_b32"] = DecodeConfig("d192_fp8_b32", 1304, 32, 32, 8, 192, 16, kv_len=4096, kv_dtype="fp8_e4m3",
                                       description="B32 32q/8kv Dk192 Dv192 N4096 P16, e4m3 KV with per-kv-head scales")
CONFIGS["d576v512_fp8_b32"] = DecodeConfig("d576v512_fp8_b32", 1305, 32, 128, 1, 576, 64, kv_len=4096, v_head_dim=512,
                                           kv_dtype="fp8_e4m3",
                                           description="B32 128q/1kv Dk576 Dv512 N4096 P64, e4m3 KV with per-kv-head scales")

# The shape behind the reference's only published figure for this path (README.md:200-202; perf loops of
# test/nvidia/test_sp_decode_attn.py:203-220 and test_decode_attn.py:294-527): batch 1, 96 q / 12 kv heads,
# head_dim 128, fp16, page size 1, local KV 8K ... 128K.
REF_SHAPE_LENGTHS = {"8k": 8192, "16k": 16384, "32k": 32768, "64k": 65536, "128k": 131072}
for _tag, _n in REF_SHAPE_LENGTHS.items():
    CONFIGS[f"ref_b1_96q12kv_p1_{_tag}"] = DecodeConfig(
        f"ref_b1_96q12kv_p1_{_tag}", 1100 + _n // 8192, 1, 96, 12, 128, 1, kv_len=_n, kv_dtype="fp16", q_dtype="fp16",
        description=f"B1 96q/12kv D128 N{_n} P1 fp16 (the reference's published perf shape)")
REF_SHAPE_ORDER: List[str] = [f"ref_b1_96q12kv_p1_{t}" for t in REF_SHAPE_LENGTHS]


@dataclass
class DecodeInputs:
    cfg: DecodeConfig
    q: torch.Tensor
    k_cache: torch.Tensor
    v_cache: torch.Tensor
    block_table: torch.Tensor
    kv_lens: torch.Tensor
    sm_scale: float
    k_scale: Optional[torch.Tensor] = None
    v_scale: Optional[torch.Tensor] = None
    kv_lens_host: List[int] = field(default_factory=list)

    def to(self, device) -> "DecodeInputs":
        mv = lambda t: None if t is None else t.to(device)
        return DecodeInputs(self.cfg, mv(self.q), mv(self.k_cache), mv(self.v_cache), mv(self.block_table),
                            mv(self.kv_lens), self.sm_scale, mv(self.k_scale), mv(self.v_scale),
                            list(self.kv_lens_host))

    def algorithmic_bytes(self) -> int:
        """Bytes a perfect implementation must move: attended K and V rows, q, out, fp32 lse, the
        block_table entries used, kv_lens, and the fp8 scales.  Split partials are not counted."""
        c = self.cfg
        e_kv = 1 if c.kv_dtype == "fp8_e4m3" else 2
        tokens = sum(self.kv_lens_host)
        pages = sum((n + c.page_size - 1) // c.page_size for n in self.kv_lens_host)
        total = tokens * c.kv_heads * (c.head_dim + c.dv) * e_kv
        total += c.batch * c.q_heads * (c.head_dim + c.dv) * 2   # q + out
        total += c.batch * c.q_heads * 4                          # lse
        total += 4 * pages + 4 * c.batch
        if c.kv_dtype == "fp8_e4m3":
            total += 2 * c.kv_heads * 4
        return total

    def flops(self) -> int:
        c = self.cfg
        return 2 * c.q_heads * (c.head_dim + c.dv) * sum(self.kv_lens_host)


def quantize_kv_fp8(cache: torch.Tensor, chunk_pages: int = 4096):
    """Per-kv-head e4m3 quantisation: ``scale[h] = amax_h / 448`` (fp32), ``q = (x / scale[h]) -> e4m3fn``.

    cache ``[pages, P, Hkv, D]`` (any float dtype) -> ``(cache8 float8_e4m3fn, scale [Hkv] fp32)``."""
    n_pages = cache.shape[0]
    amax = torch.zeros(cache.shape[2], dtype=torch.float32, device=cache.device)
    for lo in range(0, n_pages, chunk_pages):
        amax = torch.maximum(amax, cache[lo:lo + chunk_pages].to(torch.float32).abs().amax(dim=(0, 1, 3)))
    scale = amax / E4M3_MAX
    scale = torch.where(scale > 0, scale, torch.ones_like(scale))
    out = torch.empty(cache.shape, dtype=torch.float8_e4m3fn, device=cache.device)
    for lo in range(0, n_pages, chunk_pages):
        out[lo:lo + chunk_pages] = (cache[lo:lo + chunk_pages].to(torch.float32) /
                                    scale[None, None, :, None]).to(torch.float8_e4m3fn)
    return out, scale


def _randn_bf16(shape, gen: torch.Generator, chunk: int = 1 << 24, dtype=torch.bfloat16) -> torch.Tensor:
    """Seeded N(0,1) in bf16 (or ``dtype``), drawn in fp32 pieces to bound peak memory."""
    n = math.prod(shape)
    out = torch.empty(n, dtype=dtype)
    for lo in range(0, n, chunk):
        m = min(chunk, n - lo)
        out[lo:lo + m] = torch.randn(m, generator=gen, dtype=torch.float32).to(dtype)
    return out.view(shape)


def make_inputs(name_or_cfg, device="cpu", poison_tail: bool = False) -> DecodeInputs:
    """Build the tensors of one configuration.

    poison_tail  fill block_table entries past ``ceil(kv_len / P)`` with INT32_MAX / -1 instead of a
                 valid page (they must never be read)."""
    cfg = CONFIGS[name_or_cfg] if isinstance(name_or_cfg, str) else name_or_cfg
    gen = torch.Generator().manual_seed(cfg.seed)
    if cfg.kv_len is not None:
        lens = [cfg.kv_len] * cfg.batch
    else:
        lo, hi = cfg.kv_len_range
        lens = torch.randint(lo, hi + 1, (cfg.batch,), generator=gen).tolist()
    pages_per_seq = [(n + cfg.page_size - 1) // cfg.page_size for n in lens]
    max_pages = max(max(pages_per_seq), 1)
    used = sum(pages_per_seq)
    pool = used + cfg.spare_pages
    perm = torch.randperm(pool, generator=gen).to(torch.int32)
    table = torch.zeros(cfg.batch, max_pages, dtype=torch.int32)
    if poison_tail:
        table[::2] = 2**31 - 1
        table[1::2] = -1
    pos = 0
    for b, n_pg in enumerate(pages_per_seq):
        table[b, :n_pg] = perm[pos:pos + n_pg]
        pos += n_pg
    dt = torch.float16 if cfg.q_dtype == "fp16" else torch.bfloat16
    q = _randn_bf16((cfg.batch, cfg.q_heads, cfg.head_dim), gen, dtype=dt)
    if cfg.q_scale != 1.0:
        q = (q.float() * cfg.q_scale).to(dt)
    cache_shape = (pool, cfg.page_size, cfg.kv_heads, cfg.head_dim)
    k_cache = _randn_bf16(cache_shape, gen, dtype=dt)
    v_cache = _randn_bf16(cache_shape[:3] + (cfg.dv,), gen, dtype=dt)
    k_scale = v_scale = None
    if cfg.kv_dtype == "fp8_e4m3":
        k_cache, k_scale = quantize_kv_fp8(k_cache)
        v_cache, v_scale = quantize_kv_fp8(v_cache)
    inp = DecodeInputs(cfg, q, k_cache, v_cache, table, torch.tensor(lens, dtype=torch.int32),
                       cfg.head_dim ** -0.5, k_scale, v_scale, list(lens))
    return inp.to(device) if str(device) != "cpu" else inp


def scaled_down(cfg: DecodeConfig, batch: Optional[int] = None, kv_len: Optional[int] = None,
                kv_len_range: Optional[tuple] = None) -> DecodeConfig:
    """Same layout, smaller extent (for CPU-sized checks)."""
    return DecodeConfig(cfg.name + "_small", cfg.seed, batch or cfg.batch, cfg.q_heads, cfg.kv_heads, cfg.head_dim,
                        cfg.page_size, kv_len if cfg.kv_len is not None else None,
                        kv_len_range if cfg.kv_len is None else None, cfg.q_scale, cfg.kv_dtype, cfg.q_dtype,
                        min(cfg.spare_pages, 8), cfg.description, cfg.v_head_dim)
