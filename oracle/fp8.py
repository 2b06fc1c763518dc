"""OCP fp8 e4m3fn decode and the per-kv-head dequantisation of the fp8 KV-cache workload.

TEST INFRASTRUCTURE - see oracle/__init__.py.

The reference has no fp8 KV path (kernels/nvidia/flash_decode.py:208 only casts the cache to the
query dtype, without a scale), so this part is defined by the workload statement itself:
per kv head, ``scale = amax / 448`` in fp32, ``K8 = (K / scale) -> e4m3fn``; the reference
behaviour to match is "dequantise to bf16, then run the same decode":
``K_deq = (K8.float() * scale).to(bf16)``.
"""
from __future__ import annotations

import math

import numpy as np
import torch

E4M3_MAX = 448.0


def e4m3fn_value(byte: int) -> float:
    """Value of one OCP e4m3fn byte from the bit formula: 1 sign, 4 exponent (bias 7), 3 mantissa;
    no infinities; S.1111.111 is NaN; exponent 0 is subnormal (2^-6 * m/8)."""
    s = -1.0 if byte & 0x80 else 1.0
    e = (byte >> 3) & 0xF
    m = byte & 0x7
    if e == 0xF and m == 0x7:
        return math.nan
    if e == 0:
        return s * (m / 8.0) * 2.0 ** -6
    return s * (1.0 + m / 8.0) * 2.0 ** (e - 7)


def e4m3fn_table() -> np.ndarray:
    """All 256 byte values -> float32."""
    return np.array([e4m3fn_value(b) for b in range(256)], dtype=np.float32)


def dequant_per_head(cache8: torch.Tensor, scale: torch.Tensor, dtype=torch.bfloat16) -> torch.Tensor:
    """``(cache8.float() * scale[h]).to(dtype)`` for a cache ``[pages, P, Hkv, D]`` and ``scale [Hkv]``."""
    return (cache8.to(torch.float32) * scale.to(torch.float32).to(cache8.device)[None, None, :, None]).to(dtype)


def quant_per_head(cache: torch.Tensor):
    """``scale[h] = amax_h / 448`` (fp32), ``cache8 = (cache / scale[h]) -> float8_e4m3fn``."""
    amax = cache.to(torch.float32).abs().amax(dim=(0, 1, 3))
    scale = (amax / E4M3_MAX).to(torch.float32)
    scale = torch.where(scale > 0, scale, torch.ones_like(scale))
    q = (cache.to(torch.float32) / scale[None, None, :, None]).to(torch.float8_e4m3fn)
    return q, scale
