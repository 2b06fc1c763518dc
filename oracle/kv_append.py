"""Oracle of the step before the decode path: per-head RMSNorm, rotary embedding and the paged KV-cache append.

TEST INFRASTRUCTURE - see oracle/__init__.py.

Restates ``rmsnorm_rope_update_kv_cache_task_compute``
(python/triton_dist/mega_triton_kernel/kernels/norm.py:32-190; host side
``ModelBuilder.make_qk_norm_rope_update_kvcache``, models/model_builder.py:341-379), operation by operation:

  * one head row of ``qkv [B, T, Hq + 2 Hkv, D]`` at a time; q heads first, then k heads, then v heads (:84-85, :120);
  * ``kv_lens`` already includes the T new tokens: token t of sequence b sits at position
    ``pos = kv_lens[b] - T + t`` (:100-102);
  * q and k rows: ``rms = rsqrt(mean(x^2) + eps)`` in fp32, ``y = w * (x * rms)`` in fp32 (:131-138),
    halves ``y0 = y[:D/2]``, ``y1 = y[D/2:]`` rounded to bf16 (:153-169), then
    ``out0 = y0 * cos - y1 * sin``, ``out1 = y1 * cos + y0 * sin`` in fp32 with the first D/2 columns of row ``pos``
    of the fp32 cos / sin tables (:143-151, :170-171), stored as bf16 (:172-174, :183-188);
  * v rows are copied (:104-117).

Deviations, both deliberate:
  * cache slot.  The reference addresses ``block_entry_id + pos % PAGE_SIZE`` (:115, :183), which equals the paged
    slot ``block_entry_id * PAGE_SIZE + pos % PAGE_SIZE`` only for PAGE_SIZE = 1 (its models run with 1).  The slot
    here is the one the decode kernels read (flash_decode.py:203-205).
  * fp8 caches do not exist in the reference.  Quantise-on-write is defined the way the fp8 workload quantises a
    finished cache: ``clamp(x_bf16 / scale[h], -448, 448) -> e4m3fn`` (round to nearest even), x being the bf16 value
    a 16-bit cache would have received.

Pinning (tests/test_oracle_kv_append.py): against an independent float64 route (numpy ``linalg.norm`` RMS, rotation
as complex multiplication) at the reference test's own tolerance (atol = rtol = 1e-2, test_qk_norm_rope.py:115-116);
position 0 is the identity rotation; rotations preserve the norm of every (i, i + D/2) pair; v rows and every
cache row that is not a target are bit-identical; the fp8 bytes equal ``torch.float8_e4m3fn`` casts of the same
quotients.  The reference's own oracle for this operator is flashinfer (``rmsnorm``,
``apply_rope_with_cos_sin_cache_inplace``; test/torch_impl_utils.py:41-54), a third-party package that is not
in this image, and the reference holds no stored vectors for it: beyond the 1e-2 tolerance the bf16 rounding points
of its Triton kernel are "parity unpinned".
"""
from __future__ import annotations

from typing import Optional, Sequence

import torch

E4M3_MAX = 448.0


def cos_sin_tables(head_dim: int, max_positions: int, rope_theta: float = 1000000.0):
    """fp32 ``cos, sin [max_positions, D]`` laid out like the reference's tables (halves repeated,
    test/torch_impl_utils.py:30-38).  Only the first D/2 columns are ever read."""
    inv_freq = 1.0 / (rope_theta ** (torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim))
    t = torch.arange(max_positions, dtype=torch.float32)
    freqs = torch.outer(t, inv_freq)
    emb = torch.cat((freqs, freqs), dim=-1)
    return emb.cos().contiguous(), emb.sin().contiguous()


def norm_rope_row(x: torch.Tensor, w: torch.Tensor, eps: float, cos_row: torch.Tensor, sin_row: torch.Tensor):
    """One head row ``x [D]`` (16-bit) -> normalised, rotated row in x's dtype (norm.py:127-171)."""
    d = x.shape[-1]
    a = x.to(torch.float32)
    rms = torch.rsqrt((a * a).sum() / d + eps)
    y = w.to(torch.float32) * (a * rms)
    y0 = y[: d // 2].to(x.dtype).to(torch.float32)
    y1 = y[d // 2:].to(x.dtype).to(torch.float32)
    c, s = cos_row[: d // 2].to(torch.float32), sin_row[: d // 2].to(torch.float32)
    return torch.cat((y0 * c - y1 * s, y1 * c + y0 * s)).to(x.dtype)


def quantize_row(x: torch.Tensor, scale: float) -> torch.Tensor:
    """Saturating e4m3fn quantisation of a 16-bit row with one fp32 scale."""
    q = (x.to(torch.float32) / torch.tensor(scale, dtype=torch.float32)).clamp(-E4M3_MAX, E4M3_MAX)
    return q.to(torch.float8_e4m3fn)


def kv_append(qkv: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor,
              kv_lens: Sequence[int], q_weight: torch.Tensor, k_weight: torch.Tensor, cos: torch.Tensor,
              sin: torch.Tensor, num_q_heads: int, q_eps: float = 1e-6, k_eps: float = 1e-6,
              k_scale: Optional[torch.Tensor] = None, v_scale: Optional[torch.Tensor] = None):
    """Apply the operator on CPU tensors.  Returns ``q_out [B, T, Hq, D]``; the caches are updated in place.

    qkv [B, T, Hq + 2 Hkv, D] bf16/fp16; caches [pages, P, Hkv, D] in qkv's dtype or float8_e4m3fn (then with
    ``k_scale, v_scale [Hkv]``); cos, sin [S, D] or [1, S, D] fp32, indexed by absolute position."""
    b_, t_, heads, d = qkv.shape
    hkv = (heads - num_q_heads) // 2
    page = k_cache.shape[1]
    cos2, sin2 = cos.reshape(-1, cos.shape[-1]), sin.reshape(-1, sin.shape[-1])
    q_out = torch.empty((b_, t_, num_q_heads, d), dtype=qkv.dtype)
    fp8 = k_cache.dtype == torch.float8_e4m3fn
    for b in range(b_):
        for t in range(t_):
            pos = int(kv_lens[b]) - t_ + t
            if pos < 0:
                raise ValueError("kv_lens must already include the new tokens")
            slot = int(block_table[b, pos // page]) * page + pos % page
            pg, off = divmod(slot, page)
            for h in range(num_q_heads):
                q_out[b, t, h] = norm_rope_row(qkv[b, t, h], q_weight, q_eps, cos2[pos], sin2[pos])
            for h in range(hkv):
                k_row = norm_rope_row(qkv[b, t, num_q_heads + h], k_weight, k_eps, cos2[pos], sin2[pos])
                v_row = qkv[b, t, num_q_heads + hkv + h]
                if fp8:
                    k_cache[pg, off, h] = quantize_row(k_row, float(k_scale[h]))
                    v_cache[pg, off, h] = quantize_row(v_row, float(v_scale[h]))
                else:
                    k_cache[pg, off, h] = k_row
                    v_cache[pg, off, h] = v_row
    return q_out


def norm_rope_fp64(x: torch.Tensor, w: torch.Tensor, eps: float, pos: int, rope_theta: float = 1000000.0):
    """Independent float64 route for one head row: RMS through ``numpy.linalg.norm``, the rotation of the pair
    (x[i], x[i + D/2]) by the angle ``pos * theta^(-2i/D)`` as one complex multiplication."""
    import numpy as np
    xd = x.to(torch.float64).numpy()
    d = xd.shape[-1]
    rms = np.linalg.norm(xd) / np.sqrt(d)
    y = w.to(torch.float64).numpy() * xd / np.sqrt(rms * rms + eps)
    z = y[: d // 2] + 1j * y[d // 2:]
    ang = pos * rope_theta ** (-np.arange(0, d, 2, dtype=np.float64) / d)
    z = z * np.exp(1j * ang)
    return torch.from_numpy(np.concatenate((z.real, z.imag)))
