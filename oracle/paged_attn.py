"""Torch restatement of the reference's torch implementation of paged decode attention.

TEST INFRASTRUCTURE - see oracle/__init__.py.  Follows, step by step, the function the
reference's decode tests compare their kernels with:

    python/triton_dist/test/nvidia/test_decode_attn.py:67-117   (``ref_paged_attn``)

with one deliberate difference: the reference scales a *view* of the caller's query in place
(``q *= scale``, :87-88); this restatement never writes to its inputs (the mega-kernel copy
of the same function does ``q = q * scale``, mega_triton_kernel/test/torch_impl_utils.py:78).

Only decode (one query token per sequence) is restated: with query_len == 1 the causal mask
of :102-103,110 masks nothing, and the sliding-window branch (:104-107) is not on the path.
"""
from __future__ import annotations

from typing import Optional, Sequence, Union

import torch


def ref_paged_attn(
    query: torch.Tensor,          # [B, Hq, D]  (one token per sequence)
    key_cache: torch.Tensor,      # [num_pages, P, Hkv, D]
    value_cache: torch.Tensor,    # [num_pages, P, Hkv, Dv]
    kv_lens: Union[Sequence[int], torch.Tensor],
    block_tables: torch.Tensor,   # [B, max_pages] int32
    scale: float,
    soft_cap: Optional[float] = None,
) -> torch.Tensor:
    """Returns ``out [B, Hq, Dv]`` in the value dtype, like test_decode_attn.py:67-117."""
    if isinstance(kv_lens, torch.Tensor):
        kv_lens = [int(x) for x in kv_lens.cpu().tolist()]
    n_seq, n_q_heads, _ = query.shape
    _, page_size, n_kv_heads, head_size = key_cache.shape          # :80
    tables = block_tables.cpu().numpy()                               # :79
    dev = key_cache.device
    rows = []
    for i in range(n_seq):
        n_kv = kv_lens[i]
        q_i = query[i:i + 1] * scale                                   # :87-88, in the input dtype
        n_pages = (n_kv + page_size - 1) // page_size                 # :90
        page_ids = torch.as_tensor(tables[i, :n_pages].astype("int64"), device=dev)   # :91
        k_i = key_cache[page_ids].reshape(-1, n_kv_heads, head_size)[:n_kv]            # :93-94
        v_i = value_cache[page_ids].reshape(-1, n_kv_heads, value_cache.shape[-1])[:n_kv]  # :95-96
        if n_q_heads != n_kv_heads:                                    # :98-100
            rep = n_q_heads // n_kv_heads
            k_i = torch.repeat_interleave(k_i, rep, dim=1)
            v_i = torch.repeat_interleave(v_i, rep, dim=1)
        logits = torch.einsum("qhd,khd->hqk", q_i, k_i).float()       # :101, input dtype then fp32
        if soft_cap is not None and soft_cap > 0.0:                    # :108-109
            logits = soft_cap * torch.tanh(logits / soft_cap)
        probs = torch.softmax(logits, dim=-1).to(v_i.dtype)            # :111
        rows.append(torch.einsum("hqk,khd->qhd", probs, v_i))         # :112
    return torch.cat(rows, dim=0)                                      # :117
