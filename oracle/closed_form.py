"""float64 closed forms and the reference's split / combine recurrences.

TEST INFRASTRUCTURE - see oracle/__init__.py.

What each function follows in the reference (paths relative to the reference root):

attn_fp64          the definition the split kernel implements, without splitting:
                   logits = sm_scale * <q[b,h], K[b,n,h//G]>  (kernels/nvidia/flash_decode.py:208,216),
                   optional soft cap cap*tanh(x/cap) (:218-219, :64-67),
                   out = softmax(logits) @ V (:226-236), lse = max + ln(sum exp) (:238-239).
split_kv_partials  kernels/nvidia/flash_decode.py:193-239 - split ranges
                   [s*ceil(N/S), min((s+1)*ceil(N/S), N)), per-split (o_s, lse_s).  Empty splits are
                   returned as (0, -inf) instead of the reference's 0/0 garbage, which its combine
                   never reads (:428).
combine_partials   kernels/nvidia/flash_decode.py:423-449 - sequential merge over the splits.
combine_ranks      kernels/nvidia/flash_decode.py:512-532 - same merge over ranks, skip rule
                   ``kv_len[rank, b] > 0``.
merge_identity     the textbook form both merges must equal: lse = logsumexp_s(lse_s),
                   out = sum_s softmax(lse)_s * o_s.
"""
from __future__ import annotations

import math
from typing import Optional, Sequence, Tuple, Union

import torch


def _as_len_list(kv_lens) -> list:
    if isinstance(kv_lens, torch.Tensor):
        return [int(x) for x in kv_lens.cpu().tolist()]
    return [int(x) for x in kv_lens]


def gather_kv(cache: torch.Tensor, block_table_row: torch.Tensor, n_kv: int) -> torch.Tensor:
    """Rows 0..n_kv-1 of one sequence: token n lives in page ``block_table[n // P]`` at slot ``n % P``
    (flash_decode.py:203-205).  Returns ``[n_kv, Hkv, D]`` in the cache dtype."""
    page_size = cache.shape[1]
    n_pages = (n_kv + page_size - 1) // page_size
    ids = block_table_row[:n_pages].to(torch.int64).to(cache.device)
    return cache[ids].reshape(n_pages * page_size, cache.shape[2], cache.shape[3])[:n_kv]


def _logits_fp64(q_b, k_b, sm_scale, soft_cap):
    """q_b [Hq, D], k_b [N, Hkv, D] (any float dtype) -> logits [Hkv, G, N] float64."""
    n_q_heads, d = q_b.shape
    n_kv_heads = k_b.shape[1]
    g = n_q_heads // n_kv_heads
    q64 = q_b.to(torch.float64).reshape(n_kv_heads, g, d)
    k64 = k_b.to(torch.float64)
    logits = torch.einsum("hgd,nhd->hgn", q64, k64) * float(sm_scale)
    if soft_cap is not None and soft_cap > 0.0:
        logits = soft_cap * torch.tanh(logits / soft_cap)
    return logits


def attn_fp64(q, k_cache, v_cache, block_table, kv_lens, sm_scale, soft_cap: Optional[float] = None,
              k_scale: Optional[torch.Tensor] = None, v_scale: Optional[torch.Tensor] = None
              ) -> Tuple[torch.Tensor, torch.Tensor]:
    """Unsplit float64 attention on exactly up-cast inputs.

    Returns ``(out [B,Hq,Dv] float64, lse [B,Hq] float64)`` with natural-log lse over the scaled
    (and soft-capped) logits.  ``k_scale`` / ``v_scale`` ([Hkv] float) multiply the up-cast cache
    values (used only for the *exact* fp8 variant; the bf16-rounded dequantisation the fp8 workload
    is defined by lives in oracle/fp8.py).  A sequence with kv_len == 0 gives out = 0, lse = -inf.
    """
    lens = _as_len_list(kv_lens)
    n_seq, n_q_heads, _ = q.shape
    dv = v_cache.shape[-1]
    out = torch.zeros(n_seq, n_q_heads, dv, dtype=torch.float64, device=q.device)
    lse = torch.full((n_seq, n_q_heads), -math.inf, dtype=torch.float64, device=q.device)
    bt = block_table.cpu()
    for b, n_kv in enumerate(lens):
        if n_kv == 0:
            continue
        k_b = gather_kv(k_cache, bt[b], n_kv).to(torch.float64)
        v_b = gather_kv(v_cache, bt[b], n_kv).to(torch.float64)
        if k_scale is not None:
            k_b = k_b * k_scale.to(torch.float64).to(k_b.device)[None, :, None]
        if v_scale is not None:
            v_b = v_b * v_scale.to(torch.float64).to(v_b.device)[None, :, None]
        logits = _logits_fp64(q[b], k_b, sm_scale, soft_cap)               # [Hkv, G, N]
        lse_b = torch.logsumexp(logits, dim=-1)                             # [Hkv, G]
        probs = torch.exp(logits - lse_b[..., None])
        o_b = torch.einsum("hgn,nhd->hgd", probs, v_b)
        out[b] = o_b.reshape(n_q_heads, dv)
        lse[b] = lse_b.reshape(n_q_heads)
    return out, lse


def split_ranges(n_kv: int, num_splits: int) -> list:
    """[(start, end)] per split, flash_decode.py:193-195 (end <= start means empty)."""
    per = (n_kv + num_splits - 1) // num_splits
    return [(per * s, min(per * s + per, n_kv)) for s in range(num_splits)]


def split_kv_partials(q, k_cache, v_cache, block_table, kv_lens, sm_scale, num_splits: int,
                      soft_cap: Optional[float] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per-split normalised partial outputs and lse, float64.

    ``partial_o [B,Hq,S,Dv]``, ``partial_lse [B,Hq,S]``; empty splits hold (0, -inf)."""
    lens = _as_len_list(kv_lens)
    n_seq, n_q_heads, _ = q.shape
    dv = v_cache.shape[-1]
    po = torch.zeros(n_seq, n_q_heads, num_splits, dv, dtype=torch.float64)
    pl = torch.full((n_seq, n_q_heads, num_splits), -math.inf, dtype=torch.float64)
    bt = block_table.cpu()
    for b, n_kv in enumerate(lens):
        if n_kv == 0:
            continue
        k_b = gather_kv(k_cache, bt[b], n_kv)
        v_b = gather_kv(v_cache, bt[b], n_kv).to(torch.float64)
        logits = _logits_fp64(q[b], k_b, sm_scale, soft_cap).reshape(n_q_heads, n_kv)
        n_kv_heads = v_b.shape[1]
        g = n_q_heads // n_kv_heads
        for s, (lo, hi) in enumerate(split_ranges(n_kv, num_splits)):
            if hi <= lo:
                continue
            x = logits[:, lo:hi]
            m = x.max(dim=-1).values                                        # e_max   (:226)
            p = torch.exp(x - m[:, None])                                   # (:228)
            l = p.sum(dim=-1)                                               # e_sum   (:232)
            acc = torch.einsum("hgn,nhd->hgd", p.reshape(n_kv_heads, g, hi - lo), v_b[lo:hi])
            po[b, :, s] = acc.reshape(n_q_heads, dv) / l[:, None]           # (:236)
            pl[b, :, s] = m + torch.log(l)                                  # (:239)
    return po, pl


def combine_partials(partial_o: torch.Tensor, partial_lse: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Sequential merge of flash_decode.py:423-449, in float64, skipping empty (lse = -inf) splits.

    partial_o [..., S, Dv], partial_lse [..., S] -> (out [..., Dv], lse [...])."""
    po = partial_o.to(torch.float64)
    pl = partial_lse.to(torch.float64)
    lead = pl.shape[:-1]
    n_splits = pl.shape[-1]
    e_max = torch.full(lead, -math.inf, dtype=torch.float64)
    e_sum = torch.zeros(lead, dtype=torch.float64)
    acc = torch.zeros(lead + (po.shape[-1],), dtype=torch.float64)
    for s in range(n_splits):
        t = pl[..., s]
        live = torch.isfinite(t)                                            # the range test of :428
        n_max = torch.where(live, torch.maximum(t, e_max), e_max)           # :431
        safe = torch.where(torch.isfinite(n_max), n_max, torch.zeros_like(n_max))
        old = torch.exp(e_max - safe)                                       # :433
        new = torch.where(live, torch.exp(t - safe), torch.zeros_like(t))   # :435
        acc = acc * old[..., None] + new[..., None] * torch.where(live[..., None], po[..., s, :],
                                                                  torch.zeros_like(po[..., s, :]))
        e_sum = e_sum * old + new                                           # :438
        e_max = n_max
    out = acc / e_sum[..., None]                                            # :441-445
    lse = e_max + torch.log(e_sum)                                          # :446-449
    return out, lse


def merge_identity(partial_o: torch.Tensor, partial_lse: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Textbook form: lse = logsumexp_s(lse_s); out = sum_s softmax(lse)_s * o_s (float64)."""
    pl = partial_lse.to(torch.float64)
    po = partial_o.to(torch.float64)
    lse = torch.logsumexp(pl, dim=-1)
    w = torch.softmax(pl, dim=-1)
    po = torch.where(torch.isfinite(pl)[..., None], po, torch.zeros_like(po))
    return (w[..., None] * po).sum(dim=-2), lse


def combine_ranks(all_out: torch.Tensor, all_lse: torch.Tensor, global_kv_lens: torch.Tensor) -> torch.Tensor:
    """Cross-rank merge of flash_decode.py:512-532.

    all_out [R,B,Hq,Dv], all_lse [R,B,Hq], global_kv_lens [R,B]; a rank takes part for batch b only
    if ``global_kv_lens[r, b] > 0`` (:513-515).  Returns out [B,Hq,Dv] float64 (the reference stores
    no lse here)."""
    live = (global_kv_lens > 0)[..., None].to(all_lse.device)               # [R,B,1]
    pl = torch.where(live, all_lse.to(torch.float64), torch.full_like(all_lse, -math.inf, dtype=torch.float64))
    po = all_out.to(torch.float64).permute(1, 2, 0, 3)                      # [B,Hq,R,Dv]
    out, _ = combine_partials(po, pl.permute(1, 2, 0))
    return out
