"""Host mirror of the reference's sequence-parallel decode layer, for one GPU's share.

``SpGQAFlashDecodeAttention`` has the constructor and ``forward`` signature of the reference class of the same name
(python/triton_dist/layers/nvidia/sp_flash_decode_layer.py:44-185).  Its three steps are

  1. local decode of this rank's KV shard into the packed ``[B, Hq, D+1]`` block (:100-110)   - HIP, this package
  2. all-gather of the blocks of all ranks into ``[R, B, Hq, D+1]`` (:111-145)                 - NOT built here
  3. cross-rank log-sum-exp merge (:147-183)                                                   - HIP, this package

Step 2 is the reference's low-latency all-gather over NVSHMEM; this package runs on one GPU and contains no
collective.  ``forward`` therefore works as is for ``num_ranks == 1``; for more ranks the caller passes the
exchange as ``all_gather`` (any callable ``[B, Hq, D+1] -> [R, B, Hq, D+1]``, e.g. a wrapper around
``torch.distributed.all_gather_into_tensor``).  ``local_decode`` and ``combine`` expose steps 1 and 3 alone.
"""
from __future__ import annotations

from typing import Callable, Optional

import torch

from .flash_decode import LengthFeedback, gqa_fwd_batch_decode_intra_rank, inter_rank_combine


class SpGQAFlashDecodeAttention(torch.nn.Module):

    def __init__(self, rank, node, num_ranks, num_nodes, num_q_heads, num_kv_heads, q_head_dim, v_head_dim, page_size=1,
                 scale=1, soft_cap=0, max_allowed_batch=1, thrink_buffer_threshold=500, stages=20,
                 all_gather: Optional[Callable[[torch.Tensor], torch.Tensor]] = None, length_feedback: bool = True):
        super().__init__()
        # (which pairs are built - 64, 128, 256 alike; 192 with 192 or 128; 576 with 512 - is for the library to say, at the
        # first decode)
        if num_ranks > 1 and all_gather is None:
            raise ValueError("num_ranks > 1 needs an all_gather callable: this package contains no collective")
        self.rank, self.node, self.num_ranks, self.num_nodes = rank, node, num_ranks, num_nodes
        self.workspace = None
        self.num_q_heads, self.num_kv_heads = num_q_heads, num_kv_heads
        self.q_head_dim, self.v_head_dim = q_head_dim, v_head_dim
        self.page_size = page_size
        self.soft_cap = soft_cap
        self.scale = scale
        self.kv_split = -1            # the reference fixes 32 (:64); here the plan follows the shape
        self.max_allowed_batch = max_allowed_batch
        self.stages = stages
        self.all_gather = all_gather
        # forward() gets the lengths only as a GPU tensor.  Every local decode leaves their bounds in this block and
        # the next one plans with them (alike lengths that fill the GPU: one pass, no combine launch) - without a
        # synchronisation and without changing results beyond the rounding of a different split; False: every call
        # plans for unknown lengths.  Created at the first forward on a GPU.
        self._want_feedback = bool(length_feedback)
        self._feedback: Optional[LengthFeedback] = None

    def finalize(self):
        """The reference frees its symmetric buffers here (:78-80); nothing is held by this class."""

    def local_decode(self, q, k_cache, v_cache, global_kv_lens, block_table, output_combine=None):
        """Step 1: this rank's packed ``[B, Hq, D+1]`` block (attention output normalised locally, then lse)."""
        batch = q.shape[0]
        assert global_kv_lens.shape[0] == self.num_ranks
        assert global_kv_lens.shape[1] == batch
        assert batch <= self.max_allowed_batch, f"Only support {self.max_allowed_batch} queries decode now"
        if self._want_feedback and self._feedback is None and q.is_cuda and not torch.cuda.is_current_stream_capturing():
            with torch.cuda.device(q.device):
                self._feedback = LengthFeedback()           # (pinned host memory: not allocated under graph capture)
        return gqa_fwd_batch_decode_intra_rank(q, k_cache, v_cache, self.workspace, [1] * batch,
                                               global_kv_lens[self.rank], block_table, self.scale,
                                               soft_cap=self.soft_cap, output_combine=output_combine,
                                               kv_split=self.kv_split, length_feedback=self._feedback)

    def combine(self, all_ranks_output_combine, global_kv_lens, final_output=None):
        """Step 3: ``[R, B, Hq, D+1]`` blocks -> ``[B, Hq, D]``; ranks with ``kv_len == 0`` are skipped (:513-515)."""
        return inter_rank_combine(all_ranks_output_combine, global_kv_lens.contiguous(), final_output)

    def forward(self, q, k_cache, v_cache, global_kv_lens, block_table):
        """
        q: each rank has the same q
        k_cache, v_cache: this rank's shard of the paged cache
        global_kv_lens: [num_ranks, batch] lengths of every rank's shard
        block_table: this rank's table
        """
        output_combine = self.local_decode(q, k_cache, v_cache, global_kv_lens, block_table)
        if self.num_ranks == 1:
            gathered = output_combine[None]
        else:
            gathered = self.all_gather(output_combine)
            if tuple(gathered.shape) != (self.num_ranks, *output_combine.shape):
                raise ValueError(f"all_gather returned {tuple(gathered.shape)}, expected "
                                 f"{(self.num_ranks, *output_combine.shape)}")
        return self.combine(gathered, global_kv_lens)
