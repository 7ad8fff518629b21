"""Sequence-parallel GQA flash-decode attention layer for one MI355X.

Keeps the constructor and ``forward`` of the reference's SpGQAFlashDecodeAttention
(layers/nvidia/sp_flash_decode_layer.py:43-184): every rank holds a shard of the KV sequence, decodes over
its shard keeping the LSE, the (out, LSE) pairs of all ranks are gathered and merged by LSE. With one GPU
the gather has nobody to talk to: the partial results of the other ranks are passed to ``forward`` as
``peer_partials`` and take their rank's place in the gathered tensor.
"""
import torch

from triton_dist import _lib
from triton_dist.kernels.amd.flash_decode import (gqa_fwd_batch_decode_intra_rank,
                                                   gqa_fwd_batch_decode_inter_rank_combine)


class SpGQAFlashDecodeAttention(torch.nn.Module):

    def __init__(self, rank, node, num_ranks, num_nodes, num_q_heads, num_kv_heads, q_head_dim, v_head_dim, page_size=1,
                 scale=1, soft_cap=0, max_allowed_batch=1, thrink_buffer_threshold=500, stages=20):
        """Same arguments as the reference's constructor (:45-47, including its spelling of
        ``thrink_buffer_threshold``). ``node``, ``num_nodes``, ``stages`` and the threshold describe the all-gather
        buffers of the multi-GPU layer; here they are recorded and otherwise unused, because the gather is the
        caller handing in ``peer_partials``."""
        super().__init__()
        # where this shard sits among the sequence-parallel ranks
        self.rank, self.num_ranks = rank, num_ranks
        self.node, self.num_nodes = node, num_nodes
        # attention geometry
        self.num_q_heads, self.num_kv_heads = num_q_heads, num_kv_heads
        self.q_head_dim, self.v_head_dim = q_head_dim, v_head_dim
        self.page_size = page_size
        self.scale, self.soft_cap = scale, soft_cap
        self.kv_split = 32                    # splits of the local shard (the reference fixes 32, :59)
        self.max_allowed_batch = max_allowed_batch
        # the fused decode keeps its arrival counters per layer, so that two layers may run on two streams
        self.workspace = None
        self.stages = stages
        self.shrink_buffer_threshold = thrink_buffer_threshold

    def forward(self, q, k_cache, v_cache, global_kv_lens, block_table, peer_partials=None):
        """
        q: each rank has the same q
        k_cache / v_cache: this rank's shard of the cache
        global_kv_lens: int32 [num_ranks, batch], every rank's shard length
        block_table: this rank's page table
        peer_partials: (out [num_ranks, batch, Hq, Dv], lse fp32 [num_ranks, batch, Hq]) holding the other
            ranks' results (row ``rank`` is overwritten with this rank's own); required when num_ranks > 1.
        """
        batch = q.shape[0]
        assert global_kv_lens.shape[0] == self.num_ranks
        assert global_kv_lens.shape[1] == batch
        assert batch <= self.max_allowed_batch, f"Only support {self.max_allowed_batch} queries decode now"
        if self.workspace is None or self.workspace.device != q.device:
            n = _lib.load().tdist_decode_fused_counters(self.max_allowed_batch, self.num_q_heads, self.num_kv_heads)
            self.workspace = torch.zeros(max(int(n), 1), dtype=torch.int32, device=q.device)
        _, out32, lse32 = gqa_fwd_batch_decode_intra_rank(q, k_cache, v_cache, None, [1] * batch,
                                                          global_kv_lens[self.rank], block_table, self.scale,
                                                          soft_cap=self.soft_cap, kv_split=self.kv_split,
                                                          return_lse=True, counters=self.workspace)
        if self.num_ranks == 1:
            all_out, all_lse = out32.unsqueeze(0), lse32.unsqueeze(0)
        else:
            if peer_partials is None:
                raise RuntimeError("one GPU holds a single rank: pass the other ranks' (out, lse) as peer_partials")
            all_out, all_lse = peer_partials
            assert all_out.shape == (self.num_ranks, batch, self.num_q_heads, self.v_head_dim)
            assert all_lse.shape == (self.num_ranks, batch, self.num_q_heads)
            # the local copy into the gather buffer (reference :133-135)
            all_out[self.rank].copy_(out32)
            all_lse[self.rank].copy_(lse32)
        return gqa_fwd_batch_decode_inter_rank_combine(all_out, all_lse, global_kv_lens, out_dtype=q.dtype)
