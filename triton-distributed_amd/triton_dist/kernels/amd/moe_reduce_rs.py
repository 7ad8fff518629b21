"""MoE tensor-parallel second half on one MI355X: grouped GEMM over the sorted (token, k) rows, top-k weighted
reduction to tokens, reduce-scatter of the ranks' partial results.

Keeps the interface of the reference's kernels/nvidia/moe_reduce_rs.py: ``select_experts`` (:180-197),
``MoEAgScatterGroupGemmPrecomputeContext`` / ``precompute_context_helper`` (:71-237), ``create_moe_rs_context``
(:280-361) and ``moe_reduce_rs`` (:889-...). The three device steps are the library's grouped GEMM
(kernel_producer_group_gemm_tp_scatter_input, :365-468), the weighted combine (the top-k sum of
kernel_consumer_topk_reduce_scatter_intra_node, :471-546) and the ordered slice reduction (kernel_consumer_reduce,
:549-587). With one GPU the other ranks' router logits and partial results are handed to the context
(``peer_router_logits=``, ``ctx.set_peer_partials``)."""
import dataclasses
from typing import Dict, List, Optional

import torch

from triton_dist import _lib
from triton_dist.kernels.amd.allgather_group_gemm import group_gemm_gated, sort_topk_ids_align_block_size
from triton_dist.kernels.amd.low_latency_all_to_all import moe_weighted_combine


def select_experts(pg, num_ranks, topk, input_dtype, device, router_logits, peer_router_logits=None, rank=0):
    """softmax + top-k of every rank's router logits, in rank order (reference :180-197; its all-gather is the
    concatenation of ``router_logits`` [tokens_per_rank, E] with the peers' logits, a dict rank -> tensor).
    Returns (full_topk_ids int32 [M, topk], full_topk_weight input_dtype [M, topk])."""
    parts = []
    for r in range(num_ranks):
        if r == rank:
            parts.append(router_logits)
        else:
            if peer_router_logits is None or r not in peer_router_logits:
                raise RuntimeError("one GPU holds a single rank: pass the other ranks' router logits (missing rank %d)" % r)
            parts.append(peer_router_logits[r].to(device))
    score = torch.softmax(torch.cat(parts, dim=0), dim=-1)
    weight, ids = torch.topk(score, topk)
    return ids.to(torch.int32).contiguous(), weight.to(input_dtype).contiguous()


@dataclasses.dataclass
class MoEAgScatterGroupGemmPrecomputeContext:
    full_topk_weight: Optional[torch.Tensor] = None
    full_topk_ids: Optional[torch.Tensor] = None
    full_sorted_token_ids: Optional[torch.Tensor] = None
    full_token_expert_ids: Optional[torch.Tensor] = None
    block_wait_barriers: Optional[torch.Tensor] = None
    rank_block_num: Optional[torch.Tensor] = None
    full_num_tokens_post_padded_list: Optional[torch.Tensor] = None
    EM: int = 0
    full_numel: int = 0
    TOP_K: int = 0
    BLOCK_M: int = 0
    num_tokens_per_rank: int = 0


def precompute_context_helper(pg, num_ranks, topk, num_tokens_per_rank, num_experts, input_dtype, device, router_logits,
                              BLOCK_M=128, peer_router_logits=None, rank=0):
    """Routing and its align / sort, once per routing (reference :200-237)."""
    ctx = MoEAgScatterGroupGemmPrecomputeContext()
    ctx.full_topk_ids, ctx.full_topk_weight = select_experts(pg, num_ranks, topk, input_dtype, device, router_logits,
                                                             peer_router_logits, rank)
    (ctx.full_sorted_token_ids, ctx.full_token_expert_ids, ctx.block_wait_barriers, ctx.rank_block_num,
     ctx.full_num_tokens_post_padded_list) = sort_topk_ids_align_block_size(ctx.full_topk_ids, num_experts, num_ranks,
                                                                            num_tokens_per_rank, BLOCK_M)
    ctx.EM = int(ctx.full_num_tokens_post_padded_list.cpu().tolist()[0])
    ctx.full_numel = ctx.full_topk_ids.numel()
    ctx.TOP_K, ctx.BLOCK_M, ctx.num_tokens_per_rank = topk, BLOCK_M, num_tokens_per_rank
    return ctx


@dataclasses.dataclass
class MoEReduceRSContext:
    precompute_ctx: MoEAgScatterGroupGemmPrecomputeContext
    rank: int
    world_size: int
    rs_buffers: List[Optional[torch.Tensor]]   # [max_token_num, hidden]: row block r holds rank r's partial of this rank's tokens
    final_output_buffer: torch.Tensor          # [max_token_num * topk, hidden]: the grouped GEMM's rows
    topk_weight_f32: torch.Tensor              # the routing weights as the combine kernel takes them
    identity_index: torch.Tensor               # int32 [M, topk]: row t*topk + k
    output_dtype: torch.dtype = torch.bfloat16
    weight_nk: Optional[torch.Tensor] = None
    weight_key: Optional[tuple] = None
    sk_workspace: Optional[torch.Tensor] = None   # the context's GEMM workspace; None = off

    def set_peer_partials(self, partials):
        """``partials``: dict rank -> [tokens_per_rank, hidden]: what rank r computed (over its share of the intermediate
        dimension) for the tokens this rank owns."""
        if not isinstance(partials, dict):
            partials = {r: t for r, t in enumerate(partials) if t is not None}
        buf = self.rs_buffers[self.rank]
        for r, t in partials.items():
            if r != self.rank:
                buf[r * t.shape[0]:(r + 1) * t.shape[0], :t.shape[1]].copy_(t)


def create_moe_rs_context(pg, local_rank, world_size, local_world_size, max_token_num, hidden_dim, num_experts, topk,
                          input_dtype, output_dtype, device, moe_block_size, router_logits, peer_router_logits=None, split_k=True):
    """reference :280-361. ``pg`` may be None on one GPU (``local_rank`` is then the rank)."""
    if not torch.cuda.is_available():
        raise RuntimeError("create_moe_rs_context needs a GPU")
    _lib.check(_lib.load().tdist_init())
    if output_dtype != torch.bfloat16:
        raise NotImplementedError("the top-k reduction writes bf16 (reference: the input dtype, fp16 in its test)")
    rank = local_rank if pg is None else pg.rank()
    num_tokens_per_rank = router_logits.shape[0]
    assert num_tokens_per_rank * world_size <= max_token_num and max_token_num % world_size == 0
    pre = precompute_context_helper(pg, world_size, topk, num_tokens_per_rank, num_experts, input_dtype, device,
                                    router_logits, BLOCK_M=moe_block_size, peer_router_logits=peer_router_logits, rank=rank)
    M = num_tokens_per_rank * world_size
    rs_buffers: List[Optional[torch.Tensor]] = [None] * world_size
    rs_buffers[rank] = torch.zeros([max_token_num, hidden_dim], dtype=output_dtype, device=device)
    return MoEReduceRSContext(
        precompute_ctx=pre, rank=rank, world_size=world_size, rs_buffers=rs_buffers,
        final_output_buffer=torch.zeros((max_token_num * topk, hidden_dim), dtype=output_dtype, device=device),
        topk_weight_f32=pre.full_topk_weight.float().contiguous(),
        identity_index=torch.arange(M * topk, dtype=torch.int32, device=device).view(M, topk), output_dtype=output_dtype,
        sk_workspace=_lib.new_split_k_workspace(device) if split_k else None)


def _weight_nk(ctx, b):
    if b.stride(1) == 1:
        return b.transpose(1, 2)
    key = (b.data_ptr(), tuple(b.shape), b._version)
    if ctx.weight_key != key:
        ctx.weight_nk = b.transpose(1, 2).contiguous()
        ctx.weight_key = key
    return ctx.weight_nk


def moe_reduce_rs(rank, world_size, local_world_size, a, b, ctx, dump_ir=False, debug_sync=False, do_initial_sync=True,
                  do_final_sync=True):
    """a [M * topk, K_per_rank] intermediate states, row t*topk + k for token t's k-th expert; b [E, K_per_rank, hidden].
    Returns [M // world_size, hidden]: sum over k of weight[t,k] * (a[t*topk+k] @ b[expert]) for this rank's tokens,
    summed with the other ranks' partial results (reference :889-...; golden test/nvidia/test_moe_reduce_rs.py:103-133).
    The synchronisation arguments are accepted and unused: one stream runs the three steps in order."""
    _lib.require_cuda(a, b)
    pre = ctx.precompute_ctx
    M, topk = pre.full_topk_ids.shape
    assert a.shape[0] == M * topk and a.dtype == b.dtype and a.shape[1] == b.shape[1]
    hidden = b.shape[2]
    out = ctx.final_output_buffer[:M * topk, :hidden]
    flags = None
    # every sorted id names its own row of ``a`` (topk = 1 for the gather), no flag to wait for: the rows are local
    group_gemm_gated(a, None, 0, _weight_nk(ctx, b), out, pre.full_sorted_token_ids, pre.full_token_expert_ids,
                     pre.block_wait_barriers, pre.full_num_tokens_post_padded_list, pre.BLOCK_M, pre.full_numel, 1,
                     pre.num_tokens_per_rank * topk, 0, flags, rank, sk_workspace=ctx.sk_workspace)
    y = moe_weighted_combine(None, out, None, ctx.identity_index, ctx.topk_weight_f32, from_slots=False)   # [M, hidden]
    m_per = M // world_size
    buf = ctx.rs_buffers[ctx.rank]
    buf[rank * m_per:(rank + 1) * m_per, :hidden].copy_(y[rank * m_per:(rank + 1) * m_per])
    result = torch.empty((m_per, hidden), dtype=ctx.output_dtype, device=a.device)
    slab = buf[:M, :hidden]
    if not slab.is_contiguous():
        raise NotImplementedError("hidden must equal the context's hidden_dim")
    _lib.call("tdist_reduce_slices", slab.data_ptr(), m_per * hidden, world_size, (rank + 1) % world_size, m_per * hidden,
              result.data_ptr(), _lib.dtype_code(ctx.output_dtype), _lib.stream_ptr())
    return result
