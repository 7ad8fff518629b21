"""MoE tensor-parallel AG + grouped GEMM on one MI355X: the align / sort of the routing and the chunk-gated grouped
GEMM that consumes it.

Keeps the interface of the reference's kernels/nvidia/allgather_group_gemm.py: ``sort_topk_ids_align_block_size``
(:54-135; its device work is the C++ op moe_ag_scatter_align_block_size, csrc/lib/moe_utils.cu:60-186),
``MoE_AllGatherGroupGEMMTensorParallelContext`` (:494-553), ``create_ag_group_gemm_intra_node_context`` (:555-638)
and ``ag_group_gemm_intra_node`` (:641-691). As in the AG-GEMM, the other ranks' token rows are handed to the context
(``ctx.set_peer_shards``) and copy streams of this GPU deliver them into the workspace and release one flag per rank
segment (the reference's producer: cp_engine_producer_all_gather_full_mesh_push, one barrier word per rank).
"""
import dataclasses
from typing import Dict, List, Optional

import torch

from triton_dist import _lib
from triton_dist.kernels.amd.common_ops import fill_flags


_ALIGN_PLANS = {}   # (ids, experts, ranks, topk, block size) -> scratch bytes and the layout of the results


def sort_topk_ids_align_block_size(
    topk_ids: torch.Tensor,
    num_experts: int,
    num_ranks: int,
    num_tokens_per_rank: int,
    block_size: int,
    moe_stream: torch.cuda.Stream = None,
):
    """
    Sort and align the token distribution across experts to be compatible with block size for matrix multiplication.

    Parameters (reference :62-72):
    - topk_ids: [total_tokens, top_k] expert index of every (token, k), int64 (the reference's dtype) or int32.
    - num_experts, num_ranks, num_tokens_per_rank (tokens, not topk-ed, per rank), block_size.
    - moe_stream: stream for the kernels; the current stream if None.

    Returns (sorted_token_ids, expert_ids, block_barrier_ids, rank_block_num, num_tokens_post_padded), all int32,
    allocated with the reference's capacities (:100-121); padding positions of sorted_token_ids hold
    topk_ids.numel().
    """
    _lib.require_cuda(topk_ids)
    if topk_ids.dtype not in (torch.int32, torch.int64):
        raise TypeError("topk_ids must be int32 or int64, got %s" % topk_ids.dtype)
    topk_ids = topk_ids.contiguous()
    num_topk = topk_ids.shape[1]
    dev = topk_ids.device
    n_total = topk_ids.numel()
    n_per = num_tokens_per_rank * num_topk
    assert n_total == n_per * num_ranks, "topk_ids must hold num_ranks * num_tokens_per_rank tokens"
    # sizes and scratch bytes once per shape: the call itself costs less than working them out again
    key = (n_total, num_experts, num_ranks, num_topk, block_size)
    plan = _ALIGN_PLANS.get(key)
    if plan is None:
        ws_bytes = _lib.load().tdist_moe_align_workspace_bytes(n_total, num_experts, num_ranks)
        if ws_bytes == 0:
            raise _lib.TdistError(_lib.TDIST_ERR_UNSUPPORTED,
                                  "num_experts * num_ranks = %d is above what the align kernel handles" % (num_experts * num_ranks))
        # the five results are views of one allocation (sizes as in the reference, :100-121; every view 16-byte aligned)
        n_sorted = (n_per + num_experts * (block_size - 1)) * num_ranks
        n_blocks = (n_per + num_experts) * num_ranks
        sizes = (n_sorted, n_blocks, n_blocks, num_ranks, 1)
        starts, at = [], 0
        for n in sizes:
            starts.append(at)
            at += (n + 3) // 4 * 4
        plan = _ALIGN_PLANS[key] = (ws_bytes, at, tuple(starts), sizes)
    ws_bytes, n_flat, starts, sizes = plan
    flat = torch.empty(n_flat, dtype=torch.int32, device=dev)
    sorted_ids, expert_ids, block_barrier_ids, rank_block_num, num_tokens_post_pad = (
        flat[a:a + n] for a, n in zip(starts, sizes))
    base = flat.data_ptr()
    ids_ptr, ids_int64 = topk_ids.data_ptr(), 1 if topk_ids.dtype == torch.int64 else 0

    def launch(stream):
        workspace = _lib.zeroed_scratch(ws_bytes, dev)   # (cached per stream: current is `stream` here)
        # (sorted_ids.fill_(numel) of the reference, :103, is done inside the call)
        _lib.call("tdist_moe_align_block_size", ids_ptr, ids_int64, n_total, num_experts, num_ranks, n_per, block_size,
                  base + 4 * starts[0], sizes[0], base + 4 * starts[1], base + 4 * starts[2], base + 4 * starts[3],
                  base + 4 * starts[4], workspace.data_ptr(), ws_bytes, stream.cuda_stream)

    if moe_stream is None:
        launch(torch.cuda.current_stream())      # no stream switch, event or allocator bookkeeping to pay for
    else:
        with torch.cuda.stream(moe_stream):
            launch(moe_stream)
        torch.cuda.current_stream().wait_stream(moe_stream)
    return (
        sorted_ids,
        expert_ids,
        block_barrier_ids,
        rank_block_num,
        num_tokens_post_pad,
    )


_GROUP_GEMM_ENTRY = {
    torch.bfloat16: "tdist_group_gemm_gated_bf16",
    torch.float16: "tdist_group_gemm_gated_f16",
    torch.float8_e4m3fn: "tdist_group_gemm_gated_fp8e4m3",
}


def group_gemm_gated(a_ws, a_local, local_row_begin, b_nk, c, sorted_token_ids, expert_ids, block_barrier_ids,
                     num_tokens_post_padded, block_size, num_valid_tokens, topk, tokens_per_rank, first_block, flags, rank,
                     *, wait_value=1, spin_limit=0, status=None, max_workgroups=0, sk_workspace=None, stream=None):
    """Thin wrapper over tdist_group_gemm_gated_*. ``a_ws`` [tokens, K] gathered rows, ``a_local`` the own shard or
    None, ``b_nk`` [E, N, K] (K contiguous), ``c`` [num_valid_tokens, N]."""
    _lib.require_cuda(a_ws, b_nk, c, sorted_token_ids, expert_ids, block_barrier_ids, num_tokens_post_padded)
    if a_ws.dtype not in _GROUP_GEMM_ENTRY:
        raise TypeError("unsupported grouped GEMM dtype %s" % a_ws.dtype)
    if a_ws.stride(1) != 1 or b_nk.stride(2) != 1 or c.stride(1) != 1:
        raise ValueError("A, B ([E, N, K]) and C need a contiguous last dimension")
    E, N, K = b_nk.shape
    assert a_ws.shape[1] == K and c.shape[1] == N
    num_blocks = min(expert_ids.numel(), sorted_token_ids.numel() // block_size)
    _lib.call(_GROUP_GEMM_ENTRY[a_ws.dtype], a_ws.data_ptr(), a_ws.stride(0), _lib.ptr(a_local),
              a_local.stride(0) if a_local is not None else 0, int(local_row_begin),
              a_local.shape[0] if a_local is not None else 0, b_nk.data_ptr(), b_nk.stride(1), b_nk.stride(0), c.data_ptr(),
              c.stride(0), a_ws.shape[0], N, K, sorted_token_ids.data_ptr(), expert_ids.data_ptr(),
              block_barrier_ids.data_ptr(), num_tokens_post_padded.data_ptr(), num_blocks, int(block_size),
              int(num_valid_tokens), int(topk), int(tokens_per_rank), int(first_block), _lib.ptr(flags), int(wait_value),
              int(rank), int(spin_limit), _lib.ptr(status), int(max_workgroups), *_lib.workspace_args(sk_workspace),
              _lib.stream_ptr(stream))
    return c


@dataclasses.dataclass
class MoE_AllGatherGroupGEMMTensorParallelContext:
    rank: int
    num_ranks: int
    num_experts: int
    topk: int
    full_num_tokens: int
    sorted_topk_ids: torch.Tensor
    aligned_expert_ids: torch.Tensor
    aligned_barrier_ids: torch.Tensor
    aligned_num_tokens: torch.Tensor
    workspace_tensors: List[Optional[torch.Tensor]]
    barrier_tensors: List[Optional[torch.Tensor]]
    internode_ag_stream: Optional[torch.cuda.streams.Stream] = None
    ag_stream: Optional[torch.cuda.streams.Stream] = None
    group_gemm_stream: Optional[torch.cuda.streams.Stream] = None
    local_world_size: int = 8
    BLOCK_M: int = 128
    BLOCK_N: int = 256
    BLOCK_K: int = 64
    GROUP_SIZE_M: int = 8
    stages: int = 3
    warps: int = 8
    # ---- one-GPU additions -------------------------------------------------------------------
    rank_block_num: Optional[torch.Tensor] = None
    first_block: int = 0                 # first row block of the own rank's segment (consumed first)
    peer_shards: Dict[int, torch.Tensor] = dataclasses.field(default_factory=dict)
    one: Optional[torch.Tensor] = None
    status: Optional[torch.Tensor] = None
    spin_limit: int = 0
    held_ranks: tuple = ()               # test hook: segments that are never delivered
    producer_cus: int = 32               # compute units left to the copies (see the AG-GEMM context)
    weight_nk: Optional[torch.Tensor] = None   # [E, N, K] copy of a [E, K, N] weight, made once per weight tensor
    weight_key: Optional[tuple] = None
    sk_workspace: Optional[torch.Tensor] = None   # the context's GEMM workspace (split of a last round along K); None = off

    def set_peer_shards(self, shards):
        """``shards``: dict rank -> [M_per_rank, K] tensor (or a list; the own entry is ignored): the token rows that
        live on the other ranks."""
        if not isinstance(shards, dict):
            shards = {r: t for r, t in enumerate(shards) if t is not None}
        for r, t in shards.items():
            if r != self.rank:
                _lib.require_cuda(t)
                if not t.is_contiguous():
                    raise ValueError("peer shard of rank %d must be contiguous" % r)
        self.peer_shards = {r: t for r, t in shards.items() if r != self.rank}

    def check_status(self):
        """Synchronises and raises TdistError if a bounded flag wait expired in an earlier call (the earliest one
        since the last check; status[0:2] is the current call's, [2:4] the first of the calls before it)."""
        torch.cuda.synchronize()
        code, segment, first_code, first_segment = self.status.tolist()
        if first_code != 0:
            code, segment = first_code, first_segment
        if code != 0:
            self.status.zero_()
            raise _lib.TdistError(code, "flag wait expired for rank segment %d" % segment)


def create_ag_group_gemm_intra_node_context(tp_pg, tensor_A, tensor_B, full_topk_ids, num_experts, max_M=2**14, BLOCK_M=128,
                                            BLOCK_N=256, BLOCK_K=64, GROUP_SIZE_M=8, stages=3, warps=8, ag_stream=None,
                                            group_gemm_stream=None, rank=None, num_ranks=None, split_k=True):
    """create context for allgather group gemm intra-node (reference :555-638).

    tensor_A [M_per_rank, K] local tokens, tensor_B [E, K, N_per_rank] local expert weights, full_topk_ids
    [M_per_rank * num_ranks, topk]. ``tp_pg`` may be None on one GPU: pass ``rank`` / ``num_ranks``. BLOCK_M is the
    row block of the align / sort and of the GEMM tile (128 or 256); the other tiling arguments are accepted for
    signature compatibility. ``split_k``: give the context a GEMM workspace (64 MiB): the number of row blocks
    in use is seldom a multiple of the grid, and with the workspace the grouped GEMM cuts the tiles of a last round that
    fills at most half of the grid along K."""
    if not torch.cuda.is_available():
        raise RuntimeError("create_ag_group_gemm_intra_node_context needs a GPU")
    _lib.check(_lib.load().tdist_init())
    M_per_rank, K = tensor_A.shape
    _, topk = full_topk_ids.shape
    assert tensor_B.shape[1] == K, "tensor_B should have shape [E, %d, N_per_rank], got %s" % (K, tuple(tensor_B.shape))
    assert tensor_A.dtype == tensor_B.dtype
    if tp_pg is not None:
        rank, num_ranks = tp_pg.rank(), tp_pg.size()
    assert rank is not None and num_ranks is not None
    assert full_topk_ids.shape[0] == M_per_rank * num_ranks and M_per_rank * num_ranks <= max_M
    device = tensor_A.device
    workspaces: List[Optional[torch.Tensor]] = [None] * num_ranks
    barriers: List[Optional[torch.Tensor]] = [None] * num_ranks
    workspaces[rank] = torch.empty([max_M, K], dtype=tensor_A.dtype, device=device)
    barriers[rank] = torch.zeros([num_ranks], dtype=torch.int32, device=device)
    sorted_ids, expert_ids, barrier_ids, rank_block_num, post_pad = sort_topk_ids_align_block_size(
        full_topk_ids, num_experts, num_ranks, M_per_rank, BLOCK_M)
    torch.cuda.synchronize()
    first_block = int(rank_block_num[:rank].sum().item()) if rank > 0 else 0
    return MoE_AllGatherGroupGEMMTensorParallelContext(
        rank=rank, num_ranks=num_ranks, num_experts=num_experts, topk=topk, full_num_tokens=full_topk_ids.numel(),
        sorted_topk_ids=sorted_ids, aligned_expert_ids=expert_ids, aligned_barrier_ids=barrier_ids,
        aligned_num_tokens=post_pad, workspace_tensors=workspaces, barrier_tensors=barriers,
        ag_stream=torch.cuda.Stream() if ag_stream is None else ag_stream,
        group_gemm_stream=group_gemm_stream, BLOCK_M=BLOCK_M, BLOCK_N=BLOCK_N, BLOCK_K=BLOCK_K,
        GROUP_SIZE_M=GROUP_SIZE_M, stages=stages, warps=warps, rank_block_num=rank_block_num, first_block=first_block,
        one=torch.ones((16, ), dtype=torch.int32, device=device), status=torch.zeros((4, ), dtype=torch.int32, device=device),
        sk_workspace=_lib.new_split_k_workspace(device) if split_k else None)


def _weight_nk(ctx, b):
    """[E, K, N] weights as an [E, N, K] K-contiguous tensor: a view when the caller's tensor already is one
    (stride of K == 1), else a transposed copy made once per weight tensor and kept in the context."""
    if b.stride(1) == 1:
        return b.transpose(1, 2)
    key = (b.data_ptr(), tuple(b.shape), b._version)
    if ctx.weight_key != key:
        ctx.weight_nk = b.transpose(1, 2).contiguous()
        ctx.weight_key = key
    return ctx.weight_nk


def ag_group_gemm_intra_node(a, b, ctx=None, full_topk_ids=None, num_experts=None):
    """intra-node allgather group gemm (reference :641-691)

    a [M_per_rank, K] local tokens, b [E, K, N_per_rank] local expert weights. Returns C [M * topk, N_per_rank]:
    row t*topk + k is token t of the gathered A times the weights of its k-th expert."""
    if ctx is None:
        raise RuntimeError("one GPU holds a single rank: create the context first and hand it the peers' rows")
    _lib.require_cuda(a, b)
    M_per_rank, K = a.shape
    E, _, N_per_rank = b.shape
    W, rank = ctx.num_ranks, ctx.rank
    missing = [r for r in range(W) if r != rank and r not in ctx.peer_shards]
    if missing:
        raise RuntimeError("hand the other ranks' token rows to the context first (ctx.set_peer_shards); missing %s" % missing)
    out_dtype = a.dtype if a.dtype in (torch.bfloat16, torch.float16) else torch.bfloat16
    C = torch.empty([ctx.topk * M_per_rank * W, N_per_rank], dtype=out_dtype, device=a.device)
    b_nk = _weight_nk(ctx, b)
    workspace, barrier = ctx.workspace_tensors[rank], ctx.barrier_tensors[rank]
    current = torch.cuda.current_stream()
    gemm_stream = current if ctx.group_gemm_stream is None else ctx.group_gemm_stream
    fork = current.record_event()   # one event for both streams; a GEMM on the caller's own stream needs none
    ctx.ag_stream.wait_event(fork)
    if gemm_stream is not current:
        gemm_stream.wait_event(fork)
    # producer: one copy and one flag per peer rank (reference :354-361)
    nbytes = M_per_rank * K * a.element_size()
    for idx in range(1, W):
        r = (rank + idx) % W
        if r in ctx.held_ranks:
            continue
        _lib.call("tdist_producer_push_chunk", workspace.data_ptr() + r * nbytes, ctx.peer_shards[r].data_ptr(), nbytes,
                  barrier.data_ptr() + 4 * r, ctx.one.data_ptr(), 0, ctx.ag_stream.cuda_stream)
    max_wgs = max(1, _lib.load().tdist_num_cus() - ctx.producer_cus) if (W > 1 and ctx.producer_cus > 0) else 0
    # the launch before may have given up on a flag: keep what it reported, start this one clean
    _lib.call("tdist_status_retire", ctx.status.data_ptr(), ctx.status.data_ptr() + 8, gemm_stream.cuda_stream)
    # (the launch names its stream; nothing here runs on torch's current stream)
    group_gemm_gated(workspace[:M_per_rank * W], a, rank * M_per_rank, b_nk, C, ctx.sorted_topk_ids,
                     ctx.aligned_expert_ids, ctx.aligned_barrier_ids, ctx.aligned_num_tokens, ctx.BLOCK_M,
                     ctx.full_num_tokens, ctx.topk, M_per_rank, ctx.first_block, barrier, rank,
                     spin_limit=ctx.spin_limit, status=ctx.status, max_workgroups=max_wgs, sk_workspace=ctx.sk_workspace,
                     stream=gemm_stream)
    current.wait_stream(ctx.ag_stream)
    if gemm_stream is not current:
        current.wait_stream(gemm_stream)
    fill_flags(barrier, 0)   # the reference's block_barriers[rank].zero_() (:399)
    return C
