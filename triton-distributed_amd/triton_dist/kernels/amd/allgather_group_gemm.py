"""MoE align / sort for the grouped GEMM (the step that follows the dispatch), on one MI355X.

Keeps ``sort_topk_ids_align_block_size`` of the reference's kernels/nvidia/allgather_group_gemm.py (:54-135), whose
device work is the C++ op moe_ag_scatter_align_block_size (csrc/lib/moe_utils.cu:60-186); here it is
tdist_moe_align_block_size of libtdist_hip.so.
"""
import torch

from triton_dist import _lib


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
    n_per = num_tokens_per_rank * num_topk
    n_total = topk_ids.numel()
    assert n_total == n_per * num_ranks, "topk_ids must hold num_ranks * num_tokens_per_rank tokens"
    sorted_ids = torch.empty(((n_per + num_experts * (block_size - 1)) * num_ranks, ), dtype=torch.int32, device=dev)
    expert_ids = torch.empty(((n_per + num_experts) * num_ranks, ), dtype=torch.int32, device=dev)
    block_barrier_ids = torch.empty(((n_per + num_experts) * num_ranks, ), dtype=torch.int32, device=dev)
    rank_block_num = torch.empty(num_ranks, dtype=torch.int32, device=dev)
    num_tokens_post_pad = torch.empty((1), dtype=torch.int32, device=dev)
    ws_bytes = _lib.load().tdist_moe_align_workspace_bytes(n_total, num_experts, num_ranks)
    if ws_bytes == 0:
        raise _lib.TdistError(_lib.TDIST_ERR_UNSUPPORTED,
                              "num_experts * num_ranks = %d is above what the align kernel handles" % (num_experts * num_ranks))
    workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    moe_stream = torch.cuda.current_stream() if moe_stream is None else moe_stream
    with torch.cuda.stream(moe_stream):
        sorted_ids.fill_(n_total)
        _lib.call("tdist_moe_align_block_size", topk_ids.data_ptr(), 1 if topk_ids.dtype == torch.int64 else 0, n_total,
                  num_experts, num_ranks, n_per, block_size, sorted_ids.data_ptr(), expert_ids.data_ptr(),
                  block_barrier_ids.data_ptr(), rank_block_num.data_ptr(), num_tokens_post_pad.data_ptr(),
                  workspace.data_ptr(), ws_bytes, moe_stream.cuda_stream)
    torch.cuda.current_stream().wait_stream(moe_stream)
    workspace.record_stream(moe_stream)
    return (
        sorted_ids,
        expert_ids,
        block_barrier_ids,
        rank_block_num,
        num_tokens_post_pad,
    )
