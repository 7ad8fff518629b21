"""Op-level entry points (same names as the reference's triton_dist.kernels.amd, kernels/amd/__init__.py:25-30,
plus the ops the reference keeps under kernels/nvidia, which here are gfx950 kernels like the rest)."""
from .all_gather_gemm import ag_gemm_intra_node, create_ag_gemm_intra_node_context, gated_gemm
from .gemm_reduce_scatter import gemm_rs_intra_node, create_gemm_rs_intra_node_context
from .low_latency_all_to_all import (create_all_to_all_context, fast_all_to_all, all_to_all_post_process,
                                     moe_dispatch_preprocess, moe_weighted_combine, splits_to_cumsum, quant_bf16_fp8)
from .allgather_group_gemm import (sort_topk_ids_align_block_size, create_ag_group_gemm_intra_node_context,
                                   ag_group_gemm_intra_node, group_gemm_gated)
from .moe_reduce_rs import create_moe_rs_context, moe_reduce_rs, select_experts
from .flash_decode import (gqa_fwd_batch_decode, gqa_fwd_batch_decode_intra_rank, gqa_fwd_batch_decode_persistent,
                           gqa_fwd_batch_decode_inter_rank_combine)

__all__ = [
    "ag_gemm_intra_node", "create_ag_gemm_intra_node_context", "gated_gemm", "gemm_rs_intra_node",
    "create_gemm_rs_intra_node_context", "create_all_to_all_context", "fast_all_to_all", "all_to_all_post_process",
    "moe_dispatch_preprocess", "moe_weighted_combine", "splits_to_cumsum", "quant_bf16_fp8", "sort_topk_ids_align_block_size",
    "create_ag_group_gemm_intra_node_context", "ag_group_gemm_intra_node", "group_gemm_gated", "gqa_fwd_batch_decode",
    "gqa_fwd_batch_decode_intra_rank", "gqa_fwd_batch_decode_persistent", "gqa_fwd_batch_decode_inter_rank_combine", "create_moe_rs_context", "moe_reduce_rs", "select_experts",
]
