"""Import-path compatibility: the reference keeps the MoE all-to-all, the grouped GEMM and the flash-decode ops under
triton_dist.kernels.nvidia (kernels/nvidia/__init__.py:25-89), and NVIDIA-side variants of AG-GEMM and GEMM-RS with
their own argument lists. The names resolve to the same gfx950 implementations as triton_dist.kernels.amd; nothing
here is CUDA."""
from triton_dist.kernels.amd.low_latency_all_to_all import (create_all_to_all_context, fast_all_to_all,
                                                            all_to_all_post_process)
from triton_dist.kernels.amd.allgather_group_gemm import (sort_topk_ids_align_block_size,
                                                          create_ag_group_gemm_intra_node_context,
                                                          ag_group_gemm_intra_node)
from triton_dist.kernels.amd.moe_reduce_rs import create_moe_rs_context, moe_reduce_rs, select_experts
from triton_dist.kernels.amd.flash_decode import (gqa_fwd_batch_decode, gqa_fwd_batch_decode_intra_rank,
                                                  gqa_fwd_batch_decode_persistent)

from .allgather_gemm import ag_gemm_intra_node, create_ag_gemm_intra_node_context
from .gemm_reduce_scatter import create_gemm_rs_context, gemm_rs

__all__ = [
    "ag_gemm_intra_node", "create_ag_gemm_intra_node_context", "create_gemm_rs_context", "gemm_rs",
    "create_all_to_all_context", "fast_all_to_all", "all_to_all_post_process", "gqa_fwd_batch_decode",
    "gqa_fwd_batch_decode_intra_rank", "gqa_fwd_batch_decode_persistent", "sort_topk_ids_align_block_size",
    "create_ag_group_gemm_intra_node_context", "ag_group_gemm_intra_node", "create_moe_rs_context", "moe_reduce_rs", "select_experts",
]
