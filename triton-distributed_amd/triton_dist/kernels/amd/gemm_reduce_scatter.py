"""GEMM-RS on one MI355X: a GEMM whose epilogue scatters every row block to its owner's buffer, then
the fp32 reduction of the slices the owner received.

Keeps the interface of the reference's kernels/amd/gemm_reduce_scatter.py
(``create_gemm_rs_intra_node_context`` :381-426, ``gemm_rs_intra_node`` :429-446, context :368-378).
With one GPU the ``num_ranks`` scatter buffers all live on it: the GEMM still writes the row block of
owner ``o`` into ``scatter_bufs[o]`` at row block ``rank`` (:222-229), and the partial slices the other
ranks would have stored into this rank's buffer are handed over with ``ctx.set_peer_partials``.
"""
import dataclasses
from typing import List, Optional

import torch

from triton_dist import _lib


@dataclasses.dataclass
class GEMMReduceScatterTensorParallelContext:
    rank: int
    num_ranks: int
    scatter_bufs: List[torch.Tensor]
    scatter_bufs_ptr: torch.Tensor
    sync_bufs_ptr: Optional[torch.Tensor]
    sync_bufs: List[Optional[torch.Tensor]]
    output_dtype: torch.dtype
    fuse_scatter: bool
    transpose_weight: bool
    # rows every rank's slice is padded to in the scatter buffer (the NVIDIA-side entry point pads M_per_rank to its
    # BLOCK_M, kernels/nvidia/gemm_reduce_scatter.py:468-479); None = no padding
    block_m: Optional[int] = None
    # workspace of the context's GEMM launches (a last round that does not fill the grid is cut along K); None = off
    sk_workspace: Optional[torch.Tensor] = None

    def set_peer_partials(self, partials):
        """``partials``: dict rank -> [M_per_rank, N] tensor, or a list of num_ranks entries (the entry of
        ``rank`` is ignored): what rank r's GEMM computed for this rank's rows. Stored where r's epilogue
        would have put it: rows [r*M_per_rank, (r+1)*M_per_rank) of this rank's scatter buffer."""
        if not isinstance(partials, dict):
            partials = {r: t for r, t in enumerate(partials) if t is not None}
        buf = self.scatter_bufs[self.rank]
        for r, t in partials.items():
            if r == self.rank:
                continue
            m_per_rank = t.shape[0]
            stride = m_per_rank if self.block_m is None else -(-m_per_rank // self.block_m) * self.block_m
            buf[r * stride:r * stride + m_per_rank, :t.shape[1]].copy_(t)


def create_gemm_rs_intra_node_context(max_M, N, output_dtype, rank, num_ranks, tp_group, fuse_scatter=True,
                                      transpose_weight=False, split_k=True):
    """create context for gemm reduce-scatter intra-node (reference :381-426). ``tp_group`` may be None.
    ``split_k``: give the context a GEMM workspace (see create_ag_gemm_intra_node_context)."""
    if not fuse_scatter:
        raise NotImplementedError()
    if transpose_weight:
        raise NotImplementedError()
    if not torch.cuda.is_available():
        raise RuntimeError("create_gemm_rs_intra_node_context needs a GPU")
    _lib.check(_lib.load().tdist_init())
    device = torch.device("cuda", torch.cuda.current_device())
    sk_workspace = _lib.new_split_k_workspace(device) if split_k else None
    scatter_bufs = [torch.zeros([max_M, N], dtype=output_dtype, device=device) for _ in range(num_ranks)]
    scatter_bufs_ptr = torch.tensor([t.data_ptr() for t in scatter_bufs], dtype=torch.int64, device=device)
    torch.cuda.synchronize()
    return GEMMReduceScatterTensorParallelContext(
        rank=rank,
        num_ranks=num_ranks,
        scatter_bufs=scatter_bufs,
        scatter_bufs_ptr=scatter_bufs_ptr,
        sync_bufs_ptr=None,
        sync_bufs=[None] * num_ranks,
        output_dtype=output_dtype,
        fuse_scatter=fuse_scatter,
        transpose_weight=transpose_weight,
        sk_workspace=sk_workspace,
    )


_SCATTER_ENTRY = {torch.bfloat16: "tdist_gemm_rs_scatter_bf16", torch.float16: "tdist_gemm_rs_scatter_f16",
                  torch.float8_e4m3fn: "tdist_gemm_rs_scatter_fp8e4m3"}


def matmul_fuse_scatter(a, b, scatter_bufs_ptr, rank, num_ranks, transpose_weight, ldc=None, stream=None,
                        strict_alignment=True, sk_workspace=None, row_scale=None, col_scale=None):
    """GEMM with the scatter epilogue (reference :289-314). ``b`` is [N, K]. ``strict_alignment`` keeps the
    reference's assertion (M, N, K multiples of 256); without it the library's own limits apply (M / num_ranks a
    multiple of 128, K rows a multiple of 16 bytes). e4m3 inputs write bf16 partial results and take optional fp32
    ``row_scale`` [M] / ``col_scale`` [N]."""
    if transpose_weight:
        raise NotImplementedError()
    assert a.shape[1] == b.shape[1], "Incompatible dimensions"
    assert a.is_contiguous(), "Matrix A must be contiguous"
    M, K = a.shape
    N = b.shape[0]
    alignment = 256
    assert not strict_alignment or (M % alignment == 0 and N % alignment == 0 and K % alignment == 0)
    if a.dtype not in _SCATTER_ENTRY:
        raise TypeError("unsupported GEMM-RS dtype %s" % a.dtype)
    scales = []
    if a.dtype == torch.float8_e4m3fn:
        scales = [_lib.ptr(row_scale), _lib.ptr(col_scale)]
    elif row_scale is not None or col_scale is not None:
        raise ValueError("scales are only defined for fp8 inputs")
    _lib.call(_SCATTER_ENTRY[a.dtype], a.data_ptr(), a.stride(0), b.data_ptr(), b.stride(0),
              scatter_bufs_ptr.data_ptr(), N if ldc is None else ldc, M, N, K, *scales, rank, num_ranks,
              *_lib.workspace_args(sk_workspace), _lib.stream_ptr(stream))


def ring_reduce_after_scatter(rank, num_ranks, scatter_out, stream):
    """Sum of the num_ranks slices of ``scatter_out`` [M, N] in the order rank+1, rank+2, ... (reference
    :264-286 / kernel :246-258), accumulated in fp32."""
    M, N = scatter_out.shape
    assert scatter_out.is_contiguous()
    M_per_rank = M // num_ranks
    output = torch.empty((M_per_rank, N), dtype=scatter_out.dtype, device=scatter_out.device)
    _lib.call("tdist_reduce_slices", scatter_out.data_ptr(), M_per_rank * N, num_ranks, (rank + 1) % num_ranks,
              M_per_rank * N, output.data_ptr(), _lib.dtype_code(scatter_out.dtype), stream.cuda_stream)
    return output


def gemm_rs_intra_node_op(a, b, output_dtype, rank, num_ranks, scatter_bufs, scatter_bufs_ptr, sync_bufs_ptr,
                          fuse_scatter=True, transpose_weight=False, sk_workspace=None, row_scale=None, col_scale=None):
    """gemm reduce scatter for intra-node (reference :317-365)."""
    if not fuse_scatter:
        raise NotImplementedError()
    if transpose_weight:
        raise NotImplementedError()
    _lib.require_cuda(a, b)
    M, local_K = a.shape
    N, weight_local_K = b.shape
    assert weight_local_K == local_K
    assert a.dtype == b.dtype
    partial_dtype = torch.bfloat16 if a.dtype == torch.float8_e4m3fn else a.dtype
    if scatter_bufs[rank].dtype != partial_dtype:
        raise TypeError("the scatter buffers hold the GEMM's input dtype (reference :217-218; bf16 for e4m3 inputs): "
                        "ctx was created for %s, inputs are %s" % (scatter_bufs[rank].dtype, a.dtype))
    current_stream = torch.cuda.current_stream()
    matmul_fuse_scatter(a, b, scatter_bufs_ptr, rank, num_ranks, transpose_weight=transpose_weight,
                        ldc=scatter_bufs[rank].stride(0), stream=current_stream, sk_workspace=sk_workspace,
                        row_scale=row_scale, col_scale=col_scale)
    scatter_out = scatter_bufs[rank][:M]
    output = ring_reduce_after_scatter(rank, num_ranks, scatter_out, current_stream)
    return output


def gemm_rs_intra_node(a, b, ctx, *, row_scale=None, col_scale=None):
    """GEMM Reduce-Scatter for Intra-Node (reference :429-446)

    Args:
        a (torch.Tensor<bfloat16/float16/float8_e4m3fn>): local matmul A matrix. shape: [M, local_K]
        b (torch.Tensor, same dtype): local matmul B matrix. shape: [N, local_K]
        ctx (GEMMReduceScatterTensorParallelContext)
        row_scale / col_scale: e4m3 inputs only: fp32 scales per row of a ([M]) and per row of b ([N]); no
            counterpart in the reference. The context of an e4m3 call is created with output_dtype bfloat16.

    Returns:
        c (torch.Tensor<bfloat16/float16>): shape [M // world_size, N]
    """
    return gemm_rs_intra_node_op(a, b, ctx.output_dtype, ctx.rank, ctx.num_ranks, ctx.scatter_bufs,
                                 ctx.scatter_bufs_ptr, ctx.sync_bufs_ptr, ctx.fuse_scatter, ctx.transpose_weight,
                                 sk_workspace=ctx.sk_workspace, row_scale=row_scale, col_scale=col_scale)
