"""GEMM-RS behind the signatures of the reference's kernels/nvidia/gemm_reduce_scatter.py
(``create_gemm_rs_context`` :77-88, ``gemm_rs`` :524-538, row padding :468-479). The work is the gfx950 path of
triton_dist.kernels.amd.gemm_reduce_scatter."""
import torch

from triton_dist.kernels.amd import gemm_reduce_scatter as _amd

GEMMReduceScatterTensorParallelContext = _amd.GEMMReduceScatterTensorParallelContext


def create_gemm_rs_context(max_M, N, rank, world_size, local_world_size, output_dtype, rs_stream, BLOCK_M=128, BLOCK_N=256,
                           BLOCK_K=64, GROUP_M=8, stages=3):
    """``local_world_size`` and ``rs_stream`` are accepted for signature compatibility: on one GPU the reduction runs on
    the caller's stream after the GEMM. Every rank's rows are padded to BLOCK_M (a multiple of 128) in the scatter
    buffer, as the reference pads them (:468-479)."""
    if BLOCK_M % 128 != 0:
        raise NotImplementedError("BLOCK_M %d: the scatter GEMM works on row blocks that are multiples of 128" % BLOCK_M)
    padded = -(-(max_M // world_size) // BLOCK_M) * BLOCK_M * world_size
    ctx = _amd.create_gemm_rs_intra_node_context(padded, N, output_dtype, rank, world_size, None)
    ctx.block_m = BLOCK_M
    return ctx


def padded_to_BLOCK_M(input, world_size, BLOCK_SIZE_M):
    """reference :468-479: every rank's M_per_rank rows padded to a multiple of BLOCK_SIZE_M (the padding rows are
    zero here, uninitialised there; they are cut off again after the reduction)."""
    M, local_K = input.shape
    M_per_rank = M // world_size
    pad_size = (M_per_rank + BLOCK_SIZE_M - 1) // BLOCK_SIZE_M * BLOCK_SIZE_M
    if pad_size == M_per_rank:
        return input
    pad_input = torch.zeros((world_size, pad_size, local_K), dtype=input.dtype, device=input.device)
    pad_input[:, :M_per_rank].copy_(input.reshape(world_size, M_per_rank, local_K))
    return pad_input.reshape(-1, local_K)


def gemm_rs(a, b, ctx, persistent=True):
    """a [M, local_K], b [N, local_K] → [M // world_size, N] (reference :482-538)."""
    world_size = ctx.num_ranks
    orig_M_per_rank = a.shape[0] // world_size
    assert a.shape[0] % world_size == 0 and b.shape[1] == a.shape[1]
    a = padded_to_BLOCK_M(a, world_size, ctx.block_m or 128)
    M = a.shape[0]
    current_stream = torch.cuda.current_stream()
    _amd.matmul_fuse_scatter(a, b, ctx.scatter_bufs_ptr, ctx.rank, world_size, transpose_weight=False,
                             ldc=ctx.scatter_bufs[ctx.rank].stride(0), stream=current_stream, strict_alignment=False)
    output = _amd.ring_reduce_after_scatter(ctx.rank, world_size, ctx.scatter_bufs[ctx.rank][:M], current_stream)
    return output[:orig_M_per_rank]
