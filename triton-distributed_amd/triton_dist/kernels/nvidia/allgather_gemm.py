"""AG-GEMM behind the signatures of the reference's kernels/nvidia/allgather_gemm.py
(``create_ag_gemm_intra_node_context`` :785-833, ``ag_gemm_intra_node`` :835-882). The work is the gfx950 path of
triton_dist.kernels.amd.all_gather_gemm; this module only maps the arguments: the NVIDIA-side entry points take the
local tensors instead of sizes, gate per rank segment (one barrier word per rank, :222-224) and create their context
on demand."""
import torch

from triton_dist.kernels.amd import all_gather_gemm as _amd

AllGatherGEMMTensorParallelContext = _amd.AllGatherGEMMTensorParallelContext


def create_ag_gemm_intra_node_context(tensor_A, tensor_B, rank, num_ranks, max_M=2**14, max_blocks=65536, BLOCK_M=128,
                                      BLOCK_N=256, BLOCK_K=64, stages=3, for_correctness=False, ag_stream=None,
                                      gemm_stream=None, serial=False, autotune=False):
    """tensor_A [M_per_rank, K], tensor_B [N_per_rank, K]. One flag per rank segment, as in the reference
    (barriers of shape [num_ranks], :817); M_per_rank may be any number of rows (a tile of the GEMM waits for every
    rank segment its rows touch, as the reference's consumer does, :222-224). ``max_blocks`` is accepted and unused (no
    block-level barrier buffer here). ``for_correctness``: the reference's producer then sleeps with probability 0.7
    before it copies (allgather.py:72-77,118-121), to show a consumer that does not wait; here the peers' rows then
    come from the one-launch producer with seeded random delays of up to 200 us per rank segment
    (``ctx.random_delay_us``, ``ctx.delay_seed``)."""
    M_per_rank, K = tensor_A.shape
    assert tensor_B.shape[1] == K, "tensor_B should have shape [N_per_rank, %d], got %s" % (K, tuple(tensor_B.shape))
    assert tensor_A.dtype == tensor_B.dtype
    M = M_per_rank * num_ranks
    assert M <= max_M
    out_dtype = tensor_A.dtype if tensor_A.dtype in (torch.bfloat16, torch.float16) else torch.bfloat16
    ctx = _amd.create_ag_gemm_intra_node_context(M, tensor_B.shape[0], K, tensor_A.dtype, out_dtype, rank, num_ranks, None,
                                                 ag_streams=None if ag_stream is None else [ag_stream],
                                                 gemm_stream=gemm_stream, M_PER_CHUNK=M_per_rank, BLOCK_M=BLOCK_M,
                                                 BLOCK_N=BLOCK_N, BLOCK_K=BLOCK_K, stages=stages, serial=serial,
                                                 autotune=autotune, ragged_chunks=True)
    if for_correctness:
        ctx.producer_kernel, ctx.random_delay_us = True, 200.0
    return ctx


def ag_gemm_intra_node(a, b, ctx=None, rank=None, num_ranks=None, persistent=True):
    """a [M_per_rank, K], b [N_per_rank, K] → C [M, N_per_rank] (reference :835-882). A context created on demand
    has no peers' rows (one GPU holds one rank): create it first and call ``ctx.set_peer_shards`` unless
    num_ranks == 1. ``persistent`` is accepted: the kernel is always the persistent one."""
    if ctx is None:
        assert rank is not None and num_ranks is not None
        ctx = create_ag_gemm_intra_node_context(a, b, rank, num_ranks)
    return _amd.ag_gemm_intra_node(a, b, False, ctx)
