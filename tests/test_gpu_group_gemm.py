"""The chunk-gated grouped GEMM of the MoE tensor-parallel path (AG + grouped GEMM) on the GPU against the oracle.
Bar: max relative error <= 1e-2 against the fp32 closed form (the reference's own test asks for atol = rtol = 1e-3 on
fp16, test/nvidia/test_ag_moe.py:102); exact on integer-valued inputs; every row of C written exactly once."""
import pytest
import torch

from oracle import golden
from tests.conftest import announce

pytestmark = pytest.mark.gpu


def make_case(world, m_per_rank, K, N, E, topk, dtype, seed, integer=False):
    g = torch.Generator().manual_seed(seed)
    if integer:
        shards = [torch.randint(-2, 3, (m_per_rank, K), generator=g).float().to(dtype) for _ in range(world)]
        w = torch.randint(-2, 3, (E, K, N), generator=g).float().to(dtype)
    else:
        shards = [torch.randn((m_per_rank, K), generator=g).to(dtype) for _ in range(world)]
        w = (torch.randn((E, K, N), generator=g) * 0.05).to(dtype)
    ids = golden.random_distinct_experts(world * m_per_rank, E, topk, g)
    return shards, w, ids


def run(cuda, shards, w, ids, rank, E, block, **ctx_kw):
    from triton_dist.kernels.nvidia import ag_group_gemm_intra_node, create_ag_group_gemm_intra_node_context
    world = len(shards)
    a = shards[rank].to(cuda)
    b = w.to(cuda)
    ctx = create_ag_group_gemm_intra_node_context(None, a, b, ids.to(cuda), E, max_M=world * a.shape[0], BLOCK_M=block,
                                                  rank=rank, num_ranks=world)
    for k, v in ctx_kw.items():
        setattr(ctx, k, v)
    ctx.set_peer_shards({r: s.to(cuda) for r, s in enumerate(shards) if r != rank})
    ctx.workspace_tensors[rank].view(torch.uint8).fill_(0x7B)     # stale rows must never reach C
    c = ag_group_gemm_intra_node(a, b, ctx)
    return ctx, c


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float8_e4m3fn])
@pytest.mark.parametrize("block,K", [(128, 256), (256, 512), (128, 96)])
def test_exact_on_integer_inputs(cuda, dtype, block, K):
    """Integer-valued tokens and weights: the fp32 sums are exact, only the final rounding remains. K = 96 elements of
    16 bits is an odd number of 64-byte halves and takes the 128 x 128 tile."""
    if dtype == torch.float8_e4m3fn:
        K = K * 2 if K == 96 else K
    world, mpr, N, E, topk = 4, 96, 328, 6, 2
    announce("group gemm exact %s block %d K %d" % (dtype, block, K))
    shards, w, ids = make_case(world, mpr, K, N, E, topk, dtype, seed=block + K, integer=True)
    for rank in (0, 3):
        ctx, c = run(cuda, shards, w, ids, rank, E, block)
        ctx.check_status()
        ref = golden.ag_group_gemm_fp32(shards, w, ids)
        assert torch.equal(c.float().cpu(), ref.to(c.dtype).float()), "rank %d" % rank


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_random_inputs_and_the_reference_golden(cuda, dtype):
    world, mpr, K, N, E, topk = 8, 256, 1024, 768, 16, 4
    announce("group gemm random %s" % dtype)
    shards, w, ids = make_case(world, mpr, K, N, E, topk, dtype, seed=5)
    ctx, c = run(cuda, shards, w, ids, 2, E, 128)
    ctx.check_status()
    ref = golden.ag_group_gemm_fp32(shards, w, ids)
    assert golden.max_rel_err(c.float().cpu(), ref) <= 1e-2
    # the reference's own golden in the input dtype (on the CPU) at its bar for 16-bit inputs
    gold = golden.torch_moe_scatter_group_gemm(torch.cat(shards), w, ids)
    assert torch.allclose(c.float().cpu(), gold.float(), atol=2e-2, rtol=2e-2)
    # a second call on the same context (flags were reset) gives the same bytes
    c2 = run_again(cuda, ctx, shards, w, 2)
    assert torch.equal(c2, c)


def run_again(cuda, ctx, shards, w, rank):
    from triton_dist.kernels.nvidia import ag_group_gemm_intra_node
    ctx.workspace_tensors[rank].view(torch.uint8).fill_(0x11)
    c = ag_group_gemm_intra_node(shards[rank].to(cuda), w.to(cuda), ctx)
    ctx.check_status()
    return c


def test_skewed_routing_and_unused_experts(cuda):
    """All tokens of one rank go to one expert, some experts get nothing, topk = 1: blocks of very different counts
    per segment, and segments with a single block."""
    world, mpr, K, N, E = 4, 200, 256, 256, 8
    announce("group gemm skewed routing")
    g = torch.Generator().manual_seed(9)
    shards = [torch.randint(-2, 3, (mpr, K), generator=g).float().bfloat16() for _ in range(world)]
    w = torch.randint(-2, 3, (E, K, N), generator=g).float().bfloat16()
    ids = torch.cat([torch.full((mpr, 1), 7), torch.randint(0, 2, (mpr, 1), generator=g), torch.full((mpr, 1), 3),
                     torch.randint(4, 6, (mpr, 1), generator=g)]).long()
    ctx, c = run(cuda, shards, w, ids, 1, E, 128)
    ctx.check_status()
    assert torch.equal(c.float().cpu(), golden.ag_group_gemm_fp32(shards, w, ids).bfloat16().float())


def test_a_segment_that_never_arrives_times_out(cuda):
    """Host-forced failure: one rank's rows are never delivered and the spin limit is tiny. The call reports the
    segment, every other segment's rows are correct, and the missing segment's rows keep their poison."""
    from triton_dist import _lib
    world, mpr, K, N, E, topk = 4, 128, 256, 256, 4, 2
    announce("group gemm bounded wait")
    shards, w, ids = make_case(world, mpr, K, N, E, topk, torch.bfloat16, seed=13, integer=True)
    from triton_dist.kernels.nvidia import ag_group_gemm_intra_node, create_ag_group_gemm_intra_node_context
    rank, held = 0, 2
    a, b = shards[rank].to(cuda), w.to(cuda)
    ctx = create_ag_group_gemm_intra_node_context(None, a, b, ids.to(cuda), E, max_M=world * mpr, BLOCK_M=128, rank=rank,
                                                  num_ranks=world)
    ctx.set_peer_shards({r: s.to(cuda) for r, s in enumerate(shards) if r != rank})
    ctx.held_ranks, ctx.spin_limit = (held, ), 2000
    c = ag_group_gemm_intra_node(a, b, ctx)
    with pytest.raises(_lib.TdistError) as err:
        ctx.check_status()
    assert err.value.code == _lib.TDIST_ERR_TIMEOUT and "segment %d" % held in str(err.value)
    ref = golden.ag_group_gemm_fp32(shards, w, ids).bfloat16()
    rows = torch.arange(world * mpr * topk) // (mpr * topk)
    ok = rows != held
    assert torch.equal(c.cpu()[ok], ref[ok])


def test_arguments_are_checked(cuda):
    from triton_dist import _lib
    from triton_dist.kernels.amd import group_gemm_gated, sort_topk_ids_align_block_size
    announce("group gemm argument checks")
    ids = torch.zeros((64, 2), dtype=torch.int64, device=cuda)
    s, e, bb, rb, pp = sort_topk_ids_align_block_size(ids, 4, 1, 64, 64)
    a = torch.zeros((64, 128), dtype=torch.bfloat16, device=cuda)
    b = torch.zeros((4, 64, 128), dtype=torch.bfloat16, device=cuda)
    c = torch.zeros((128, 64), dtype=torch.bfloat16, device=cuda)
    with pytest.raises(_lib.TdistError) as err:
        group_gemm_gated(a, None, 0, b, c, s, e, bb, pp, 64, 128, 2, 64, 0, None, 0)
    assert err.value.code == _lib.TDIST_ERR_UNSUPPORTED and "block_size" in str(err.value)
