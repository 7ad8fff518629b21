"""Grouped GEMM + top-k reduction + reduce-scatter (the second half of the MoE tensor-parallel layer) on the GPU
against the fp32 restatement of the reference's own golden (test/nvidia/test_moe_reduce_rs.py:103-133).
Bar: exact on integer-valued inputs and weights; max relative error <= 2e-2 on random inputs (three bf16 roundings:
GEMM rows, token sums, the reduced slice; the reference's test asks for atol = rtol = 1e-2 on fp16, :241-247)."""
import pytest
import torch

from oracle import golden
from tests.conftest import announce

pytestmark = pytest.mark.gpu


def make_ctx(cuda, world, rank, mpr, hidden, E, topk, block, logits, in_dtype=torch.bfloat16):
    from triton_dist.kernels.amd.moe_reduce_rs import create_moe_rs_context
    return create_moe_rs_context(None, rank, world, world, world * mpr, hidden, E, topk, in_dtype, torch.bfloat16, cuda, block,
                                 logits[rank].to(cuda), peer_router_logits={r: l.to(cuda) for r, l in enumerate(logits) if r != rank})


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float8_e4m3fn])
@pytest.mark.parametrize("block", [128, 256])
def test_exact_on_integer_inputs(cuda, dtype, block):
    from triton_dist.kernels.amd.moe_reduce_rs import moe_reduce_rs
    world, mpr, K, hidden, E, topk = 4, 80, 128, 328, 6, 2
    announce("moe reduce-rs exact %s block %d" % (dtype, block))
    g = torch.Generator().manual_seed(block)
    logits = [torch.randn((mpr, E), generator=g) for _ in range(world)]
    states = torch.randint(-1, 2, (world * mpr * topk, K), generator=g).float().to(dtype)
    w = torch.randint(-1, 2, (E, K, hidden), generator=g).float().to(dtype)
    for rank in (0, 2):
        ctx = make_ctx(cuda, world, rank, mpr, hidden, E, topk, block, logits)
        weight = torch.randint(1, 3, (world * mpr, topk), generator=g).float()
        ctx.topk_weight_f32 = weight.to(cuda)
        peers = [torch.randint(-8, 9, (mpr, hidden), generator=g).to(torch.bfloat16) for _ in range(world)]
        ctx.set_peer_partials({r: p.to(cuda) for r, p in enumerate(peers)})
        ctx.final_output_buffer.view(torch.uint8).fill_(0x7B)
        out = moe_reduce_rs(rank, world, world, states.to(cuda), w.to(cuda), ctx)
        torch.cuda.synchronize()
        ref = golden.torch_group_gemm_reduce_rs(states, w, ctx.precompute_ctx.full_topk_ids.cpu(), weight, peers, rank, world)
        assert ref.abs().max() <= 256      # every value is an integer that bf16 holds
        assert torch.equal(out.float().cpu(), ref), "rank %d" % rank


def test_random_inputs_and_the_routing(cuda):
    from triton_dist.kernels.amd.moe_reduce_rs import moe_reduce_rs
    world, mpr, K, hidden, E, topk, rank = 8, 128, 512, 1024, 16, 4, 5
    announce("moe reduce-rs random")
    g = torch.Generator().manual_seed(77)
    logits = [torch.randn((mpr, E), generator=g) for _ in range(world)]
    states = torch.randn((world * mpr * topk, K), generator=g).to(torch.bfloat16)
    w = (torch.randn((E, hidden, K), generator=g) * 0.05).to(torch.bfloat16).transpose(1, 2)    # [E, K, hidden], K contiguous
    ctx = make_ctx(cuda, world, rank, mpr, hidden, E, topk, 128, logits)
    # the routing is softmax + top-k of the ranks' logits in rank order (reference :180-197)
    score = torch.softmax(torch.cat(logits), dim=-1)
    want_w, want_ids = torch.topk(score, topk)
    assert torch.equal(ctx.precompute_ctx.full_topk_ids.cpu().long(), want_ids)
    assert torch.allclose(ctx.precompute_ctx.full_topk_weight.float().cpu(), want_w, atol=4e-3)
    peers = [torch.randn((mpr, hidden), generator=g).to(torch.bfloat16) for _ in range(world)]
    ctx.set_peer_partials({r: p.to(cuda) for r, p in enumerate(peers)})
    out = moe_reduce_rs(rank, world, world, states.to(cuda), w.to(cuda), ctx)
    torch.cuda.synchronize()
    ref = golden.torch_group_gemm_reduce_rs(states, w, want_ids, ctx.topk_weight_f32.cpu(), peers, rank, world)
    err = (out.float().cpu() - ref).abs().max() / ref.abs().max()
    assert err <= 2e-2, err
    # a second call on the same context, smaller routing weights: nothing of the first call may remain
    ctx.topk_weight_f32.mul_(0.5)
    out2 = moe_reduce_rs(rank, world, world, states.to(cuda), w.to(cuda), ctx)
    ref2 = golden.torch_group_gemm_reduce_rs(states, w, want_ids, ctx.topk_weight_f32.cpu(), peers, rank, world)
    assert (out2.float().cpu() - ref2).abs().max() / ref2.abs().max() <= 2e-2


def test_argument_errors(cuda):
    from triton_dist.kernels.amd.moe_reduce_rs import create_moe_rs_context, select_experts
    logits = torch.randn((16, 4), device=cuda)
    with pytest.raises(RuntimeError, match="missing rank 1"):
        select_experts(None, 2, 2, torch.bfloat16, cuda, logits)
    with pytest.raises(NotImplementedError):
        create_moe_rs_context(None, 0, 1, 1, 16, 64, 4, 2, torch.float16, torch.float16, cuda, 128, logits)
