"""Split last round of the GEMM entry points (the tiles of a round that fills at most half of the grid are cut along
K into 2, 4 or 8 equal pieces, one per workgroup; the pieces go through the caller's workspace and every workgroup adds
up and stores its share of the tile) against the oracle and against the whole-tile form.
Bar: exact on integer-valued inputs (every partial sum is an integer that fp32 holds), max relative error <= 1e-2 on
random inputs; a piece that never arrives ends in TDIST_ERR_TIMEOUT, not in a hang."""

import pytest
import torch

from oracle import golden
from tests.conftest import announce

pytestmark = pytest.mark.gpu


@pytest.fixture
def split_k(cuda, switches):
    """A workspace of this test's own, with the split forced wherever it is possible (whatever the cost estimate says)."""
    from triton_dist import _lib
    ws = _lib.new_split_k_workspace()
    switches(_lib.TDIST_DEBUG_GEMM_SPLIT_K, 1)
    yield ws


def ints(shape, g, dtype, lo=-2, hi=3):
    return torch.randint(lo, hi, shape, generator=g).float().to(dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float8_e4m3fn])
@pytest.mark.parametrize("M,N,K,wgs", [(1024, 768, 1024, 40), (1024, 768, 1024, 24), (1024, 768, 1024, 7), (512, 640, 2048, 256),
                                       (1280, 768, 1024, 12), (384, 200, 1088, 13)])
def test_exact_on_integer_inputs(cuda, split_k, dtype, M, N, K, wgs):
    """12 tiles on 40 workgroups and on 24 (two pieces each); on 7 (a last round of 5 that is not split); 6 tiles on
    256 workgroups (eight pieces each); a whole round of 12 followed by 3 tiles in four pieces each; a ragged shape on
    the 128 x 128 tile (6 tiles on 13 workgroups: two pieces each)."""
    from triton_dist.kernels.amd import gated_gemm
    announce("split-k exact %s %dx%dx%d wgs %d" % (dtype, M, N, K, wgs))
    g = torch.Generator().manual_seed(M + N + wgs)
    a, b = ints((M, K), g, dtype), ints((N, K), g, dtype)
    out_dtype = torch.bfloat16 if dtype == torch.float8_e4m3fn else dtype
    c = torch.full((M, N), float("nan"), dtype=out_dtype, device=cuda)
    status = torch.zeros(2, dtype=torch.int32, device=cuda)
    gated_gemm(a.to(cuda), None, 0, b.to(cuda), c, None, 0, 0, 1, status=status, max_workgroups=wgs, sk_workspace=split_k)
    torch.cuda.synchronize()
    assert status.tolist() == [0, 0]
    ref = (a.float() @ b.float().T).to(out_dtype)
    assert torch.equal(c.cpu(), ref)


def test_exchange_within_an_xcd_and_through_memory_agree(cuda, split_k, switches):
    """The pieces of a tile exchange their partial sums through the L2 of the XCD they share (only where tdist_init has
    seen workgroup i land on XCD i mod 8: on this device it must have) or through device-coherent stores (forced here
    through the library's switch): the same bits either way, exact on integer-valued inputs, and no piece reports a
    partner on another XCD."""
    from triton_dist import _lib
    from triton_dist.kernels.amd import gated_gemm
    M, N, K = 512, 640, 2048          # 6 tiles of 256 x 256 on 256 workgroups: eight pieces each, all on one XCD
    announce("split-k exchange paths %dx%dx%d" % (M, N, K))
    g = torch.Generator().manual_seed(77)
    a, b = ints((M, K), g, torch.bfloat16), ints((N, K), g, torch.bfloat16)
    ref = (a.float() @ b.float().T).to(torch.bfloat16)
    outs = []
    for coherent in (0, 1, 0):
        switches(_lib.TDIST_DEBUG_GEMM_SK_COHERENT, coherent)
        c = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=cuda)
        status = torch.zeros(2, dtype=torch.int32, device=cuda)
        gated_gemm(a.to(cuda), None, 0, b.to(cuda), c, None, 0, 0, 1, status=status, sk_workspace=split_k)
        torch.cuda.synchronize()
        assert status.tolist() == [0, 0], "a piece found its partner on another XCD (or timed out): %s" % status.tolist()
        assert torch.equal(c.cpu(), ref)
        outs.append(c)
    assert int(split_k.view(torch.int32)[0]) != 0   # (the split form really ran: the workspace's epoch word has moved)


def test_random_inputs_match_the_whole_tile_form(cuda, split_k):
    from triton_dist.kernels.amd import gated_gemm
    M, N, K = 2048, 1536, 4096
    announce("split-k random %dx%dx%d" % (M, N, K))
    g = torch.Generator().manual_seed(5)
    a = torch.randn((M, K), generator=g).to(torch.bfloat16)
    b = (torch.randn((N, K), generator=g) * 0.02).to(torch.bfloat16)
    c_sk = torch.empty((M, N), dtype=torch.bfloat16, device=cuda)
    c_dp = torch.empty_like(c_sk)
    gated_gemm(a.to(cuda), None, 0, b.to(cuda), c_sk, None, 0, 0, 1, sk_workspace=split_k)
    gated_gemm(a.to(cuda), None, 0, b.to(cuda), c_dp, None, 0, 0, 1)          # no workspace: whole tiles
    torch.cuda.synchronize()
    ref = a.float() @ b.float().T
    assert golden.max_rel_err(c_sk.float().cpu(), ref) <= 1e-2
    # the two forms add the same products in another order: a few results differ by one rounding step of bf16
    assert golden.max_rel_err(c_sk.float().cpu(), c_dp.float().cpu()) <= 1e-2
    # launch after launch on the same workspace (new tags each time): nothing of an earlier launch is taken, and
    # the sum does not depend on which workgroup finishes first
    for _ in range(3):
        c2 = torch.empty_like(c_sk)
        gated_gemm(a.to(cuda), None, 0, b.to(cuda), c2, None, 0, 0, 1, sk_workspace=split_k)
        assert torch.equal(c2, c_sk)


def test_scaled_fp8_and_gated_chunks(cuda, split_k):
    """Row and column scales in the epilogue of the workgroup that adds the pieces; chunk flags on the pieces."""
    from triton_dist.kernels.amd import gated_gemm
    M, N, K, world = 1024, 512, 2048, 4
    announce("split-k fp8 scales + flags")
    g = torch.Generator().manual_seed(6)
    a, b = ints((M, K), g, torch.float8_e4m3fn), ints((N, K), g, torch.float8_e4m3fn)
    sa = (2.0 ** torch.randint(-3, 3, (M, ), generator=g)).float()
    sb = (2.0 ** torch.randint(-3, 3, (N, ), generator=g)).float()
    c = torch.empty((M, N), dtype=torch.bfloat16, device=cuda)
    flags = torch.ones(world, dtype=torch.int32, device=cuda)
    status = torch.zeros(2, dtype=torch.int32, device=cuda)
    gated_gemm(a.to(cuda), None, 0, b.to(cuda), c, flags, M // world, 1, world, row_scale=sa.to(cuda), col_scale=sb.to(cuda),
               status=status, max_workgroups=24, sk_workspace=split_k)
    torch.cuda.synchronize()
    assert status.tolist() == [0, 0]
    ref = ((a.float() @ b.float().T) * sa[:, None] * sb[None, :]).to(torch.bfloat16)
    assert torch.equal(c.cpu(), ref)


def test_a_chunk_that_never_arrives_times_out(cuda, split_k):
    from triton_dist import _lib
    from triton_dist.kernels.amd import gated_gemm
    M, N, K, world = 1024, 512, 2048, 4
    announce("split-k held chunk")
    g = torch.Generator().manual_seed(7)
    a, b = ints((M, K), g, torch.bfloat16), ints((N, K), g, torch.bfloat16)
    c = torch.zeros((M, N), dtype=torch.bfloat16, device=cuda)
    flags = torch.ones(world, dtype=torch.int32, device=cuda)
    flags[2] = 0
    status = torch.zeros(2, dtype=torch.int32, device=cuda)
    gated_gemm(a.to(cuda), None, 0, b.to(cuda), c, flags, M // world, 0, world, status=status, spin_limit=200, max_workgroups=24,
               sk_workspace=split_k)
    torch.cuda.synchronize()
    assert status[0].item() == _lib.TDIST_ERR_TIMEOUT
    ref = (a.float() @ b.float().T).to(torch.bfloat16)
    rows = M // world
    for ch in (0, 1, 3):   # the chunks that did arrive are complete
        assert torch.equal(c[ch * rows:(ch + 1) * rows].cpu(), ref[ch * rows:(ch + 1) * rows]), ch
    assert (c[2 * rows:3 * rows] == 0).all()          # the rows of the chunk that never came are left alone
    # the workspace stays usable after a launch that timed out
    flags[2] = 1
    status.zero_()
    gated_gemm(a.to(cuda), None, 0, b.to(cuda), c, flags, M // world, 0, world, status=status, spin_limit=200, max_workgroups=24,
               sk_workspace=split_k)
    torch.cuda.synchronize()
    assert status.tolist() == [0, 0] and torch.equal(c.cpu(), ref)


def test_gemm_rs_scatter_and_grouped_forms(cuda, split_k):
    from triton_dist.kernels.amd import create_gemm_rs_intra_node_context, gemm_rs_intra_node
    from tests.test_gpu_group_gemm import make_case, run
    announce("split-k gemm-rs")
    W, rank, M, N, K = 4, 1, 1024, 768, 2048
    g = torch.Generator().manual_seed(8)
    a, b = ints((M, K), g, torch.bfloat16, -1, 2), ints((N, K), g, torch.bfloat16, -1, 2)
    peers = [None if r == rank else ints((M // W, N), g, torch.bfloat16) for r in range(W)]
    ctx = create_gemm_rs_intra_node_context(M, N, torch.bfloat16, rank, W, None)
    ctx.set_peer_partials(peers)
    out = gemm_rs_intra_node(a.to(cuda), b.to(cuda), ctx)
    torch.cuda.synchronize()
    ref = golden.gemm_rs_fp32(a, b, peers, rank, W).to(torch.bfloat16)
    assert torch.equal(out.cpu(), ref)
    announce("split-k grouped")
    world, mpr, K, N, E, topk = 4, 96, 2048, 328, 6, 2
    for dtype, block in ((torch.bfloat16, 128), (torch.float8_e4m3fn, 256)):
        shards, w, ids = make_case(world, mpr, K, N, E, topk, dtype, seed=block, integer=True)
        ctx, c = run(cuda, shards, w, ids, 2, E, block)
        ctx.check_status()
        ref = golden.ag_group_gemm_fp32(shards, w, ids)
        assert torch.equal(c.float().cpu(), ref.to(c.dtype).float()), (dtype, block)


def test_graph_replay_with_new_inputs(cuda, split_k):
    """Every replay of a captured launch takes fresh tags from the workspace: a replay on new operands must not see
    anything of the one before."""
    from triton_dist.kernels.amd import gated_gemm
    M, N, K, wgs = 1024, 768, 1024, 40
    announce("split-k graph replay")
    g = torch.Generator().manual_seed(11)
    a_d = torch.empty((M, K), dtype=torch.bfloat16, device=cuda)
    b_d = torch.empty((N, K), dtype=torch.bfloat16, device=cuda)
    c = torch.empty((M, N), dtype=torch.bfloat16, device=cuda)
    status = torch.zeros(2, dtype=torch.int32, device=cuda)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        gated_gemm(a_d, None, 0, b_d, c, None, 0, 0, 1, status=status, max_workgroups=wgs, sk_workspace=split_k)   # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        gated_gemm(a_d, None, 0, b_d, c, None, 0, 0, 1, status=status, max_workgroups=wgs, sk_workspace=split_k,
                   stream=torch.cuda.current_stream())
    torch.cuda.synchronize()
    for replay in range(4):
        a, b = ints((M, K), g, torch.bfloat16), ints((N, K), g, torch.bfloat16)
        a_d.copy_(a)
        b_d.copy_(b)
        c.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert status.tolist() == [0, 0]
        assert torch.equal(c.cpu(), (a.float() @ b.float().T).to(torch.bfloat16)), "replay %d" % replay
    # and an eager launch afterwards on the same workspace
    gated_gemm(a_d, None, 0, b_d, c, None, 0, 0, 1, status=status, max_workgroups=wgs, sk_workspace=split_k)
    torch.cuda.synchronize()
    assert torch.equal(c.cpu(), (a.float() @ b.float().T).to(torch.bfloat16))


def test_two_launches_in_flight_on_two_streams(cuda, split_k):
    """Two split GEMMs at the same time on two streams, each with a workspace of its own: no state is shared."""
    from triton_dist import _lib
    from triton_dist.kernels.amd import gated_gemm
    announce("split-k two streams")
    M, N, K, wgs = 1024, 768, 2048, 40
    g = torch.Generator().manual_seed(13)
    cases = []
    for i in range(2):
        a, b = ints((M, K), g, torch.bfloat16), ints((N, K), g, torch.bfloat16)
        cases.append((a, b, a.to(cuda), b.to(cuda), torch.empty((M, N), dtype=torch.bfloat16, device=cuda),
                      torch.zeros(2, dtype=torch.int32, device=cuda), torch.cuda.Stream(),
                      split_k if i == 0 else _lib.new_split_k_workspace()))
    torch.cuda.synchronize()
    for rep in range(5):
        for a, b, a_d, b_d, c, status, stream, ws in cases:
            gated_gemm(a_d, None, 0, b_d, c, None, 0, 0, 1, status=status, max_workgroups=wgs, sk_workspace=ws, stream=stream)
    torch.cuda.synchronize()
    for a, b, a_d, b_d, c, status, stream, ws in cases:
        assert status.tolist() == [0, 0]
        assert torch.equal(c.cpu(), (a.float() @ b.float().T).to(torch.bfloat16))


def test_workspace_argument_errors(cuda):
    from triton_dist import _lib
    from triton_dist.kernels.amd import gated_gemm
    lib = _lib.load()
    need = lib.tdist_gemm_split_k_workspace_bytes()
    assert need == 12288 + lib.tdist_num_cus() * 256 * 256 * 4
    a = torch.zeros((128, 64), dtype=torch.bfloat16, device=cuda)
    c = torch.zeros((128, 128), dtype=torch.bfloat16, device=cuda)
    buf = torch.zeros(1 << 20, dtype=torch.uint8, device=cuda)
    with pytest.raises(_lib.TdistError) as e:
        gated_gemm(a, None, 0, a, c, None, 0, 0, 1, sk_workspace=buf[16:])            # misaligned
    assert e.value.code == _lib.TDIST_ERR_WORKSPACE
    with pytest.raises(_lib.TdistError) as e:
        gated_gemm(a, None, 0, a, c, None, 0, 0, 1, sk_workspace=buf[:4096])          # smaller than the header
    assert e.value.code == _lib.TDIST_ERR_WORKSPACE
    gated_gemm(a, None, 0, a, c, None, 0, 0, 1, sk_workspace=buf)                     # too small for a round: left unused
    torch.cuda.synchronize()
