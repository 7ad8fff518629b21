"""(a)/(b1) chunk-gated GEMM and the GEMM-RS scatter GEMM on the GPU against the oracle.
Bar: max relative error <= 1e-2 against the fp32 reference; exact on integer-valued inputs; gating checked
through host-forced conditions (held flags with a tiny spin limit, shuffled arrival, poisoned workspace)."""
import itertools

import numpy as np
import pytest
import torch

from oracle import cref, golden
from tests.conftest import announce

pytestmark = pytest.mark.gpu


def plain_gemm(a, b, out_dtype, cuda, row_scale=None, col_scale=None):
    from triton_dist.kernels.amd import gated_gemm
    c = torch.full((a.shape[0], b.shape[0]), float("nan"), dtype=out_dtype, device=cuda)
    gated_gemm(a.to(cuda), None, 0, b.to(cuda), c, None, 0, 0, 1,
               row_scale=None if row_scale is None else row_scale.to(cuda),
               col_scale=None if col_scale is None else col_scale.to(cuda))
    torch.cuda.synchronize()
    return c.cpu()


@pytest.mark.parametrize("M,N,K", [(128, 128, 64), (256, 128, 128), (200, 72, 96), (1, 1, 32), (130, 257, 64), (512, 384, 256)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_small_gemm_exact_on_integer_inputs(cuda, M, N, K, dtype):
    announce("gemm exact M=%d N=%d K=%d %s" % (M, N, K, dtype))
    g = torch.Generator().manual_seed(M + N + K)
    a = torch.randint(-3, 4, (M, K), generator=g).to(dtype)
    b = torch.randint(-3, 4, (N, K), generator=g).to(dtype)
    want = torch.from_numpy(cref.gemm_nt_f64(a.float().numpy(), b.float().numpy()))   # |entries| <= 9*K < 2^8 * 16: check range
    got = plain_gemm(a, b, dtype, cuda)
    assert not torch.isnan(got.float()).any(), "part of C was not written"
    assert torch.equal(got.double(), want.to(dtype).double())


@pytest.mark.parametrize("M,N,K", [(128, 128, 64), (200, 72, 128), (256, 256, 256), (64, 48, 192)])
def test_small_fp8_gemm_exact_and_scaled(cuda, M, N, K):
    announce("fp8 gemm M=%d N=%d K=%d" % (M, N, K))
    g = torch.Generator().manual_seed(M * 7 + K)
    a = torch.randint(-2, 3, (M, K), generator=g).float().to(torch.float8_e4m3fn)
    b = torch.randint(-2, 3, (N, K), generator=g).float().to(torch.float8_e4m3fn)
    want = cref.gemm_e4m3_nt_f64(a.view(torch.uint8).numpy(), b.view(torch.uint8).numpy(), None, None)
    got = plain_gemm(a, b, torch.bfloat16, cuda)
    assert torch.equal(got.double(), torch.from_numpy(want).to(torch.bfloat16).double())
    # random e4m3 data with scales: closed form, <= 1e-2 relative
    a = torch.randn((M, K), generator=g).to(torch.float8_e4m3fn)
    b = torch.randn((N, K), generator=g).to(torch.float8_e4m3fn)
    sa = torch.rand(M, generator=g) * 0.09 + 0.01
    sb = torch.rand(N, generator=g) * 0.009 + 0.001
    ref = golden.fp8_scaled_gemm_fp32(a, sa, b, sb)
    got = plain_gemm(a, b, torch.bfloat16, cuda, sa, sb)
    assert golden.max_rel_err(got.float(), ref) <= 1e-2
    assert torch.allclose(got.float(), ref, rtol=2.0**-7, atol=1e-6)   # nothing but the bf16 rounding of C


def make_ag_case(world, m_per_rank, K, N, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    if dtype == torch.float8_e4m3fn:
        shards = [torch.randn((m_per_rank, K), generator=g).to(dtype) for _ in range(world)]
        b = torch.randn((N, K), generator=g).to(dtype)
    else:
        shards = [torch.randn((m_per_rank, K), generator=g).to(dtype) for _ in range(world)]
        b = (torch.randn((N, K), generator=g) * 0.02).to(dtype)
    return shards, b


def run_ag_gemm(cuda, shards, b, rank, m_per_chunk, **ctx_kw):
    from triton_dist.kernels.amd import ag_gemm_intra_node, create_ag_gemm_intra_node_context
    world = len(shards)
    m_per_rank, K = shards[0].shape
    ctx = create_ag_gemm_intra_node_context(world * m_per_rank, b.shape[0], K, shards[0].dtype, torch.bfloat16, rank, world,
                                            None, M_PER_CHUNK=m_per_chunk)
    for k, v in ctx_kw.items():
        setattr(ctx, k, v)
    ctx.set_peer_shards({r: s.to(cuda) for r, s in enumerate(shards) if r != rank})
    # garbage in the workspace must never leak into C (test/nvidia/test_ag_gemm_intra_node.py:122-127)
    ctx.workspace_tensors[rank].view(torch.uint8).fill_(0x7B)
    return ctx


def test_ag_gemm_config1(cuda):
    """BASELINE config 1: 4 chunks of [1024, 4096] bf16, B [1536, 4096], flags released by the copy streams."""
    from triton_dist.kernels.amd import ag_gemm_intra_node
    announce("ag_gemm C1")
    shards, b = make_ag_case(4, 1024, 4096, 1536, torch.bfloat16, seed=3 + 0)
    ref = golden.ag_gemm_fp32(shards, b)
    gold = golden.torch_ag_gemm(shards, b)
    for rank, order in [(0, None), (2, [(3, 0), (1, 0), (0, 0)])]:
        ctx = run_ag_gemm(cuda, shards, b, rank, 1024, arrival_order=order)
        for it in range(2):   # flags are reset between calls
            c = ag_gemm_intra_node(shards[rank].to(cuda), b.to(cuda), False, ctx)
            ctx.check_status()
            assert c.shape == (4096, 1536) and c.dtype == torch.bfloat16
            assert golden.max_rel_err(c.float().cpu(), ref) <= 1e-2
            torch.testing.assert_close(c.cpu().float(), gold.float(), atol=1e-2, rtol=1e-2)   # test_ag_gemm_intra_node.py:257
            assert int(ctx.barrier_tensors[rank].abs().sum()) == 0


def test_ag_gemm_copy_engine_option(cuda):
    """The chunk copies on the copy engines (hipMemcpyDeviceToDeviceNoCU), flags still published after the data."""
    from triton_dist.kernels.amd import ag_gemm_intra_node
    announce("ag_gemm use_sdma")
    shards, b = make_ag_case(4, 512, 1024, 768, torch.bfloat16, seed=17)
    ref = golden.ag_gemm_fp32(shards, b)
    rank = 1
    ctx = run_ag_gemm(cuda, shards, b, rank, 256, use_sdma=True)
    for _ in range(2):
        c = ag_gemm_intra_node(shards[rank].to(cuda), b.to(cuda), False, ctx)
        ctx.check_status()
        assert golden.max_rel_err(c.float().cpu(), ref) <= 1e-2


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float8_e4m3fn])
def test_ag_gemm_any_arrival_order(cuda, dtype):
    """Result independent of the order in which chunks arrive: all 3! orders of the peers of rank 1, two chunks each."""
    from triton_dist.kernels.amd import ag_gemm_intra_node
    announce("ag_gemm arrival orders %s" % dtype)
    world, rank, m_per_rank, mpc, K, N = 4, 1, 256, 128, 256, 384
    shards, b = make_ag_case(world, m_per_rank, K, N, dtype, seed=11)
    if dtype == torch.float8_e4m3fn:
        ref = golden.fp8_scaled_gemm_fp32(torch.cat(shards), None, b, None)
    else:
        ref = golden.ag_gemm_fp32(shards, b)
    first = None
    for perm in itertools.permutations([0, 2, 3]):
        order = [(r, c) for c in (1, 0) for r in perm]
        ctx = run_ag_gemm(cuda, shards, b, rank, mpc, arrival_order=order)
        c = ag_gemm_intra_node(shards[rank].to(cuda), b.to(cuda), False, ctx)
        ctx.check_status()
        assert golden.max_rel_err(c.float().cpu(), ref) <= 1e-2
        if first is None:
            first = c.clone()
        assert torch.equal(first, c), "output depends on the arrival order"


def test_gate_holds_and_times_out(cuda):
    """A chunk whose flag is never released: with a small spin limit the call reports TDIST_ERR_TIMEOUT, the rows
    of that chunk stay untouched and every other row is correct (the 1-GPU pattern of test_distributed_wait.py:206-243)."""
    from triton_dist import _lib
    from triton_dist.kernels.amd import gated_gemm
    announce("gate timeout")
    M, N, K, mpc = 1024, 256, 128, 256
    g = torch.Generator().manual_seed(5)
    a = torch.randn((M, K), generator=g).to(torch.bfloat16)
    b = (torch.randn((N, K), generator=g) * 0.02).to(torch.bfloat16)
    flags = torch.tensor([1, 1, 0, 1], dtype=torch.int32, device=cuda)
    status = torch.zeros(2, dtype=torch.int32, device=cuda)
    c = torch.full((M, N), -7.0, dtype=torch.bfloat16, device=cuda)
    gated_gemm(a.to(cuda), None, 0, b.to(cuda), c, flags, mpc, 0, 1, spin_limit=50, status=status)
    torch.cuda.synchronize()
    assert status.tolist() == [_lib.TDIST_ERR_TIMEOUT, 2]
    ref = golden.ag_gemm_fp32([a], b)
    got = c.float().cpu()
    assert (got[512:768] == -7.0).all(), "rows of the held chunk were written"
    keep = torch.ones(M, dtype=torch.bool)
    keep[512:768] = False
    assert golden.max_rel_err(got[keep], ref[keep]) <= 1e-2
    # released later (wait_value 1 present from the start this time): complete result
    status.zero_()
    flags.fill_(1)
    gated_gemm(a.to(cuda), None, 0, b.to(cuda), c, flags, mpc, 0, 1, spin_limit=50, status=status)
    torch.cuda.synchronize()
    assert status.tolist() == [0, 0]
    assert golden.max_rel_err(c.float().cpu(), ref) <= 1e-2


def test_a_timeout_slows_down_one_call_and_is_not_forgotten(cuda):
    """The op after a call whose flag wait expired runs normally (the status words are retired in front of every
    launch: an expired wait makes the waits of ITS launch give up at once, not those of the next), and check_status
    still reports the first expired wait, however many calls followed; tdist_status_retire by itself on the C-ABI."""
    from triton_dist import _lib
    from triton_dist.kernels.amd import ag_gemm_intra_node, create_ag_gemm_intra_node_context
    announce("ag-gemm timeout retired by the next call")
    world, rank, mpr, K, N = 4, 0, 256, 256, 384
    shards, b = make_ag_case(world, mpr, K, N, torch.bfloat16, seed=17)
    ctx = create_ag_gemm_intra_node_context(world * mpr, N, K, torch.bfloat16, torch.bfloat16, rank, world, None, M_PER_CHUNK=256)
    ctx.set_peer_shards({r: s.to(cuda) for r, s in enumerate(shards) if r != rank})
    a_d, b_d = shards[rank].to(cuda), b.to(cuda)
    ref = golden.ag_gemm_fp32(shards, b)
    ctx.held_chunks, ctx.spin_limit = (2, ), 200
    ag_gemm_intra_node(a_d, b_d, False, ctx)
    torch.cuda.synchronize()
    assert ctx.status.tolist()[:2] == [_lib.TDIST_ERR_TIMEOUT, 2]
    ctx.held_chunks, ctx.spin_limit = (), 0
    for _ in range(2):
        c = ag_gemm_intra_node(a_d, b_d, False, ctx)
        torch.cuda.synchronize()
        assert golden.max_rel_err(c.float().cpu(), ref) <= 1e-2
        assert ctx.status.tolist() == [0, 0, _lib.TDIST_ERR_TIMEOUT, 2]
    with pytest.raises(_lib.TdistError, match="chunk 2"):
        ctx.check_status()
    assert ctx.status.tolist() == [0, 0, 0, 0]
    ctx.check_status()
    # the entry point: a later error does not replace the first one; a null first_error drops the status
    words = torch.tensor([_lib.TDIST_ERR_TIMEOUT, 5, _lib.TDIST_ERR_TIMEOUT, 2], dtype=torch.int32, device=cuda)
    _lib.call("tdist_status_retire", words.data_ptr(), words.data_ptr() + 8, None)
    torch.cuda.synchronize()
    assert words.tolist() == [0, 0, _lib.TDIST_ERR_TIMEOUT, 2]
    words[0], words[1] = 7, 9
    _lib.call("tdist_status_retire", words.data_ptr(), None, None)
    torch.cuda.synchronize()
    assert words.tolist() == [0, 0, _lib.TDIST_ERR_TIMEOUT, 2]


def test_gate_released_by_a_stream_while_the_gemm_waits(cuda):
    """Flags are set by a second stream while the GEMM waits for them (explicit chunk order, last chunk first)."""
    from triton_dist import _lib
    from triton_dist.kernels.amd import gated_gemm
    from triton_dist.kernels.amd.common_ops import set_signal
    announce("gate released late")
    M, N, K, mpc = 1024, 256, 256, 256
    g = torch.Generator().manual_seed(6)
    a = torch.randn((M, K), generator=g).to(torch.bfloat16)
    b = (torch.randn((N, K), generator=g) * 0.02).to(torch.bfloat16)
    flags = torch.zeros(4, dtype=torch.int32, device=cuda)
    status = torch.zeros(2, dtype=torch.int32, device=cuda)
    order = torch.tensor([3, 1, 0, 2], dtype=torch.int32, device=cuda)
    c = torch.empty((M, N), dtype=torch.bfloat16, device=cuda)
    a_dev, b_dev = a.to(cuda), b.to(cuda)
    side = torch.cuda.Stream()
    stamp = torch.zeros(1, dtype=torch.int64, device=cuda)
    torch.cuda.synchronize()
    # The releases are queued BEFORE the GEMM (work queued behind a spinning GEMM may share its hardware queue and never
    # run) and held back on the device: a one-wave kernel sleeps 300 us past the stamp before the flags are set.
    _lib.call("tdist_producer_mark", stamp.data_ptr(), side.cuda_stream)
    _lib.call("tdist_producer_wait_until", stamp.data_ptr(), 300000, side.cuda_stream)
    for chunk in (3, 1, 0, 2):
        set_signal(flags.data_ptr() + 4 * chunk, 1, side)
    gated_gemm(a_dev, None, 0, b_dev, c, flags, mpc, 0, 1, chunk_order=order, status=status)
    torch.cuda.synchronize()
    assert status.tolist() == [0, 0]
    assert golden.max_rel_err(c.float().cpu(), golden.ag_gemm_fp32([a], b)) <= 1e-2


@pytest.mark.parametrize("schedule", ["arrival", "static"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float8_e4m3fn])
def test_tiles_in_arrival_order(cuda, switches, schedule, dtype):
    """More than one round of tiles (384 tiles of 256 x 256 on 256 workgroups), so that a gated call's workgroups take
    their tiles in the order in which the chunks arrive: flags released late and out of the expected order by a second
    stream, a straggler behind the kernel producer, and a chunk that never arrives (every other row right, the held
    chunk's rows untouched, TDIST_ERR_TIMEOUT naming it, and the next launch clean). The static order, forced through
    the library's switch, must give the same bits."""
    from triton_dist import _lib
    from triton_dist.kernels.amd import ag_gemm_intra_node, create_ag_gemm_intra_node_context, gated_gemm
    from triton_dist.kernels.amd.common_ops import set_signal
    announce("gemm tiles in %s order %s" % (schedule, dtype))
    if schedule == "static":
        switches(_lib.TDIST_DEBUG_GEMM_SCHEDULE, 0)
    world, mpc, N, K = 8, 512, 6144, 256
    M = world * mpc
    g = torch.Generator().manual_seed(31)
    a = torch.randint(-2, 3, (M, K), generator=g).float()
    b = torch.randint(-2, 3, (N, K), generator=g).float()
    want = golden.ag_gemm_fp32([a], b).to(torch.bfloat16)
    a_d, b_d = a.to(dtype).to(cuda), b.to(dtype).to(cuda)
    ws = _lib.new_split_k_workspace(cuda)
    status = torch.zeros(2, dtype=torch.int32, device=cuda)
    # (1) flags released 200 us into the launch, last chunk first, by a second stream (queued before the GEMM)
    flags = torch.zeros(world, dtype=torch.int32, device=cuda)
    flags[3] = 1
    c = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=cuda)
    side = torch.cuda.Stream()
    stamp = torch.zeros(1, dtype=torch.int64, device=cuda)
    torch.cuda.synchronize()
    _lib.call("tdist_producer_mark", stamp.data_ptr(), side.cuda_stream)
    _lib.call("tdist_producer_wait_until", stamp.data_ptr(), 200000, side.cuda_stream)
    for chunk in (7, 6, 5, 4, 2, 1, 0):
        set_signal(flags.data_ptr() + 4 * chunk, 1, side)
    gated_gemm(a_d, None, 0, b_d, c, flags, mpc, 3, world, status=status, sk_workspace=ws)
    torch.cuda.synchronize()
    assert status.tolist() == [0, 0]
    assert torch.equal(c.cpu(), want)
    # (2) a chunk that never arrives
    flags.fill_(1)
    flags[5] = 0
    c.fill_(-7.0)
    gated_gemm(a_d, None, 0, b_d, c, flags, mpc, 3, world, spin_limit=50, status=status, sk_workspace=ws)
    torch.cuda.synchronize()
    assert status.tolist() == [_lib.TDIST_ERR_TIMEOUT, 5]
    got = c.cpu()
    assert (got[5 * mpc:6 * mpc] == -7.0).all(), "rows of the held chunk were written"
    keep = torch.ones(M, dtype=torch.bool)
    keep[5 * mpc:6 * mpc] = False
    assert torch.equal(got[keep], want[keep])
    # the launch after the timeout is clean
    flags.fill_(1)
    status.zero_()
    gated_gemm(a_d, None, 0, b_d, c, flags, mpc, 3, world, status=status, sk_workspace=ws)
    torch.cuda.synchronize()
    assert status.tolist() == [0, 0] and torch.equal(c.cpu(), want)
    # (3) the op with the kernel producer and a straggler: rank 2's first chunk 300 us late, its second one behind it
    rank = 1
    shards = [a[r * mpc:(r + 1) * mpc] for r in range(world)]
    ctx = create_ag_gemm_intra_node_context(M, N, K, dtype, torch.bfloat16, rank, world, None, M_PER_CHUNK=256)
    ctx.set_peer_shards({r: s_.to(dtype).to(cuda) for r, s_ in enumerate(shards) if r != rank})
    ctx.producer_kernel, ctx.late_chunks_us = True, {2 * 2: 300}
    for _ in range(3):
        ctx.workspace_tensors[rank].view(torch.uint8).fill_(0x7B if dtype != torch.float8_e4m3fn else 0x7F)
        out = ag_gemm_intra_node(shards[rank].to(dtype).to(cuda), b_d, False, ctx)
        ctx.check_status()
        assert torch.equal(out.cpu(), want)


@pytest.mark.parametrize("max_workgroups,late", [(48, False), (48, True), (2, False), (2, True)])
def test_arrival_order_on_a_capped_grid(cuda, max_workgroups, late):
    """A grid held to a few workgroups: 96 tiles of 256 x 256 are 2 rounds on 48 workgroups (every workgroup takes its
    tiles in arrival order) and 48 rounds on 2; held to one workgroup they are more rounds than the schedule keeps
    track of, and the workgroup waits at each tile's flag in turn. With the flags up from the start and with all but
    the own chunk released late and last chunk first, against the oracle bit for bit."""
    from triton_dist import _lib
    from triton_dist.kernels.amd import gated_gemm
    from triton_dist.kernels.amd.common_ops import set_signal
    announce("gemm arrival order with %d workgroups, late=%s" % (max_workgroups, late))
    world, mpc, N, K, rank = 4, 512, 3072, 256, 1
    M = world * mpc
    g = torch.Generator().manual_seed(77)
    a = torch.randint(-2, 3, (M, K), generator=g).float()
    b = torch.randint(-2, 3, (N, K), generator=g).float()
    want = golden.ag_gemm_fp32([a], b).to(torch.bfloat16)
    a_d, b_d = a.to(torch.bfloat16).to(cuda), b.to(torch.bfloat16).to(cuda)
    for cap in (max_workgroups, 1):
        flags = torch.ones(world, dtype=torch.int32, device=cuda)
        c = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=cuda)
        status = torch.zeros(2, dtype=torch.int32, device=cuda)
        if late:
            flags.zero_()
            flags[rank] = 1
            side = torch.cuda.Stream()
            stamp = torch.zeros(1, dtype=torch.int64, device=cuda)
            torch.cuda.synchronize()
            _lib.call("tdist_producer_mark", stamp.data_ptr(), side.cuda_stream)
            _lib.call("tdist_producer_wait_until", stamp.data_ptr(), 100000, side.cuda_stream)
            for chunk in (3, 2, 0):
                set_signal(flags.data_ptr() + 4 * chunk, 1, side)
        gated_gemm(a_d, None, 0, b_d, c, flags, mpc, rank, world, status=status, max_workgroups=cap)
        torch.cuda.synchronize()
        assert status.tolist() == [0, 0], cap
        assert torch.equal(c.cpu(), want), cap


def test_gemm_rs_small_and_owner_mapping(cuda):
    from triton_dist.kernels.amd import create_gemm_rs_intra_node_context, gemm_rs_intra_node
    announce("gemm_rs small")
    W, rank, M, N, K = 4, 2, 1024, 512, 256
    g = torch.Generator().manual_seed(8)
    a = torch.randn((M, K), generator=g).to(torch.bfloat16)
    b = (torch.randn((N, K), generator=g) * 0.02).to(torch.bfloat16)
    m_per = M // W
    peers = [None if r == rank else torch.randn((m_per, N), generator=g).to(torch.bfloat16) for r in range(W)]
    ctx = create_gemm_rs_intra_node_context(M, N, torch.bfloat16, rank, W, None)
    ctx.set_peer_partials(peers)
    out = gemm_rs_intra_node(a.to(cuda), b.to(cuda), ctx)
    torch.cuda.synchronize()
    assert out.shape == (m_per, N)
    ref = golden.gemm_rs_fp32(a, b, peers, rank, W)
    assert golden.max_rel_err(out.float().cpu(), ref) <= 1e-2
    gold = golden.torch_gemm_rs(a, b, peers, rank, W)
    torch.testing.assert_close(out.float().cpu(), gold.float(), atol=1e-2, rtol=1e-2)   # test_gemm_rs_intra_node.py:261
    # epilogue placement (gemm_reduce_scatter.py:222-229): owner o's rows sit in scatter_bufs[o] at row block `rank`
    full = golden.ag_gemm_fp32([a], b)
    for o in range(W):
        blk = ctx.scatter_bufs[o][rank * m_per:(rank + 1) * m_per].float().cpu()
        assert golden.max_rel_err(blk, full[o * m_per:(o + 1) * m_per]) <= 1e-2, "owner %d" % o
    # the reduction is bit-exact given what the GEMM stored
    stored = ctx.scatter_bufs[rank][:M].cpu().view(W, m_per, N)
    assert torch.equal(out.cpu().view(torch.int16), golden.reduce_slices_ordered(stored, (rank + 1) % W).view(torch.int16))


@pytest.mark.parametrize("scaled", [False, True])
def test_gemm_rs_with_e4m3_inputs(cuda, scaled):
    """e4m3 inputs (optionally with per-row and per-column scales), bf16 partial results scattered to their owners'
    buffers, fp32 sum of the slices: the scattered partials against the up-cast fp32 golden on random inputs, bit for
    bit on integer-valued ones (power-of-two scales), and the reduction bit for bit given what the GEMM stored."""
    from triton_dist.kernels.amd import create_gemm_rs_intra_node_context, gemm_rs_intra_node
    announce("gemm_rs e4m3 scaled=%s" % scaled)
    W, rank, M, N, K = 4, 1, 1024, 768, 512
    m_per = M // W
    g = torch.Generator().manual_seed(5)
    ctx = create_gemm_rs_intra_node_context(M, N, torch.bfloat16, rank, W, None)
    peers = [None if r == rank else torch.randn((m_per, N), generator=g).to(torch.bfloat16) for r in range(W)]
    ctx.set_peer_partials(peers)
    for integer in (True, False):
        if integer:
            a = torch.randint(-2, 3, (M, K), generator=g).float().to(torch.float8_e4m3fn)
            b = torch.randint(-2, 3, (N, K), generator=g).float().to(torch.float8_e4m3fn)
            sa = 2.0 ** torch.randint(-3, 3, (M,), generator=g).float() if scaled else None
            sb = 2.0 ** torch.randint(-3, 3, (N,), generator=g).float() if scaled else None
        else:
            a = torch.randn((M, K), generator=g).to(torch.float8_e4m3fn)
            b = (torch.randn((N, K), generator=g) * 0.05).to(torch.float8_e4m3fn)
            sa = torch.rand(M, generator=g) * 0.09 + 0.01 if scaled else None
            sb = torch.rand(N, generator=g) * 0.9 + 0.1 if scaled else None
        out = gemm_rs_intra_node(a.to(cuda), b.to(cuda), ctx, row_scale=None if sa is None else sa.to(cuda),
                                 col_scale=None if sb is None else sb.to(cuda))
        torch.cuda.synchronize()
        assert out.shape == (m_per, N) and out.dtype == torch.bfloat16
        full = golden.fp8_scaled_gemm_fp32(a, sa, b, sb)
        for o in range(W):
            blk = ctx.scatter_bufs[o][rank * m_per:(rank + 1) * m_per].cpu()
            want = full[o * m_per:(o + 1) * m_per]
            if integer:
                assert torch.equal(blk, want.to(torch.bfloat16)), "owner %d" % o
            else:
                assert golden.max_rel_err(blk.float(), want) <= 1e-2, "owner %d" % o
        stored = ctx.scatter_bufs[rank][:M].cpu().view(W, m_per, N)
        assert torch.equal(out.cpu().view(torch.int16), golden.reduce_slices_ordered(stored, (rank + 1) % W).view(torch.int16))
    with pytest.raises(TypeError):
        f16ctx = create_gemm_rs_intra_node_context(M, N, torch.float16, rank, W, None)
        gemm_rs_intra_node(a.to(cuda), b.to(cuda), f16ctx)


def test_gemm_rs_config2_full_size(cuda):
    """BASELINE config 2: A [8192, 3584] x B [3584, 8192] (stored [8192, 3584]), rank 0 of 8, 7 synthetic peers."""
    from triton_dist.kernels.amd import create_gemm_rs_intra_node_context, gemm_rs_intra_node
    announce("gemm_rs C2 full size")
    W, rank, M, N, K = 8, 0, 8192, 8192, 3584
    g = torch.Generator().manual_seed(3 + 1)
    a = torch.randn((M, K), generator=g).to(torch.bfloat16)
    b = (torch.randn((N, K), generator=g) * 0.02).to(torch.bfloat16)
    peers = [None if r == rank else torch.randn((M // W, N), generator=g).to(torch.bfloat16) for r in range(W)]
    ctx = create_gemm_rs_intra_node_context(M, N, torch.bfloat16, rank, W, None)
    ctx.set_peer_partials(peers)
    out = gemm_rs_intra_node(a.to(cuda), b.to(cuda), ctx)
    torch.cuda.synchronize()
    ref = golden.gemm_rs_fp32(a, b, peers, rank, W)
    assert golden.max_rel_err(out.float().cpu(), ref) <= 1e-2
    # Element by element, every owner's row block: the bf16 partial that the scatter epilogue stored for owner o (rows
    # o*1024 .. of the product, at this rank's place in o's buffer) against the fp32 product of those rows, to the bf16
    # rounding of the stored value (a tile stored in the wrong place, or a dropped K tile, cannot meet that).
    for o in range(W):
        blk = ctx.scatter_bufs[o][rank * 1024:(rank + 1) * 1024].float().cpu()
        want = golden.ag_gemm_fp32([a[o * 1024:(o + 1) * 1024]], b)
        assert golden.max_rel_err(blk, want) <= 1e-2, "owner %d" % o
        assert torch.allclose(blk, want, rtol=2.0**-7, atol=2e-3 * float(want.abs().max())), "owner %d" % o
    # and the reduced output element by element: its own rounding plus that of the stored own partial
    assert torch.allclose(out.float().cpu(), ref, rtol=2.0**-6, atol=2e-3 * float(ref.abs().max()))


def test_fp8_ag_gemm_config3_full_size(cuda):
    """BASELINE config 3: 8 chunks of [2048, 8192] e4m3, B [7168, 8192] e4m3, per-row and per-column fp32 scales."""
    from triton_dist.kernels.amd import ag_gemm_intra_node
    announce("fp8 ag_gemm C3 full size")
    world, rank, m_per_rank, K, N = 8, 0, 2048, 8192, 7168
    g = torch.Generator().manual_seed(3 + 2)
    shards = [torch.randn((m_per_rank, K), generator=g).to(torch.float8_e4m3fn) for _ in range(world)]
    b = torch.randn((N, K), generator=g).to(torch.float8_e4m3fn)
    sa = torch.rand(world * m_per_rank, generator=g) * 0.09 + 0.01
    sb = torch.rand(N, generator=g) * 0.009 + 0.001
    ctx = run_ag_gemm(cuda, shards, b, rank, 2048)
    c = ag_gemm_intra_node(shards[rank].to(cuda), b.to(cuda), False, ctx, row_scale=sa.to(cuda), col_scale=sb.to(cuda))
    ctx.check_status()
    assert c.shape == (16384, 7168) and c.dtype == torch.bfloat16
    # closed form on every row of every chunk: the fp32 golden of one 2048-row chunk is a fraction of a second of CPU
    # work, so all 16384 x 7168 outputs are compared (the stated bar against the chunk's own largest value, and
    # element by element to the bf16 rounding of C, which a tile stored in the wrong place cannot meet)
    for r in range(world):
        rows = slice(r * m_per_rank, (r + 1) * m_per_rank)
        ref = golden.fp8_scaled_gemm_fp32(shards[r], sa[rows], b, sb)
        got = c[rows].float().cpu()
        assert golden.max_rel_err(got, ref) <= 1e-2, "chunk %d" % r
        assert torch.allclose(got, ref, rtol=2.0**-7, atol=2e-3 * float(ref.abs().max())), "chunk %d" % r
        del ref, got
    # linearity in the scales: doubling a row scale doubles that row (size-independent property)
    sa2 = sa.clone()
    sa2[::2] *= 2
    c2 = ag_gemm_intra_node(shards[rank].to(cuda), b.to(cuda), False, ctx, row_scale=sa2.to(cuda), col_scale=sb.to(cuda))
    ctx.check_status()
    assert torch.equal(c2[::2].float(), c[::2].float() * 2) and torch.equal(c2[1::2], c[1::2])


@pytest.mark.parametrize("dtype,K", [(torch.bfloat16, 96), (torch.bfloat16, 128), (torch.float8_e4m3fn, 192),
                                     (torch.float16, 224), (torch.bfloat16, 64)])
def test_many_tiles_with_short_and_odd_k(cuda, dtype, K):
    """Enough 256 x 256 tiles for the large-tile path, with K rows of one K tile, of an odd number of 64-byte halves
    (which must take the small tiles) and of a single 64-byte half."""
    from triton_dist.kernels.amd import gated_gemm
    announce("gemm many tiles K=%d %s" % (K, dtype))
    M, N = 4096, 6144
    g = torch.Generator().manual_seed(K)
    a = torch.randint(-3, 4, (M, K), generator=g).float()
    b = torch.randint(-3, 4, (N, K), generator=g).float()
    c = torch.empty((M, N), dtype=torch.float16 if dtype == torch.float16 else torch.bfloat16, device=cuda)
    gated_gemm(a.to(dtype).to(cuda), None, 0, b.to(dtype).to(cuda), c, None, 0, 0, 1)
    torch.cuda.synchronize()
    ref = golden.ag_gemm_fp32([a], b)    # small integers: the fp32 sums are exact, so only the final rounding differs
    assert torch.equal(c.cpu(), ref.to(c.dtype))


@pytest.mark.parametrize("M,N,K,pad", [(4100, 6150, 256, 0), (4097, 6408, 384, 64), (5000, 5001, 128, 8)])
def test_large_tiles_with_ragged_edges_and_padded_rows(cuda, M, N, K, pad):
    """The 256 x 256 path on shapes that are no multiple of the tile, with padded row strides and an output stride
    that rules out vector stores."""
    from triton_dist.kernels.amd import gated_gemm
    announce("gemm ragged M=%d N=%d K=%d pad=%d" % (M, N, K, pad))
    g = torch.Generator().manual_seed(M + N)
    a = torch.randint(-3, 4, (M, K + pad), generator=g).float()
    b = torch.randint(-3, 4, (N, K + pad), generator=g).float()
    a_d = a.to(torch.bfloat16).to(cuda)[:, :K]
    b_d = b.to(torch.bfloat16).to(cuda)[:, :K]
    c = torch.full((M + 1, N), 7.0, dtype=torch.bfloat16, device=cuda)
    gated_gemm(a_d, None, 0, b_d, c[:M], None, 0, 0, 1)
    torch.cuda.synchronize()
    ref = golden.ag_gemm_fp32([a[:, :K]], b[:, :K])
    assert torch.equal(c[:M].cpu(), ref.to(torch.bfloat16))
    assert torch.all(c[M] == 7.0)   # nothing written past the last row


def test_randomised_shapes_gating_and_layouts(cuda):
    """Forty seeded random cases over both tile paths: ragged M / N, K in 64- or 16-byte steps, padded row strides, the three
    dtypes, gating with a local shard and pre-released flags in either chunk order, plain calls. Integer-valued inputs,
    so the only rounding is the final one."""
    import random
    from triton_dist.kernels.amd import gated_gemm
    rnd = random.Random(1234)
    for case in range(40):
        dtype = rnd.choice([torch.bfloat16, torch.float16, torch.float8_e4m3fn])
        esz = 1 if dtype == torch.float8_e4m3fn else 2
        big = rnd.random() < 0.4
        gated = rnd.random() < 0.5
        K = rnd.randrange(1, 9) * 64 // esz if rnd.random() < 0.6 else rnd.randrange(1, 40) * 16 // esz
        pad_a, pad_b = rnd.choice([0, 16, 64]), rnd.choice([0, 16, 128])
        if gated:
            world = rnd.choice([2, 4, 8])
            mpc = rnd.choice([256, 512]) if big else rnd.choice([128, 256, 384, 40, 200])
            cpr = rnd.choice([1, 2])
            M = world * cpr * mpc
            N = rnd.randrange(20, 30) * 256 - rnd.choice([0, 8, 100]) if big else rnd.randrange(1, 700)
            if big and (M // 256) * ((N + 255) // 256) < 384:
                N = 256 * (384 * 256 // M + 1)
            rank = rnd.randrange(world)
        else:
            M = rnd.randrange(4000, 5200) if big else rnd.randrange(1, 900)
            N = rnd.randrange(6000, 6600) if big else rnd.randrange(1, 900)
            world, rank, mpc, cpr = 1, 0, 0, 1
        announce("gemm case %d: %s M=%d N=%d K=%d gated=%s world=%d mpc=%d rank=%d pads=%d,%d" %
                 (case, dtype, M, N, K, gated, world, mpc, rank, pad_a, pad_b))
        g = torch.Generator().manual_seed(case)
        a = torch.randint(-2, 3, (M, K + pad_a), generator=g).float()
        b = torch.randint(-2, 3, (N, K + pad_b), generator=g).float()
        a_d, b_d = a.to(dtype).to(cuda)[:, :K], b.to(dtype).to(cuda)[:, :K]
        out_dtype = torch.float16 if dtype == torch.float16 else torch.bfloat16
        c = torch.empty((M, N), dtype=out_dtype, device=cuda)
        if gated:
            mpr = M // world
            local = a_d[rank * mpr:(rank + 1) * mpr].contiguous()
            ws = a_d.clone()
            if mpc % 128 == 0:
                ws[rank * mpr:(rank + 1) * mpr] = 0      # the own rows must come from the local shard
            else:
                local = None                              # (chunks that are no whole tiles: everything through the flags)
            flags = torch.ones(world * cpr, dtype=torch.int32, device=cuda)
            gated_gemm(ws, local, rank * mpr, b_d, c, flags, mpc, rank, world)
        else:
            gated_gemm(a_d, None, 0, b_d, c, None, 0, 0, 1)
        torch.cuda.synchronize()
        ref = golden.ag_gemm_fp32([a[:, :K]], b[:, :K]).to(out_dtype)
        assert torch.equal(c.cpu(), ref), "case %d differs" % case


@pytest.mark.parametrize("tile", [0, 1, 2, 3, 4])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float8_e4m3fn])
def test_each_tile_configuration_forced(cuda, switches, tile, dtype):
    """Every compiled tile (256x256, 256x128, 128x128, 128x192, 128x256) forced through the library's measurement switch on the same
    ragged, padded, gated and scaled cases; integer-valued inputs, so only the final rounding remains."""
    from triton_dist.kernels.amd import gated_gemm
    from triton_dist import _lib
    switches(_lib.TDIST_DEBUG_GEMM_TILE, tile)
    esz = 1 if dtype == torch.float8_e4m3fn else 2
    out_dtype = torch.float16 if dtype == torch.float16 else torch.bfloat16
    for case, (M, N, K, pad, gated) in enumerate([(1030, 1290, 256 // esz, 16, False), (2048, 1536, 640 // esz, 0, True),
                                                   (512, 200, 128 // esz, 64, True), (300, 2100, 1152 // esz, 0, False)]):
        announce("gemm forced tile %d %s M=%d N=%d K=%d gated=%s" % (tile, dtype, M, N, K, gated))
        g = torch.Generator().manual_seed(100 * tile + case)
        a = torch.randint(-2, 3, (M, K + pad), generator=g).float()
        b = torch.randint(-2, 3, (N, K + pad), generator=g).float()
        a_d, b_d = a.to(dtype).to(cuda)[:, :K], b.to(dtype).to(cuda)[:, :K]
        c = torch.full((M, N), float("nan"), dtype=out_dtype, device=cuda)
        sa = sb = None
        if dtype == torch.float8_e4m3fn and case % 2 == 1:   # power-of-two scales keep the result exact
            sa = (2.0 ** torch.randint(-3, 3, (M,), generator=g).float()).to(cuda)
            sb = (2.0 ** torch.randint(-3, 3, (N,), generator=g).float()).to(cuda)
        if gated:
            world, rank = 2, 1
            mpr = M // world
            local = a_d[rank * mpr:(rank + 1) * mpr].contiguous()
            ws = a_d.clone()
            ws[rank * mpr:(rank + 1) * mpr] = 0
            flags = torch.ones(world, dtype=torch.int32, device=cuda)
            gated_gemm(ws, local, rank * mpr, b_d, c, flags, mpr, rank, world, row_scale=sa, col_scale=sb)
        else:
            gated_gemm(a_d, None, 0, b_d, c, None, 0, 0, 1, row_scale=sa, col_scale=sb)
        torch.cuda.synchronize()
        ref = golden.ag_gemm_fp32([a[:, :K]], b[:, :K])
        if sa is not None:
            ref = ref * sa.cpu()[:, None] * sb.cpu()[None, :]
        assert torch.equal(c.cpu(), ref.to(out_dtype)), "tile %d case %d differs" % (tile, case)


def test_paced_arrivals_hold_the_chunks_back(cuda):
    """Link pacing of the one-GPU producer: with a slow emulated link the call cannot finish before the last chunk's
    link time has passed, and the result is the unpaced one."""
    from triton_dist.kernels.amd import ag_gemm_intra_node, create_ag_gemm_intra_node_context
    announce("ag-gemm with paced arrivals")
    world, rank, mpr, K, N = 4, 1, 256, 512, 384
    shards, b = make_ag_case(world, mpr, K, N, torch.bfloat16, seed=77)
    ctx = create_ag_gemm_intra_node_context(world * mpr, N, K, torch.bfloat16, torch.bfloat16, rank, world, None, M_PER_CHUNK=128)
    ctx.set_peer_shards({r: s.to(cuda) for r, s in enumerate(shards) if r != rank})
    a_d, b_d = shards[rank].to(cuda), b.to(cuda)
    want = ag_gemm_intra_node(a_d, b_d, False, ctx)
    ctx.check_status()
    chunk_bytes = 128 * K * 2
    ctx.link_gbps = chunk_bytes / 1.5e6          # 1.5 ms per chunk, two chunks per peer: the last one is due at 3 ms
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    got = ag_gemm_intra_node(a_d, b_d, False, ctx)
    stop.record()
    ctx.check_status()
    assert torch.equal(got, want)
    assert golden.max_rel_err(got.float().cpu(), golden.ag_gemm_fp32(shards, b)) <= 1e-2
    assert start.elapsed_time(stop) >= 2.9, "the last chunk was released before its link time"
    assert start.elapsed_time(stop) < 200


@pytest.mark.parametrize("producer_kernel,link_gbps", [(False, 0.0), (True, 0.0), (True, 50.0)])
def test_ag_gemm_kernel_producer_and_graph_replay(cuda, producer_kernel, link_gbps):
    """The whole op (producer on its stream, gated GEMM, flag reset) captured into a HIP graph and replayed three
    times with eager work in between: every replay must reproduce the eager result from a poisoned workspace. Runs
    with the copy producer and with the one-launch kernel producer (unpaced and paced)."""
    from triton_dist.kernels.amd import ag_gemm_intra_node, create_ag_gemm_intra_node_context
    announce("ag-gemm graph replay, kernel producer %s, link %s" % (producer_kernel, link_gbps))
    world, rank, mpr, K, N = 4, 2, 512, 1024, 640
    shards, b = make_ag_case(world, mpr, K, N, torch.bfloat16, seed=91)
    # capture needs streams other than the default one
    ctx = create_ag_gemm_intra_node_context(world * mpr, N, K, torch.bfloat16, torch.bfloat16, rank, world, None,
                                            M_PER_CHUNK=256, gemm_stream=torch.cuda.Stream(),
                                            ag_streams=[torch.cuda.Stream(), torch.cuda.Stream()])
    ctx.set_peer_shards({r: s.to(cuda) for r, s in enumerate(shards) if r != rank})
    ctx.producer_kernel, ctx.link_gbps = producer_kernel, link_gbps
    a_d, b_d = shards[rank].to(cuda), b.to(cuda)
    want = ag_gemm_intra_node(a_d, b_d, False, ctx).clone()
    ctx.check_status()
    assert golden.max_rel_err(want.float().cpu(), golden.ag_gemm_fp32(shards, b)) <= 1e-2
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        ag_gemm_intra_node(a_d, b_d, False, ctx)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = ag_gemm_intra_node(a_d, b_d, False, ctx)
    torch.cuda.synchronize()
    for replay in range(3):
        ctx.workspace_tensors[rank].view(torch.uint8).fill_(0x7B)   # eager work between the replays
        out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want), "replay %d differs from the eager result" % replay
    ctx.check_status()
    if producer_kernel:
        assert int(ctx.producer_counters.abs().sum()) == 0


@pytest.mark.parametrize("dtype,world,mpr,mpc,K,N", [(torch.bfloat16, 4, 1024, 256, 512, 1536), (torch.float8_e4m3fn, 8, 512, 256, 1024, 1280),
                                                     (torch.float16, 4, 512, 512, 256, 640)])
def test_seeded_random_chunk_delays(cuda, dtype, world, mpr, mpc, K, N):
    """Race provocation as in the reference (its producer sleeps with probability 0.7 before it copies when run "for
    correctness", kernels/nvidia/allgather.py:72-77,118-121, and its test overwrites the workspace between iterations,
    test/nvidia/test_ag_gemm_intra_node.py:122-127): about 7 of 10 chunks, another set on every call, arrive up to
    150 us late, from a workspace full of garbage. Integer-valued inputs, so a tile that read a row before it had
    arrived cannot hide in a tolerance: every call must give the exact product, bit for bit the same."""
    from triton_dist.kernels.amd import ag_gemm_intra_node, create_ag_gemm_intra_node_context
    announce("ag-gemm with seeded random chunk delays %s world=%d" % (dtype, world))
    g = torch.Generator().manual_seed(world + K)
    shards = [torch.randint(-2, 3, (mpr, K), generator=g).float() for _ in range(world)]
    b = torch.randint(-2, 3, (N, K), generator=g).float()
    want = golden.ag_gemm_fp32(shards, b).to(torch.float16 if dtype == torch.float16 else torch.bfloat16)
    for rank in (0, world - 1):
        ctx = create_ag_gemm_intra_node_context(world * mpr, N, K, dtype, torch.bfloat16, rank, world, None, M_PER_CHUNK=mpc)
        ctx.set_peer_shards({r: s.to(dtype).to(cuda) for r, s in enumerate(shards) if r != rank})
        ctx.producer_kernel, ctx.random_delay_us, ctx.delay_seed = True, 150.0, 1234 + rank
        a_d, b_d = shards[rank].to(dtype).to(cuda), b.to(dtype).to(cuda)
        for call in range(6):
            ctx.workspace_tensors[rank].view(torch.uint8).fill_(0x7B if dtype != torch.float8_e4m3fn else 0x7F)
            c = ag_gemm_intra_node(a_d, b_d, False, ctx)
            ctx.check_status()
            assert torch.equal(c.cpu(), want), "rank %d call %d" % (rank, call)
        assert ctx.delay_calls == 6 and int(ctx.producer_counters.abs().sum()) == 0


def test_for_correctness_context_delays_its_producer(cuda):
    """The NVIDIA-side context created with for_correctness=True (kernels/nvidia/allgather_gemm.py:786-828) delays
    its arrivals at random; the result is the closed form all the same."""
    from triton_dist.kernels.nvidia.allgather_gemm import ag_gemm_intra_node, create_ag_gemm_intra_node_context
    announce("ag-gemm nvidia-side for_correctness")
    world, rank, mpr, K, N = 4, 2, 384, 256, 512
    g = torch.Generator().manual_seed(5)
    shards = [torch.randint(-2, 3, (mpr, K), generator=g).float() for _ in range(world)]
    b = torch.randint(-2, 3, (N, K), generator=g).float()
    a_d, b_d = shards[rank].bfloat16().to(cuda), b.bfloat16().to(cuda)
    ctx = create_ag_gemm_intra_node_context(a_d, b_d, rank, world, for_correctness=True)
    assert ctx.producer_kernel and ctx.random_delay_us > 0
    ctx.set_peer_shards({r: s.bfloat16().to(cuda) for r, s in enumerate(shards) if r != rank})
    for _ in range(3):
        c = ag_gemm_intra_node(a_d, b_d, ctx)
        ctx.check_status()
        assert torch.equal(c.cpu(), golden.ag_gemm_fp32(shards, b).to(torch.bfloat16))


@pytest.mark.parametrize("m_per,K", [(256, 256), (200, 320), (72, 96)])
def test_nvidia_side_signatures(cuda, m_per, K):
    """The NVIDIA-side entry points of the reference (kernels/nvidia/allgather_gemm.py:785-882,
    gemm_reduce_scatter.py:77-88, 468-538): context from the local tensors, one flag per rank segment, M_per_rank padded
    to BLOCK_M for the reduce-scatter."""
    from triton_dist.kernels.nvidia import (ag_gemm_intra_node, create_ag_gemm_intra_node_context, create_gemm_rs_context,
                                            gemm_rs)
    announce("nvidia-side signatures m_per=%d K=%d" % (m_per, K))
    W, rank, N = 4, 1, 384
    g = torch.Generator().manual_seed(m_per)
    # GEMM-RS with padded rows
    a = torch.randn((W * m_per, K), generator=g).to(torch.bfloat16)
    b = (torch.randn((N, K), generator=g) * 0.02).to(torch.bfloat16)
    peers = [None if r == rank else torch.randn((m_per, N), generator=g).to(torch.bfloat16) for r in range(W)]
    ctx = create_gemm_rs_context(W * m_per, N, rank, W, W, torch.bfloat16, torch.cuda.current_stream())
    ctx.set_peer_partials(peers)
    out = gemm_rs(a.to(cuda), b.to(cuda), ctx)
    torch.cuda.synchronize()
    assert out.shape == (m_per, N)
    assert golden.max_rel_err(out.float().cpu(), golden.gemm_rs_fp32(a, b, peers, rank, W)) <= 1e-2
    # AG-GEMM gated per rank segment
    # (rank segments of 200 and 72 rows are no whole tiles: a tile then waits for every segment it touches)
    shards, bb = make_ag_case(W, m_per, K, N, torch.bfloat16, seed=K)
    actx = create_ag_gemm_intra_node_context(shards[rank].to(cuda), bb.to(cuda), rank, W)
    assert actx.barrier_tensors[rank].numel() == W and actx.M_PER_CHUNK == m_per
    actx.set_peer_shards({r: s.to(cuda) for r, s in enumerate(shards) if r != rank})
    for _ in range(2):   # (the second call finds the flags reset by the first)
        actx.workspace_tensors[rank].view(torch.uint8).fill_(0x7B)
        c = ag_gemm_intra_node(shards[rank].to(cuda), bb.to(cuda), actx)
        actx.check_status()
        assert golden.max_rel_err(c.float().cpu(), golden.ag_gemm_fp32(shards, bb)) <= 1e-2


@pytest.mark.parametrize("dtype,K", [(torch.bfloat16, 8), (torch.bfloat16, 40), (torch.float16, 72), (torch.bfloat16, 200),
                                     (torch.bfloat16, 1000), (torch.float8_e4m3fn, 16), (torch.float8_e4m3fn, 80),
                                     (torch.float8_e4m3fn, 1008), (torch.float16, 4104)])
def test_k_ending_inside_a_k_tile(cuda, dtype, K):
    """K rows of any whole number of 16-byte pieces: the last K tile is filled up with zeros on its way into the LDS.
    The bytes behind a row's end are poisoned with NaN, so a lane that read them would show. Integer-valued inputs:
    exact up to the final rounding. With and without a split last round."""
    from triton_dist import _lib
    from triton_dist.kernels.amd import gated_gemm
    announce("gemm K tail K=%d %s" % (K, dtype))
    esz = 1 if dtype == torch.float8_e4m3fn else 2
    pad = 48 // esz
    out_dtype = torch.float16 if dtype == torch.float16 else torch.bfloat16
    # (2176 x 2048 is 272 tiles: with the workspace and a long K the last 16 are cut along K)
    for M, N, ws in [(300, 200, None), (1100, 1290, None), (2176, 2048, _lib.new_split_k_workspace(cuda))]:
        g = torch.Generator().manual_seed(K + M)
        a = torch.randint(-2, 3, (M, K + pad), generator=g).float()
        b = torch.randint(-2, 3, (N, K + pad), generator=g).float()
        a_d, b_d = a.to(dtype).to(cuda), b.to(dtype).to(cuda)
        for t in (a_d, b_d):
            if esz == 1:
                t.view(torch.uint8)[:, K:] = 0x7F
            else:
                t.view(torch.int16)[:, K:] = 0x7FC0
            assert torch.isnan(t[:, K:].float()).all()
        c = torch.full((M, N), float("nan"), dtype=out_dtype, device=cuda)
        gated_gemm(a_d[:, :K], None, 0, b_d[:, :K], c, None, 0, 0, 1, sk_workspace=ws)
        torch.cuda.synchronize()
        ref = golden.ag_gemm_fp32([a[:, :K]], b[:, :K])
        assert torch.equal(c.cpu(), ref.to(out_dtype)), "M=%d N=%d differs" % (M, N)
    with pytest.raises(_lib.TdistError, match="16 bytes"):
        gated_gemm(a_d[:, :K - 4 // esz], None, 0, b_d[:, :K - 4 // esz], c, None, 0, 0, 1)


@pytest.mark.parametrize("dtype,K", [(torch.bfloat16, 2056), (torch.float8_e4m3fn, 4112)])
def test_ragged_chunks_k_tail_and_split_round_together(cuda, dtype, K):
    """Chunks of 200 rows, a K that ends 16 bytes into its last K tile and a last round cut along K (21 tiles of
    128 x 128 on 256 workgroups: four pieces each, the last piece holding the ragged K tile), three launches in a row
    on one workspace: exact on integer-valued inputs."""
    from triton_dist import _lib
    from triton_dist.kernels.amd import gated_gemm
    announce("gemm ragged chunks + K tail + split round %s" % dtype)
    world, mpc, rank, N = 4, 200, 2, 328
    M = world * mpc
    ws = _lib.new_split_k_workspace(cuda)
    status = torch.zeros(2, dtype=torch.int32, device=cuda)
    flags = torch.ones(world, dtype=torch.int32, device=cuda)
    for launch in range(3):
        g = torch.Generator().manual_seed(K + launch)
        a = torch.randint(-2, 3, (M, K), generator=g).float()
        b = torch.randint(-2, 3, (N, K), generator=g).float()
        c = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=cuda)
        gated_gemm(a.to(dtype).to(cuda), None, 0, b.to(dtype).to(cuda), c, flags, mpc, rank, world, status=status, sk_workspace=ws)
        torch.cuda.synchronize()
        assert status.tolist() == [0, 0]
        assert torch.equal(c.cpu(), golden.ag_gemm_fp32([a], b).to(torch.bfloat16)), "launch %d" % launch
    # (the split form really ran: the workspace's epoch word has moved)
    assert int(ws.view(torch.int32)[0]) != 0


@pytest.mark.parametrize("world,mpc,rank", [(4, 200, 1), (8, 72, 7), (2, 1000, 0), (3, 130, 2)])
def test_chunks_that_are_no_whole_tiles(cuda, world, mpc, rank):
    """m_per_chunk of any size: a 128-row tile waits for every flag its rows touch. With every flag but one released,
    exactly the tiles that hold rows of the withheld chunk give up (bounded wait, status names that chunk) and every
    other row of C is right; with all flags released the whole result is."""
    from triton_dist.kernels.amd import gated_gemm
    announce("gemm ragged chunks world=%d mpc=%d rank=%d" % (world, mpc, rank))
    M, N, K = world * mpc, 328, 160
    g = torch.Generator().manual_seed(mpc)
    a = torch.randint(-2, 3, (M, K), generator=g).float()
    b = torch.randint(-2, 3, (N, K), generator=g).float()
    a_d, b_d = a.to(torch.bfloat16).to(cuda), b.to(torch.bfloat16).to(cuda)
    ref = golden.ag_gemm_fp32([a], b).to(torch.bfloat16).to(cuda)
    status = torch.zeros(2, dtype=torch.int32, device=cuda)
    flags = torch.ones(world, dtype=torch.int32, device=cuda)
    c = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=cuda)
    gated_gemm(a_d, None, 0, b_d, c, flags, mpc, rank, world, status=status)
    torch.cuda.synchronize()
    assert status.tolist() == [0, 0] and torch.equal(c, ref)
    held = (rank + 1) % world
    flags[held] = 0
    c.fill_(float("nan"))
    gated_gemm(a_d, None, 0, b_d, c, flags, mpc, rank, world, status=status, spin_limit=200)
    torch.cuda.synchronize()
    from triton_dist import _lib
    assert status.tolist() == [_lib.TDIST_ERR_TIMEOUT, held]
    rows = torch.arange(M, device=cuda)
    tile_lo, tile_hi = rows // 128 * 128, torch.clamp(rows // 128 * 128 + 127, max=M - 1)
    touches = (tile_lo // mpc <= held) & (tile_hi // mpc >= held)
    assert torch.equal(c[~touches], ref[~touches])
    assert torch.isnan(c[touches].float()).all()
    # a local shard that is no whole number of tiles cannot be handed in beside such chunks
    with pytest.raises(_lib.TdistError, match="local shard"):
        gated_gemm(a_d, a_d[rank * mpc:(rank + 1) * mpc], rank * mpc, b_d, c, flags, mpc, rank, world)
