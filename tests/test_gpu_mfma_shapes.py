"""The split-ring GEMM tiles (256 x 256, 256 x 128, 128 x 256, 128 x 192) run on the 16-row MFMA blocks (16x16x32 for bf16/f16,
16x16x128 for e4m3) with their accumulators in fixed registers; the 128 x 128 tile runs on the 32-row blocks (32x32x16
/ 32x32x64) with accumulators the compiler places. Each form is held against the exact result on integer-valued inputs (every partial sum is an
integer that fp32 holds) over the K-loop's corner cases, and on random inputs to max relative error <= 1e-2 of fp32 and
to each other within the rounding of the output."""

import pytest
import torch

from tests.conftest import announce

pytestmark = pytest.mark.gpu


@pytest.fixture
def tile_env(switches):
    """Puts the forced tile back to "the library decides" when the test ends."""
    from triton_dist import _lib
    switches(_lib.TDIST_DEBUG_GEMM_TILE, None)
    yield


def run_tile(cuda, a, b, out_dtype, tile, **kw):
    from triton_dist import _lib
    from triton_dist.kernels.amd import gated_gemm
    _lib.check(_lib.load().tdist_debug_set(_lib.TDIST_DEBUG_GEMM_TILE, tile))
    c = torch.full((a.shape[0], b.shape[0]), float("nan"), dtype=out_dtype, device=cuda)
    status = torch.zeros(2, dtype=torch.int32, device=cuda)
    gated_gemm(a, None, 0, b, c, None, 0, 0, 1, status=status, **kw)
    torch.cuda.synchronize()
    assert status.tolist() == [0, 0]
    return c


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float8_e4m3fn])
@pytest.mark.parametrize("tile", [0, 1, 2, 3, 4])
@pytest.mark.parametrize("M,N,K", [(512, 512, 128), (768, 512, 384), (300, 200, 640), (1024, 1280, 1152), (640, 1536, 256)])
def test_exact_on_integer_inputs(cuda, tile_env, dtype, tile, M, N, K):
    """One K tile (e4m3) or two; an odd number of K tiles (the e4m3 loop works in pairs of tiles); a ragged shape (the
    bounds-checked epilogue); several tiles per workgroup row; a width that is whole 192-column tiles. tile 0 = 256x256,
    1 = 256x128, 2 = 128x128, 3 = 128x192, 4 = 128x256."""
    announce("mfma shapes exact %s tile %d %dx%dx%d" % (dtype, tile, M, N, K))
    g = torch.Generator().manual_seed(M + N + K + tile)
    a = torch.randint(-2, 3, (M, K), generator=g).float().to(dtype).to(cuda)
    b = torch.randint(-2, 3, (N, K), generator=g).float().to(dtype).to(cuda)
    out_dtype = torch.bfloat16 if dtype == torch.float8_e4m3fn else dtype
    ref = (a.float() @ b.float().T).to(out_dtype)
    assert torch.equal(run_tile(cuda, a, b, out_dtype, tile), ref)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float8_e4m3fn])
@pytest.mark.parametrize("tile", [0, 1, 3, 4])
def test_every_k_tile_count_from_one_to_thirteen(cuda, tile_env, dtype, tile):
    """The split ring's K loop is unrolled over its six (A stage, B stage) pairs: every number of 128-byte K tiles
    from 1 to 13 leaves the loop after a different pair, twice over. Two tiles of C per workgroup column so that a
    second tile starts on a ring the first one has used. Exact on integer-valued inputs."""
    esz = 1 if dtype == torch.float8_e4m3fn else 2
    out_dtype = torch.bfloat16 if dtype == torch.float8_e4m3fn else dtype
    for kt in range(1, 14):
        M, N, K = 512, 768, kt * 128 // esz
        announce("mfma shapes k tiles %s tile %d kt %d (%dx%dx%d)" % (dtype, tile, kt, M, N, K))
        g = torch.Generator().manual_seed(kt + 100 * tile)
        a = torch.randint(-2, 3, (M, K), generator=g).float().to(dtype).to(cuda)
        b = torch.randint(-2, 3, (N, K), generator=g).float().to(dtype).to(cuda)
        ref = (a.float() @ b.float().T).to(out_dtype)
        assert torch.equal(run_tile(cuda, a, b, out_dtype, tile, max_workgroups=2), ref), "kt = %d" % kt


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float8_e4m3fn])
def test_random_inputs_close_in_every_form(cuda, tile_env, dtype):
    M, N, K = 1536, 1024, 4224
    announce("mfma shapes random %s %dx%dx%d" % (dtype, M, N, K))
    g = torch.Generator().manual_seed(11)
    a = torch.randn((M, K), generator=g).to(dtype).to(cuda)
    b = (torch.randn((N, K), generator=g) * 0.05).to(dtype).to(cuda)
    kw = {}
    ref = a.float() @ b.float().T
    if dtype == torch.float8_e4m3fn:
        kw["row_scale"] = (torch.rand(M, generator=g) * 0.09 + 0.01).to(cuda)
        kw["col_scale"] = (torch.rand(N, generator=g) * 0.9 + 0.1).to(cuda)
        ref = ref * kw["row_scale"][:, None] * kw["col_scale"][None, :]
    out = [run_tile(cuda, a, b, torch.bfloat16, tile, **kw) for tile in (0, 1, 2, 3, 4)]
    for c in out:
        rel = (c.float() - ref).abs().max() / ref.abs().max()
        assert rel.item() <= 1e-2
        # (the forms differ in the order of the fp32 sums only: one rounding step of the bf16 output at most)
        assert torch.allclose(c.float(), out[0].float(), rtol=2.0**-7, atol=1e-3 * float(ref.abs().max()))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float8_e4m3fn])
@pytest.mark.parametrize("block", [128, 256])
def test_grouped_blocks_exact(cuda, dtype, block):
    """The grouped form (gathered A rows, per-block expert weights, scattered C rows) on both block sizes."""
    from oracle import golden
    from tests.test_gpu_group_gemm import make_case, run
    world, mpr, K, N, E, topk = 4, 96, 640, 328, 6, 2
    announce("mfma shapes grouped %s block %d" % (dtype, block))
    shards, w, ids = make_case(world, mpr, K, N, E, topk, dtype, seed=block, integer=True)
    ref = golden.ag_group_gemm_fp32(shards, w, ids)
    ctx, c = run(cuda, shards, w, ids, 1, E, block)
    ctx.check_status()
    assert torch.equal(c.float().cpu(), ref.to(c.dtype).float())
