"""(b2) slice reduction on the GPU against the oracle: bit-exact (fp32 accumulation in a fixed order)."""
import numpy as np
import pytest
import torch

from oracle import cref, golden
from tests.conftest import announce

pytestmark = pytest.mark.gpu


def run_reduce(c, first, dtype_code=None):
    from triton_dist import _lib
    R = c.shape[0]
    n = c[0].numel()
    out = torch.empty(c.shape[1:], dtype=c.dtype, device=c.device)
    _lib.call("tdist_reduce_slices", c.data_ptr(), c.stride(0), R, first, n, out.data_ptr(),
              _lib.dtype_code(c.dtype) if dtype_code is None else dtype_code, _lib.stream_ptr())
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("R", [1, 2, 4, 8, 16, 5, 3])
@pytest.mark.parametrize("n", [8 * 512 * 3, 8 * 777, 1001, 7])
def test_reduce_matches_oracle_bit_exact(cuda, R, n):
    announce("reduce R=%d n=%d" % (R, n))
    g = torch.Generator().manual_seed(R * 1000 + n)
    c = torch.randn((R, n), generator=g).to(torch.bfloat16)
    first = (R // 2 + 1) % R
    want = golden.reduce_slices_ordered(c, first)
    got = run_reduce(c.to(cuda), first).cpu()
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))


def test_reduce_f16(cuda):
    announce("reduce f16")
    g = torch.Generator().manual_seed(3)
    c = torch.randn((8, 8 * 1000), generator=g).to(torch.float16)
    want = golden.reduce_slices_ordered(c, 1)
    got = run_reduce(c.to(cuda), 1).cpu()
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))


def test_reduce_full_size_gemm_rs_slices(cuda):
    """BASELINE config 2: 8 slices [1024, 8192] bf16 -> [1024, 8192], rank 0 (first slice 1)."""
    announce("reduce full size 8x[1024,8192]")
    g = torch.Generator().manual_seed(4)
    c = torch.randn((8, 1024, 8192), generator=g).to(torch.bfloat16)
    want = golden.reduce_slices_ordered(c, 1)
    got = run_reduce(c.to(cuda), 1).cpu()
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    # the scalar C restatement agrees on a sample of rows
    rows = c[:, 100:102].reshape(8, -1)
    bits = rows.contiguous().view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(cref.reduce_slices_bf16(bits, 1), got[100:102].reshape(-1).view(torch.int16).numpy().view(np.uint16))


def test_reduce_through_the_op_entry_point(cuda):
    from triton_dist.kernels.amd.gemm_reduce_scatter import ring_reduce_after_scatter
    announce("ring_reduce_after_scatter")
    g = torch.Generator().manual_seed(5)
    R, rank = 8, 3
    c = torch.randn((R * 64, 512), generator=g).to(torch.bfloat16)
    out = ring_reduce_after_scatter(rank, R, c.to(cuda), torch.cuda.current_stream())
    torch.cuda.synchronize()
    want = golden.reduce_slices_ordered(c.view(R, 64, 512), (rank + 1) % R)
    assert torch.equal(out.cpu().view(torch.int16), want.view(torch.int16))


def test_copy_bytes_helper(cuda):
    from triton_dist import _lib
    announce("copy_bytes")
    src = torch.randint(0, 255, (1 << 20, ), dtype=torch.uint8, device=cuda)
    dst = torch.zeros_like(src)
    _lib.bench_call("tdist_copy_bytes", dst.data_ptr(), src.data_ptr(), src.numel(), _lib.stream_ptr())
    torch.cuda.synchronize()
    assert torch.equal(src, dst)


def test_mfma_rate_probe_runs(cuda):
    from triton_dist import _lib
    announce("mfma rate probe")
    cus = _lib.load().tdist_num_cus()
    sink = torch.full((cus * 256, ), float("nan"), dtype=torch.float32, device=cuda)
    for code in (_lib.TDIST_BF16, _lib.TDIST_F8E4M3):
        for rnd in (0, 1):
            _lib.bench_call("tdist_mfma_rate_probe", code, rnd, 8, sink.data_ptr(), _lib.stream_ptr())
            torch.cuda.synchronize()
            assert torch.isfinite(sink).all()
    # constant operands: 1.0 x 1.0 summed over K (16 per bf16 MFMA), 8 K steps, the first accumulator of 16 blocks
    _lib.bench_call("tdist_mfma_rate_probe", _lib.TDIST_BF16, 0, 8, sink.data_ptr(), _lib.stream_ptr())
    torch.cuda.synchronize()
    assert torch.all(sink == 16 * 8 * 16.0)
    with pytest.raises(_lib.TdistError):
        _lib.bench_call("tdist_mfma_rate_probe", _lib.TDIST_BF16, 0, 7, sink.data_ptr(), _lib.stream_ptr())
    # the 16-row blocks: 64 blocks, K = 32 per bf16 MFMA
    for code in (_lib.TDIST_BF16, _lib.TDIST_F8E4M3):
        for rnd in (0, 1):
            _lib.bench_call("tdist_mfma_rate_probe_16row", code, rnd, 8, sink.data_ptr(), _lib.stream_ptr())
            torch.cuda.synchronize()
            assert torch.isfinite(sink).all()
    _lib.bench_call("tdist_mfma_rate_probe_16row", _lib.TDIST_BF16, 0, 8, sink.data_ptr(), _lib.stream_ptr())
    torch.cuda.synchronize()
    assert torch.all(sink == 64 * 8 * 32.0)
    with pytest.raises(_lib.TdistError):
        _lib.bench_call("tdist_mfma_rate_probe_16row", _lib.TDIST_BF16, 0, 7, sink.data_ptr(), _lib.stream_ptr())
