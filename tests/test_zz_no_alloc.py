"""tdist_moe_scatter_index_static, the index build for callers that cannot allocate (its scratch is an array inside
the library): called through the C ABI and held, bit for bit, against tdist_moe_scatter_index on the same ids, on two
calls in a row of which the second is smaller (the scratch keeps what the first call left in it), and against the
oracle. Sizes beyond the built-in scratch are refused."""
import pytest
import torch

from oracle import golden
from tests.conftest import announce

pytestmark = pytest.mark.gpu


def run_both(cuda, ids, G):
    from triton_dist import _lib
    lib = _lib.load()
    T, topk = ids.shape
    n = T * topk
    ids_d = ids.to(cuda)

    def outputs():
        return [torch.full((G, ), -7, dtype=torch.int32, device=cuda), torch.full((G + 1, ), -7, dtype=torch.int32, device=cuda),
                torch.full((n, ), -7, dtype=torch.int32, device=cuda), torch.full((n, ), -7, dtype=torch.int32, device=cuda),
                torch.full((n, ), -7, dtype=torch.int32, device=cuda)]
    ref, got = outputs(), outputs()
    ws = torch.zeros(lib.tdist_moe_workspace_bytes(n, G), dtype=torch.uint8, device=cuda)
    torch.cuda.synchronize()
    stream = _lib.stream_ptr()
    _lib.call("tdist_moe_scatter_index", ids_d.data_ptr(), n, topk, G, *[t.data_ptr() for t in ref], ws.data_ptr(), ws.numel(), stream)
    _lib.call("tdist_moe_scatter_index_static", ids_d.data_ptr(), n, topk, G, *[t.data_ptr() for t in got], stream)
    torch.cuda.synchronize()
    return ref, got


@pytest.mark.parametrize("launches", ["one", "three"])
def test_static_scratch_entry_matches_the_workspace_entry(cuda, switches, launches):
    from triton_dist import _lib
    if launches == "three":
        switches(_lib.TDIST_DEBUG_MOE_INDEX_FORM, 3)
    g = torch.Generator().manual_seed(21)
    # BASELINE's MoE config first, then smaller ones: the second call finds the first call's leftovers in the scratch
    for T, topk, G in [(4096, 8, 256), (500, 8, 256), (37, 2, 16), (4096, 8, 256)]:
        announce("no-alloc index build T=%d topk=%d G=%d (%s launch)" % (T, topk, G, launches))
        ids = golden.random_distinct_experts(T, G, topk, g)
        ref, got = run_both(cuda, ids, G)
        for a, b in zip(got, ref):
            assert torch.equal(a, b), (T, topk, G)
        want = golden.moe_preprocess(ids, G)      # splits, cumsum, scatter, gather, topk index
        for a, b in zip(got, want):
            assert torch.equal(a.cpu().view(-1), b.view(-1)), (T, topk, G)


def test_static_scratch_entry_rejects_what_does_not_fit(cuda):
    from triton_dist import _lib
    lib = _lib.load()
    announce("no-alloc index build limits")
    buf = torch.zeros(16, dtype=torch.int32, device=cuda)
    p = buf.data_ptr()
    # 256 experts: 261 632 ids fit the 1 MiB scratch, 262 145 do not; nothing is launched for a call that is refused
    assert lib.tdist_moe_workspace_bytes(261632, 256) <= 1 << 20 < lib.tdist_moe_workspace_bytes(262145, 256)
    assert lib.tdist_moe_scatter_index_static(p, 262145, 8, 256, p, p, p, p, None, None) == _lib.TDIST_ERR_UNSUPPORTED
    assert "1048576" in _lib.last_error()
    assert lib.tdist_moe_scatter_index_static(p, 1024, 8, 4096 * 2, p, p, p, p, None, None) in (_lib.TDIST_ERR_UNSUPPORTED,
                                                                                               _lib.TDIST_ERR_INVALID)
    assert lib.tdist_moe_scatter_index_static(None, 16, 2, 4, p, p, p, p, None, None) == _lib.TDIST_ERR_INVALID
    torch.cuda.synchronize()
    assert int(buf.abs().sum()) == 0
