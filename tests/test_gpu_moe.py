"""(c) MoE dispatch / combine on the GPU against the oracle: indices, splits and moved bytes bit-exact;
the weighted combine within 1e-2 relative (fp32 accumulation, fixed k order)."""
import numpy as np
import pytest
import torch

from oracle import golden
from tests.conftest import announce

pytestmark = pytest.mark.gpu


def make_case(T, topk, G, H, seed, distinct=True):
    g = torch.Generator().manual_seed(seed)
    if distinct and topk <= G:
        ids = golden.random_distinct_experts(T, G, topk, g)
    else:
        ids = torch.randint(0, G, (T, topk), generator=g).to(torch.int32)
    x = torch.randn((T, H), generator=g)
    q, s = golden.quantize_per_token_e4m3(x)
    w = torch.softmax(torch.randn((T, topk), generator=g), dim=-1).float().contiguous()
    return ids, x, q, s, w


@pytest.mark.parametrize("T,topk,G", [(4096, 8, 256), (64, 8, 16), (1, 1, 1), (1, 8, 256), (1000, 6, 48), (257, 4, 7),
                                      (5000, 2, 1024), (3, 2, 3)])
def test_preprocess_bit_exact(cuda, T, topk, G):
    from triton_dist.kernels.amd import moe_dispatch_preprocess
    announce("moe preprocess T=%d topk=%d G=%d" % (T, topk, G))
    ids, *_ = make_case(T, topk, G, 16, seed=T + topk + G)
    splits, cumsum, scatter, gather, topk_idx = moe_dispatch_preprocess(ids.to(cuda), G, want_topk_index=True)
    torch.cuda.synchronize()
    w_splits, w_cumsum, w_scatter, w_gather, w_topk = golden.moe_preprocess(ids, G)
    assert torch.equal(splits.cpu(), w_splits)
    assert torch.equal(cumsum.cpu(), w_cumsum)
    assert torch.equal(scatter.cpu(), w_scatter)
    assert torch.equal(gather.cpu(), w_gather)
    assert torch.equal(topk_idx.cpu(), w_topk)


def test_preprocess_repeated_ids_and_skewed_load(cuda):
    from triton_dist.kernels.amd import moe_dispatch_preprocess
    announce("moe preprocess skewed")
    g = torch.Generator().manual_seed(77)
    ids = torch.randint(0, 4, (3000, 8), generator=g).to(torch.int32)   # every wave sees long runs of equal ids
    ids[:, 0] = 0
    out = moe_dispatch_preprocess(ids.to(cuda), 64)
    torch.cuda.synchronize()
    want = golden.moe_preprocess(ids, 64)
    for a, b in zip(out, want[:4]):
        assert torch.equal(a.cpu(), b)


@pytest.mark.parametrize("launches", ["one", "one with rendezvous", "three"])
def test_preprocess_paths_sizes_in_turn_and_context_buffers(cuda, switches, launches):
    """The one-launch index build in both of its forms (up to 32 blocks every block counts all the ids itself; beyond,
    or forced here through the library's switch, the blocks exchange their histograms) and the three-launch form it
    falls back to (forced likewise; taken by itself beyond one block per compute unit, as the 560 000 ids below do):
    calls of different sizes in turn on the same cached scratch, id counts that are no multiple of four, ids outside
    [0, G) (dropped: scatter index -1), and the context-owned result tensors, two sets used in turn."""
    from triton_dist.kernels.amd import create_all_to_all_context, moe_dispatch_preprocess
    from triton_dist import _lib
    if launches == "three":
        switches(_lib.TDIST_DEBUG_MOE_INDEX_FORM, 3)
    if launches == "one with rendezvous":
        switches(_lib.TDIST_DEBUG_MOE_INDEX_FORM, 2)
    announce("moe preprocess paths (%s launch)" % launches)
    g = torch.Generator().manual_seed(9)
    for T, topk, G in [(4096, 8, 256), (300, 4, 2048), (70000, 8, 64), (1000, 8, 256), (5, 3, 4096), (333, 3, 100),
                       (3001, 5, 300), (20000, 8, 128), (8191, 8, 3500)]:
        ids = torch.randint(0, G, (T, topk), generator=g).to(torch.int32)
        out = moe_dispatch_preprocess(ids.to(cuda), G, want_topk_index=True)
        torch.cuda.synchronize()
        for a, b in zip(out, golden.moe_preprocess(ids, G)):
            assert torch.equal(a.cpu(), b), (T, topk, G)
    # ids outside the range take no place in the order
    T, topk, G = 777, 4, 32
    ids = torch.randint(0, G, (T, topk), generator=g).to(torch.int32)
    bad = torch.rand((T, topk), generator=g) < 0.1
    ids_bad = torch.where(bad, torch.where(torch.rand((T, topk), generator=g) < 0.5, torch.tensor(-1), torch.tensor(G + 5)), ids).int()
    splits, cumsum, scatter, gather = moe_dispatch_preprocess(ids_bad.to(cuda), G)
    torch.cuda.synchronize()
    flat, keep = ids_bad.view(-1), ~bad.view(-1)
    want_splits = torch.bincount(flat[keep].long(), minlength=G).int()
    assert torch.equal(splits.cpu(), want_splits) and torch.equal(cumsum.cpu(), golden.splits_to_cumsum(want_splits))
    order = torch.argsort(flat[keep], stable=True)
    want_scatter = torch.full((T * topk, ), -1, dtype=torch.int32)
    kept_pos = torch.nonzero(keep).view(-1)
    want_scatter[kept_pos[order]] = torch.arange(order.numel(), dtype=torch.int32)
    assert torch.equal(scatter.cpu().view(-1), want_scatter)
    assert torch.equal(gather.cpu()[:order.numel()], (kept_pos[order] // topk).int())
    # context-owned tensors: the result of a call stays valid through the next call
    ctx = create_all_to_all_context(64, 128, 0, 16, 4, 4, dtype=torch.float8_e4m3fn)
    ids_a = torch.randint(0, 16, (200, 4), generator=g).to(torch.int32)
    ids_b = torch.randint(0, 16, (200, 4), generator=g).to(torch.int32)
    out_a = moe_dispatch_preprocess(ids_a.to(cuda), 16, ctx=ctx)
    out_b = moe_dispatch_preprocess(ids_b.to(cuda), 16, ctx=ctx)
    torch.cuda.synchronize()
    for a, b in zip(out_a, golden.moe_preprocess(ids_a, 16)[:4]):
        assert torch.equal(a.cpu(), b)
    for a, b in zip(out_b, golden.moe_preprocess(ids_b, 16)[:4]):
        assert torch.equal(a.cpu(), b)
    out_c = moe_dispatch_preprocess(ids_a.to(cuda), 16, ctx=ctx)
    assert out_c[2].data_ptr() == out_a[2].data_ptr() and out_c[2].data_ptr() != out_b[2].data_ptr()
    # int64 ids (what torch.topk returns) on a shape the context has seen: converted into the context's own int32
    # staging tensor, the same two result sets in turn, nothing allocated
    ids64 = ids_b.long().to(cuda)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    out_d = moe_dispatch_preprocess(ids64, 16, ctx=ctx)
    out_e = moe_dispatch_preprocess(ids64.t().contiguous().t(), 16, ctx=ctx)    # and a non-contiguous view
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert out_d[2].data_ptr() == out_b[2].data_ptr() and out_e[2].data_ptr() == out_a[2].data_ptr()
    for got in (out_d, out_e):
        for a, b in zip(got, golden.moe_preprocess(ids_b, 16)[:4]):
            assert torch.equal(a.cpu(), b)


def test_splits_cumsum_entry_point(cuda):
    from triton_dist import _lib
    announce("moe splits_cumsum")
    ids, *_ = make_case(777, 8, 100, 16, seed=5)
    dev_ids = ids.to(cuda)
    splits = torch.empty(100, dtype=torch.int32, device=cuda)
    cumsum = torch.empty(101, dtype=torch.int32, device=cuda)
    ws = torch.zeros(_lib.load().tdist_moe_workspace_bytes(ids.numel(), 100), dtype=torch.uint8, device=cuda)
    _lib.call("tdist_moe_splits_cumsum", dev_ids.data_ptr(), ids.numel(), 100, splits.data_ptr(), cumsum.data_ptr(),
              ws.data_ptr(), ws.numel(), _lib.stream_ptr())
    torch.cuda.synchronize()
    want = torch.bincount(ids.view(-1).long(), minlength=100).int()
    assert torch.equal(splits.cpu(), want) and torch.equal(cumsum.cpu(), golden.splits_to_cumsum(want))
    # too small a workspace is refused
    assert _lib.load().tdist_moe_splits_cumsum(dev_ids.data_ptr(), ids.numel(), 100, splits.data_ptr(), cumsum.data_ptr(),
                                               ws.data_ptr(), 16, None) == _lib.TDIST_ERR_WORKSPACE


@pytest.mark.parametrize("T,topk,G,W,H,max_m,fused", [(4096, 8, 256, 32, 7168, 4096, True), (4096, 8, 256, 32, 7168, 4096, False),
                                                     (4096, 8, 256, 32, 7168, 4096, "tokens"), (96, 4, 16, 4, 48, 160, True),
                                                     (96, 4, 16, 4, 48, 160, "tokens"), (50, 3, 6, 2, 24, 40, False),
                                                     (50, 3, 6, 2, 24, 40, "tokens"), (10, 2, 8, 8, 1024, 8, True),
                                                     (10, 2, 8, 8, 1024, 8, "tokens"), (33, 5, 8, 2, 12000, 128, "tokens"),
                                                     (21, 3, 4, 4, 52, 64, "tokens"), (300, 4, 128, 64, 64, 48, "tokens"),
                                                     (300, 4, 126, 63, 64, 48, "tokens"), (300, 4, 160, 80, 64, 48, "tokens"),
                                                     (4096, 8, 256, 32, 7168, 4096, "ids"), (96, 4, 16, 4, 48, 160, "ids"), (50, 3, 6, 2, 24, 40, "ids"), (10, 2, 8, 8, 1024, 8, "ids"), (33, 5, 8, 2, 12000, 128, "ids"), (21, 3, 4, 4, 52, 64, "ids"), (300, 4, 128, 64, 64, 48, "ids"), (300, 4, 126, 63, 64, 48, "ids"), (300, 4, 160, 80, 64, 48, "ids"), (33, 5, 8, 2, 20000, 128, "ids"), (77, 3, 12, 4, 40000, 64, "ids"), (100, 7, 30, 5, 200, 300, "ids"),
                                                     (20, 2, 4, 2, 30000, 32, "ids"), (9000, 8, 64, 8, 64, 9100, "ids")])
def test_dispatch_bytes_bit_exact_and_round_trip(cuda, T, topk, G, W, H, max_m, fused):
    from triton_dist.kernels.amd import (all_to_all_post_process, create_all_to_all_context, fast_all_to_all,
                                         moe_dispatch_preprocess)
    announce("moe dispatch T=%d topk=%d G=%d W=%d H=%d max_m=%d fused=%s" % (T, topk, G, W, H, max_m, fused))
    Er = G // W
    ids, x, q, s, w = make_case(T, topk, G, H, seed=T * 3 + H)
    ctx = create_all_to_all_context(max_m, H, 0, G, W, Er, dtype=torch.float8_e4m3fn)
    ctx.recv_buf.view(torch.uint8).fill_(0xAB)
    splits, cumsum, scatter, gather = moe_dispatch_preprocess(ids.to(cuda), G)
    dq, ds = q.to(cuda), s.to(cuda)
    if fused == "ids":
        # straight from the raw expert ids (int64, as torch.topk gives them): index build and dispatch in one launch
        out_splits, recv, recv_scale = fast_all_to_all(ctx, dq, None, ds, expert_ids=ids.long().to(cuda))
        torch.cuda.synchronize()
        for got_t, want_t in zip(ctx.last_index, golden.moe_preprocess(ids, G)[:4]):
            assert torch.equal(got_t.cpu(), want_t), "index tensors written by the dispatch"
    elif fused == "tokens":
        out_splits, recv, recv_scale = fast_all_to_all(ctx, dq, cumsum, ds, scatter_index=scatter)
    elif fused:
        out_splits, recv, recv_scale = fast_all_to_all(ctx, dq, cumsum, ds, gather_index=gather)
    else:
        rows = torch.index_select(dq.view(torch.uint8), 0, gather.long()).view(torch.float8_e4m3fn)
        scales = torch.index_select(ds, 0, gather.long())
        out_splits, recv, recv_scale = fast_all_to_all(ctx, rows, cumsum, scales)
    torch.cuda.synchronize()
    w_splits, w_cumsum, w_scatter, w_gather, _ = golden.moe_preprocess(ids, G)
    sorted_rows = q.view(torch.uint8)[w_gather.long()]
    sorted_scales = s[w_gather.long()]
    assert torch.equal(out_splits.cpu(), w_splits)
    recv_u8 = recv.view(torch.uint8).cpu()
    recv_scale = recv_scale.cpu()
    for d in range(W):
        st, ed = int(w_cumsum[d * Er]), int(w_cumsum[(d + 1) * Er])
        n = min(ed - st, max_m)
        assert torch.equal(recv_u8[d * max_m:d * max_m + n], sorted_rows[st:st + n]), "slot %d rows" % d
        assert torch.equal(recv_scale[d * max_m:d * max_m + n], sorted_scales[st:st + n]), "slot %d scales" % d
        assert (recv_u8[d * max_m + n:(d + 1) * max_m] == 0xAB).all(), "slot %d: rows past the split were written" % d
    if max(int(w_cumsum[(d + 1) * Er] - w_cumsum[d * Er]) for d in range(W)) <= max_m:
        out, out_scale = all_to_all_post_process(ctx, out_splits, recv, recv_scale.to(cuda))
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.uint8).cpu(), sorted_rows)
        assert torch.equal(out_scale.cpu(), sorted_scales)


def test_dispatch_from_ids_matches_the_two_calls_with_ids_out_of_range(cuda):
    """The one-launch form against index build + token-major dispatch on ids of which some lie outside [0, G) (they
    take no place and their rows are not sent) and some repeat within a token: the same slot bytes, scales, splits and
    index tensors; three calls in a row on one context (its two sets of index tensors and receive buffers in turn)."""
    from triton_dist.kernels.amd import create_all_to_all_context, fast_all_to_all, moe_dispatch_preprocess
    announce("moe dispatch from ids, ids out of range")
    T, topk, G, W, H, max_m = 333, 6, 24, 4, 272, 700
    g = torch.Generator().manual_seed(4)
    ctx_a = create_all_to_all_context(max_m, H, 0, G, W, G // W, dtype=torch.float8_e4m3fn)
    ctx_b = create_all_to_all_context(max_m, H, 0, G, W, G // W, dtype=torch.float8_e4m3fn)
    for call in range(3):
        ids = torch.randint(-2, G + 3, (T, topk), generator=g).to(torch.int32)
        q, s_ = golden.quantize_per_token_e4m3(torch.randn((T, H), generator=g))
        for ctx in (ctx_a, ctx_b):
            ctx.recv_buf.view(torch.uint8).fill_(0xAB)
            ctx.scale_recv_buf.fill_(-1.0)
        dq, ds, dids = q.to(cuda), s_.to(cuda), ids.to(cuda)
        splits, cumsum, scatter, gather = moe_dispatch_preprocess(dids, G, ctx=ctx_a)
        want = fast_all_to_all(ctx_a, dq, cumsum, ds, scatter_index=scatter)
        got = fast_all_to_all(ctx_b, dq, None, ds, expert_ids=dids)
        torch.cuda.synchronize()
        n_valid = int(cumsum[-1])
        for a, b in zip(got, want):
            assert torch.equal(a.view(torch.uint8), b.view(torch.uint8)), "call %d" % call
        i_splits, i_cumsum, i_scatter, i_gather = ctx_b.last_index
        assert torch.equal(i_splits, splits) and torch.equal(i_cumsum, cumsum) and torch.equal(i_scatter, scatter)
        assert torch.equal(i_gather[:n_valid], gather[:n_valid])


def test_dispatch_bf16_rows_without_scales_and_odd_row_bytes(cuda):
    from triton_dist.kernels.amd import create_all_to_all_context, fast_all_to_all, moe_dispatch_preprocess
    announce("moe dispatch bf16 H=36 (72-byte rows: scalar copy path)")
    T, topk, G, W, H, max_m = 40, 2, 4, 2, 36, 64
    g = torch.Generator().manual_seed(12)
    ids = golden.random_distinct_experts(T, G, topk, g)
    x = torch.randn((T, H), generator=g).to(torch.bfloat16)
    ctx = create_all_to_all_context(max_m, H, 0, G, W, G // W, dtype=torch.bfloat16)
    splits, cumsum, scatter, gather = moe_dispatch_preprocess(ids.to(cuda), G)
    rows = x.to(cuda)[gather.long()]
    out_splits, recv, none = fast_all_to_all(ctx, rows, cumsum, None)
    torch.cuda.synchronize()
    assert none is None
    w_splits, w_cumsum, _, w_gather, _ = golden.moe_preprocess(ids, G)
    _, want, _ = golden.dispatch_slots(x[w_gather.long()], None, w_cumsum, W, G // W, max_m)
    got = recv.view(torch.uint8).cpu()
    for d in range(W):
        n = int(w_cumsum[(d + 1) * (G // W)] - w_cumsum[d * (G // W)])
        assert torch.equal(got[d * max_m:d * max_m + n], want[d * max_m:d * max_m + n])
    assert torch.equal(out_splits.cpu(), w_splits)


def test_context_double_buffering(cuda):
    from triton_dist.kernels.amd import create_all_to_all_context, fast_all_to_all
    announce("moe ctx act_pos alternates")
    ctx = create_all_to_all_context(8, 16, 0, 2, 2, 1, dtype=torch.bfloat16)
    cumsum = torch.tensor([0, 2, 4], dtype=torch.int32, device=cuda)
    a = torch.ones((4, 16), dtype=torch.bfloat16, device=cuda)
    r1 = fast_all_to_all(ctx, a, cumsum, None)[1]
    r2 = fast_all_to_all(ctx, a * 2, cumsum, None)[1]
    r3 = fast_all_to_all(ctx, a * 3, cumsum, None)[1]
    torch.cuda.synchronize()
    assert r1.data_ptr() != r2.data_ptr() and r1.data_ptr() == r3.data_ptr()   # reference :195, :239
    assert float(r2[0, 0]) == 2.0 and float(r3[0, 0]) == 3.0 and float(r3[8, 0]) == 3.0


@pytest.mark.parametrize("T,topk,G,W,H,max_m", [(4096, 8, 256, 32, 7168, 4096), (96, 4, 16, 4, 64, 160), (7, 3, 8, 2, 16, 32),
                                                (300, 4, 128, 64, 1040, 48), (300, 4, 126, 63, 1040, 48),
                                                (300, 4, 160, 80, 1040, 48), (40, 12, 24, 3, 2064, 512)])
def test_weighted_combine(cuda, T, topk, G, W, H, max_m):
    from triton_dist.kernels.amd import (create_all_to_all_context, fast_all_to_all, moe_dispatch_preprocess,
                                         moe_weighted_combine)
    announce("moe combine T=%d topk=%d G=%d H=%d" % (T, topk, G, H))
    ids, x, q, s, w = make_case(T, topk, G, H, seed=T + 99)
    ctx = create_all_to_all_context(max_m, H, 0, G, W, G // W, dtype=torch.float8_e4m3fn)
    splits, cumsum, scatter, gather = moe_dispatch_preprocess(ids.to(cuda), G)
    out_splits, recv, recv_scale = fast_all_to_all(ctx, q.to(cuda), cumsum, s.to(cuda), gather_index=gather)
    y = moe_weighted_combine(ctx, recv, recv_scale, scatter, w.to(cuda), cumsum)
    torch.cuda.synchronize()
    _, _, w_scatter, w_gather, _ = golden.moe_preprocess(ids, G)
    ref = golden.weighted_combine(q[w_gather.long()].float(), s[w_gather.long()], w_scatter, w)
    assert golden.max_rel_err(y.float().cpu(), ref) <= 1e-2
    # the weights of a token sum to 1 and its topk copies are one row: y is the dequantised token
    deq = q.float() * s[:, None]
    assert golden.max_rel_err(y.float().cpu(), deq) <= 1e-2


def test_combine_reference_round_trip_bf16(cuda):
    """dispatch -> combine with unit weights gives topk * input (test_all_to_all.py:366-370)."""
    from triton_dist.kernels.amd import (all_to_all_post_process, create_all_to_all_context, fast_all_to_all,
                                         moe_dispatch_preprocess, moe_weighted_combine, splits_to_cumsum)
    announce("moe round trip bf16")
    T, topk, G, W, H, max_m = 128, 4, 32, 8, 256, 128
    g = torch.Generator().manual_seed(21)
    ids = golden.random_distinct_experts(T, G, topk, g)
    x = torch.randn((T, H), generator=g).to(torch.bfloat16)
    ctx = create_all_to_all_context(max_m, H, 0, G, W, G // W, dtype=torch.bfloat16)
    splits, cumsum, scatter, gather = moe_dispatch_preprocess(ids.to(cuda), G)
    d_splits, d_tok, _ = fast_all_to_all(ctx, x.to(cuda), cumsum, None, gather_index=gather)
    tok, _ = all_to_all_post_process(ctx, d_splits, d_tok)
    c_splits, c_tok, _ = fast_all_to_all(ctx, tok, splits_to_cumsum(d_splits), None)
    y_slots = moe_weighted_combine(ctx, c_tok, None, scatter, None, cumsum)
    tok2, _ = all_to_all_post_process(ctx, c_splits, c_tok)
    y_compact = moe_weighted_combine(None, tok2, None, scatter, None, from_slots=False)
    torch.cuda.synchronize()
    torch.testing.assert_close(y_slots.float().cpu(), x.float() * topk, rtol=1e-2, atol=1e-2)
    assert torch.equal(y_slots, y_compact)


@pytest.mark.parametrize("R,T,topk,E,BS,dtype", [(1, 4, 3, 4, 4, torch.int64), (8, 1024, 8, 256, 128, torch.int64),
                                                 (8, 512, 6, 64, 64, torch.int32), (3, 37, 4, 11, 8, torch.int64),
                                                 (2, 5, 2, 300, 1, torch.int32), (4, 1, 1, 1, 16, torch.int64),
                                                 (16, 96, 8, 256, 128, torch.int64), (5, 300, 2, 7, 256, torch.int32),
                                                 (8, 1024, 6, 64, 128, torch.int64), (3, 5461, 4, 32, 16, torch.int32),
                                                 (2, 40000, 1, 8, 64, torch.int64)])
@pytest.mark.parametrize("launches", ["one", "three"])
def test_align_sort_bit_exact(cuda, switches, R, T, topk, E, BS, dtype, launches):
    """sort_topk_ids_align_block_size against the oracle (the reference's align kernel restated): the one-launch form
    that up to 65 536 entries take (blocks of 512 or of 1024 entries; 4096 groups do not fit it) and the three
    launches behind it."""
    from triton_dist import _lib
    from triton_dist.kernels.nvidia import sort_topk_ids_align_block_size
    if launches == "three":
        switches(_lib.TDIST_DEBUG_MOE_INDEX_FORM, 3)
    announce("moe align R=%d T=%d topk=%d E=%d BS=%d (%s)" % (R, T, topk, E, BS, launches))
    g = torch.Generator().manual_seed(R * 1000 + T + E)
    if topk <= E:
        ids = torch.stack([torch.randperm(E, generator=g)[:topk] for _ in range(R * T)])
    else:
        ids = torch.randint(0, E, (R * T, topk), generator=g)
    if E > 4:
        ids[ids == 3] = 2   # leave an expert without tokens
    want = golden.sort_topk_ids_align_block_size(ids, E, R, T, BS)
    got = sort_topk_ids_align_block_size(ids.to(dtype).to(cuda), E, R, T, BS)
    torch.cuda.synchronize()
    n = want[4]
    assert int(got[4].item()) == n
    assert torch.equal(got[0].cpu(), want[0])                 # whole buffer: padding positions included
    nb = n // BS
    assert torch.equal(got[1].cpu()[:nb], want[1]) and torch.equal(got[2].cpu()[:nb], want[2])
    assert torch.equal(got[3].cpu(), want[3])


def test_align_sort_rejects_too_many_groups(cuda):
    from triton_dist import _lib
    from triton_dist.kernels.amd import sort_topk_ids_align_block_size
    ids = torch.zeros((64, 2), dtype=torch.int64, device=cuda)
    with pytest.raises(_lib.TdistError):
        sort_topk_ids_align_block_size(ids, 1024, 8, 8, 16)


@pytest.mark.parametrize("m,N", [(1, 128), (37, 1024), (64, 7168), (5, 2176)])
def test_group_quantiser_bit_exact(cuda, m, N):
    from triton_dist.kernels.amd import quant_bf16_fp8
    announce("group quant m=%d N=%d" % (m, N))
    g = torch.Generator().manual_seed(m + N)
    mags = torch.tensor([1e-4, 1e-2, 1.0, 3.0, 100.0, 3e4])[torch.randint(0, 6, (m, 1), generator=g)]
    x = (torch.randn((m, N), generator=g) * mags).to(torch.bfloat16)
    x[0, :8] = torch.tensor([0.0, -0.0, 1.0, -1.0, 0.5, 3.0, 448.0, -448.0]).to(torch.bfloat16)
    want_q, want_s = golden.quantize_groups_e4m3(x)
    got_q, got_s = quant_bf16_fp8(x.to(cuda))
    torch.cuda.synchronize()
    assert torch.equal(got_s.cpu(), want_s)
    assert torch.equal(got_q.cpu().view(torch.uint8), want_q.view(torch.uint8))


@pytest.mark.parametrize("T,topk,G,W,H,max_m", [(4096, 8, 256, 32, 7168, 4096), (96, 4, 16, 4, 256, 160), (33, 5, 8, 2, 1152, 128),
                                                (300, 4, 128, 64, 128, 48)])
def test_dispatch_with_online_quantisation_and_grouped_combine(cuda, T, topk, G, W, H, max_m):
    """The fused path: bf16 tokens in, e4m3 slot rows + group scales out (bit-exact against quantise-then-dispatch),
    then the weighted combine reading the group scales."""
    from triton_dist.kernels.amd import (create_all_to_all_context, fast_all_to_all, moe_dispatch_preprocess,
                                         moe_weighted_combine)
    announce("moe online quant T=%d topk=%d G=%d H=%d" % (T, topk, G, H))
    ids, x, _, _, w = make_case(T, topk, G, H, seed=T + 7)
    xb = x.to(torch.bfloat16)
    q, s = golden.quantize_groups_e4m3(xb)
    ctx = create_all_to_all_context(max_m, H, 0, G, W, G // W, dtype=torch.float8_e4m3fn, fp8_group_size=128)
    ctx.recv_buf.view(torch.uint8).zero_()
    ctx.scale_recv_buf.zero_()
    splits, cumsum, scatter, gather = moe_dispatch_preprocess(ids.to(cuda), G)
    o_splits, recv, recv_scale = fast_all_to_all(ctx, xb.to(cuda), cumsum, None, scatter_index=scatter, online_quant_fp8=True)
    torch.cuda.synchronize()
    # expected slots: sorted row p = token gather[p]; destination d takes rows [cumsum[d*Er], cumsum[(d+1)*Er])
    w_splits, w_cumsum, w_scatter, w_gather, _ = golden.moe_preprocess(ids, G)
    Er = G // W
    exp_rows = torch.zeros((W * max_m, H), dtype=torch.uint8)
    exp_scale = torch.zeros((W * max_m, H // 128))
    for d in range(W):
        lo, hi = int(w_cumsum[d * Er]), int(w_cumsum[(d + 1) * Er])
        n = min(hi - lo, max_m)
        tok = w_gather[lo:lo + n].long()
        exp_rows[d * max_m:d * max_m + n] = q.view(torch.uint8)[tok]
        exp_scale[d * max_m:d * max_m + n] = s[tok]
    assert torch.equal(o_splits.cpu(), w_splits)
    assert torch.equal(recv.view(torch.uint8).cpu(), exp_rows)
    assert torch.equal(recv_scale.cpu(), exp_scale)
    y = moe_weighted_combine(ctx, recv, recv_scale, scatter, w.to(cuda), cumsum)
    torch.cuda.synchronize()
    deq = q.float().view(T, H // 128, 128) * s[..., None]
    ref = (deq.view(T, H) * w.sum(-1, keepdim=True))           # every copy of token t carries token t's row
    assert golden.max_rel_err(y.float().cpu(), ref) <= 1e-2
