"""(d) split-KV flash decode and the LSE merges on the GPU against the oracle.
Bar: <= 2e-3 absolute on outputs and LSE against the exact fp64 closed form, with no allowance. A 16-bit final
output is checked in two parts that together say the same thing: the merge's fp32 result is within 2e-3 of the exact
value, and the 16-bit output is exactly that fp32 result rounded to nearest even (the one step no kernel can avoid).
The 16-bit output is also held to the reference's own golden at the reference test's tolerance (atol = rtol = 1e-2,
test/nvidia/test_decode_attn.py:164)."""
import math

import pytest
import torch

from oracle import golden
from tests.conftest import announce

pytestmark = pytest.mark.gpu

ATOL = 2e-3


def assert_final_output(out16, out32, exact):
    """``out32``: the merge's result as fp32, ``out16``: the same call's 16-bit output."""
    assert out32.dtype == torch.float32
    err = float((out32.cpu().double() - exact).abs().max())
    assert err <= ATOL, "fp32 result off by %g" % err
    assert torch.equal(out16.view(torch.int16), out32.to(out16.dtype).view(torch.int16)), \
        "the 16-bit output must be the fp32 result rounded to nearest even"


def merged_fp32(out_split, lse_split, S, lens_dev):
    """The merge of the splits with an fp32 result (the same kernel that writes the 16-bit output)."""
    from triton_dist.kernels.amd.flash_decode import decode_combine
    B, Hq, _, dv = out_split.shape
    out32 = torch.empty((B, Hq, dv), dtype=torch.float32, device=out_split.device)
    decode_combine(out_split, lse_split, S, 1, lens_dev, B, Hq, dv,
                   (out_split.stride(2), out_split.stride(0), out_split.stride(1)),
                   (lse_split.stride(2), lse_split.stride(0), lse_split.stride(1)), out32)
    return out32


def build_case(kv_lens, heads, head_size, block_size, dtype, seed, num_pages=None, v_head_size=None):
    g = torch.Generator().manual_seed(seed)
    Hq, Hkv = heads
    B = len(kv_lens)
    q = torch.randn((B, Hq, head_size), generator=g).to(dtype)
    k_cache, v_cache, table = golden.make_paged_kv(B, max(max(kv_lens), 1), Hkv, head_size, block_size, dtype, g,
                                                   v_head_dim=v_head_size)
    return q, k_cache, v_cache, table


# the reference's own grid (test/nvidia/test_decode_attn.py:126-131) in both 16-bit dtypes
@pytest.mark.parametrize("kv_lens", [[1320, 18, 463], [1, 54, 293, 70]])
@pytest.mark.parametrize("num_heads", [(16, 16), (32, 8), (64, 8), (6, 1)])
@pytest.mark.parametrize("head_size", [128, 256])
@pytest.mark.parametrize("block_size", [1, 16])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("soft_cap", [0, 30, 50])
def test_decode_with_paged_kv(cuda, kv_lens, num_heads, head_size, dtype, block_size, soft_cap):
    from triton_dist.kernels.nvidia import gqa_fwd_batch_decode
    announce("decode kv_lens=%s heads=%s D=%d page=%d %s cap=%s" % (kv_lens, num_heads, head_size, block_size, dtype, soft_cap))
    q, k_cache, v_cache, table = build_case(kv_lens, num_heads, head_size, block_size, dtype, seed=sum(kv_lens) + head_size)
    scale = head_size**-0.5
    B = len(kv_lens)
    workspace = torch.zeros([B * num_heads[0] * 32], dtype=torch.int32, device=cuda)
    lens_dev = torch.tensor(kv_lens, dtype=torch.int32, device=cuda)
    qd, kd, vd, td = q.to(cuda), k_cache.to(cuda), v_cache.to(cuda), table.to(cuda)
    out = gqa_fwd_batch_decode(qd, kd, vd, workspace, [1] * B, lens_dev, td, scale, soft_cap)
    out32 = gqa_fwd_batch_decode(qd, kd, vd, workspace, [1] * B, lens_dev, td, scale, soft_cap,
                                 output_combine=torch.empty((B, num_heads[0], head_size), dtype=torch.float32, device=cuda))
    torch.cuda.synchronize()
    ref = golden.ref_paged_attn(q, k_cache, v_cache, [1] * B, kv_lens, table, scale, soft_cap)
    torch.testing.assert_close(out.cpu().float(), ref.float(), atol=1e-2, rtol=1e-2)
    exact, _ = golden.decode_exact(q, k_cache, v_cache, kv_lens, table, scale, soft_cap)
    assert_final_output(out, out32, exact)


@pytest.mark.parametrize("kv_lens,S", [([1320, 18, 463, 5], 32), ([1, 54, 293, 70], 16), ([2048, 2047, 33, 16], 8), ([100], 1)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_split_partials_and_lse(cuda, kv_lens, S, dtype):
    from triton_dist.kernels.amd.flash_decode import _split_kv
    announce("decode partials kv_lens=%s S=%d %s" % (kv_lens, S, dtype))
    heads, D, page = (64, 8), 128, 16
    q, k_cache, v_cache, table = build_case(kv_lens, heads, D, page, dtype, seed=S)
    scale = D**-0.5
    lens_dev = torch.tensor(kv_lens, dtype=torch.int32, device=cuda)
    out_split, lse_split, _ = _split_kv(q.to(cuda), k_cache.to(cuda), v_cache.to(cuda), lens_dev, table.to(cuda), scale, 0.0, S)
    torch.cuda.synchronize()
    w_out, w_lse = golden.decode_split_exact(q, k_cache, v_cache, kv_lens, table, scale, S)
    got_lse = lse_split.cpu().double()
    empty = torch.isinf(w_lse)
    assert torch.equal(torch.isinf(got_lse), empty), "empty splits must carry LSE = -inf"
    assert (got_lse[~empty] - w_lse[~empty]).abs().max() <= ATOL
    assert (out_split.cpu().double() - w_out).abs().max() <= ATOL
    assert (out_split.cpu()[empty] == 0).all()


@pytest.mark.parametrize("dims", [(192, 128), (576, 512)])
@pytest.mark.parametrize("num_heads,kv_lens,S", [((16, 16), [1320, 18, 463], 4), ((32, 8), [1, 54, 293, 70], 8),
                                                  ((6, 1), [777, 16, 5], 3), ((128, 1), [300, 33], 2)])
@pytest.mark.parametrize("block_size", [1, 16])
@pytest.mark.parametrize("dtype,soft_cap", [(torch.bfloat16, 0), (torch.float16, 30)])
def test_heads_with_extra_key_dimensions(cuda, dims, num_heads, kv_lens, S, block_size, dtype, soft_cap):
    """Key dimension 192 = 128 + 64 and 576 = 512 + 64 with value dimension 128 / 512 (the reference's BLOCK_DPE
    heads, flash_decode.py:771-772,186-190,209-213): per-split partials and LSE, then the merged output."""
    from triton_dist.kernels.amd.flash_decode import _split_kv
    from triton_dist.kernels.nvidia import gqa_fwd_batch_decode
    dk, dv = dims
    announce("decode dims=%s heads=%s kv_lens=%s S=%d page=%d %s cap=%s" % (dims, num_heads, kv_lens, S, block_size, dtype, soft_cap))
    q, k_cache, v_cache, table = build_case(kv_lens, num_heads, dk, block_size, dtype, seed=dk + S, v_head_size=dv)
    scale = dk**-0.5
    B = len(kv_lens)
    lens_dev = torch.tensor(kv_lens, dtype=torch.int32, device=cuda)
    qd, kd, vd, td = q.to(cuda), k_cache.to(cuda), v_cache.to(cuda), table.to(cuda)
    out_split, lse_split, _ = _split_kv(qd, kd, vd, lens_dev, td, scale, soft_cap, S)
    torch.cuda.synchronize()
    w_out, w_lse = golden.decode_split_exact(q, k_cache, v_cache, kv_lens, table, scale, S, soft_cap)
    got_lse = lse_split.cpu().double()
    empty = torch.isinf(w_lse)
    assert torch.equal(torch.isinf(got_lse), empty)
    assert (got_lse[~empty] - w_lse[~empty]).abs().max() <= ATOL
    assert (out_split.cpu().double() - w_out).abs().max() <= ATOL
    out = gqa_fwd_batch_decode(qd, kd, vd, None, [1] * B, lens_dev, td, scale, soft_cap, kv_split=S)
    out32 = gqa_fwd_batch_decode(qd, kd, vd, None, [1] * B, lens_dev, td, scale, soft_cap, kv_split=S,
                                 output_combine=torch.empty((B, num_heads[0], dv), dtype=torch.float32, device=cuda))
    torch.cuda.synchronize()
    assert out.shape == (B, num_heads[0], dv)
    exact, _ = golden.decode_exact(q, k_cache, v_cache, kv_lens, table, scale, soft_cap)
    assert_final_output(out, out32, exact)


@pytest.mark.parametrize("num_heads,dims", [((64, 8), (128, 128)), ((6, 1), (128, 128)), ((40, 2), (64, 64)),
                                            ((16, 16), (192, 128)), ((32, 2), (256, 256)), ((16, 1), (576, 512))])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_fused_decode_is_the_two_launch_result(cuda, num_heads, dims, dtype):
    """One launch (the last workgroup of a sequence and head block merges the splits) against split-KV followed by
    the combine: bit-identical outputs and LSE, three calls in a row on the same counters with different lengths
    (empty splits, a sequence of length 0), counters back at zero after each; and the oracle's bar."""
    from triton_dist.kernels.amd.flash_decode import _split_kv, decode_combine, decode_fused, gqa_fwd_batch_decode_persistent
    dk, dv = dims
    Hq, Hkv = num_heads
    page = 16
    counters = torch.zeros(4096, dtype=torch.int32, device=cuda)
    for call, (kv_lens, S) in enumerate([([1320, 18, 463, 5], 32), ([40, 0, 7, 2047], 16), ([100, 3, 64, 1], 1)]):
        announce("fused decode heads=%s dims=%s %s kv_lens=%s S=%d" % (num_heads, dims, dtype, kv_lens, S))
        q, k_cache, v_cache, table = build_case(kv_lens, num_heads, dk, page, dtype, seed=call + dk, v_head_size=dv)
        scale = dk**-0.5
        B = len(kv_lens)
        lens_dev = torch.tensor(kv_lens, dtype=torch.int32, device=cuda)
        qd, kd, vd, td = q.to(cuda), k_cache.to(cuda), v_cache.to(cuda), table.to(cuda)
        out_split, lse_split, _ = _split_kv(qd, kd, vd, lens_dev, td, scale, 0.0, S)
        want = torch.empty((B, Hq, dv), dtype=dtype, device=cuda)
        want_lse = torch.empty((B, Hq), dtype=torch.float32, device=cuda)
        decode_combine(out_split, lse_split, S, 1, lens_dev, B, Hq, dv,
                       (out_split.stride(2), out_split.stride(0), out_split.stride(1)),
                       (lse_split.stride(2), lse_split.stride(0), lse_split.stride(1)), want, want_lse)
        got = torch.full((B, Hq, dv), float("nan"), dtype=dtype, device=cuda)
        got_lse = torch.full((B, Hq), float("nan"), dtype=torch.float32, device=cuda)
        decode_fused(qd, kd, vd, lens_dev, td, scale, 0.0, S, got, got_lse, workspace=counters)
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), "fused output differs from split + combine"
        assert torch.equal(got_lse.view(torch.int32), want_lse.view(torch.int32))
        assert int(counters.abs().sum()) == 0, "the arrival counters must be left at zero"
        exact, exact_lse = golden.decode_exact(q, k_cache, v_cache, kv_lens, table, scale)
        assert_final_output(got, merged_fp32(out_split, lse_split, S, lens_dev), exact)
        live = ~torch.isinf(exact_lse)
        assert torch.equal(torch.isinf(got_lse.cpu()), ~live)
        assert (got_lse.cpu().double()[live] - exact_lse[live]).abs().max() <= ATOL
    # the launcher with the reference's signature (the library's own counters, default output); a caller's workspace
    # full of garbage, as torch.empty may hand it out, must not matter
    garbage = torch.full((4096,), 0x7B7B7B7B, dtype=torch.int32, device=cuda)
    out = gqa_fwd_batch_decode_persistent(qd, kd, vd, garbage, [1] * B, lens_dev, td, scale, kv_split=S)
    torch.cuda.synchronize()
    assert torch.equal(out.view(torch.int16), want.view(torch.int16))
    assert int((garbage != 0x7B7B7B7B).sum()) == 0
    with pytest.raises(ValueError):
        decode_fused(qd, kd, vd, lens_dev, td, scale, 0.0, S, got, got_lse, workspace=torch.zeros(4, dtype=torch.int64, device=cuda))


def test_page_indices_beyond_2_31_bytes(cuda):
    """Pages far apart: byte offsets above 2^31 (the reference sizes NUM_BLOCKS = 32000 for this,
    test_decode_attn.py:123)."""
    from triton_dist.kernels.nvidia import gqa_fwd_batch_decode
    announce("decode large page indices")
    Hq, Hkv, D, page = 16, 8, 128, 16
    num_pages = 100000                     # 100000 * 16*8*128*2 B = 3.3 GB per cache
    kv_lens = [70, 300]
    g = torch.Generator().manual_seed(3)
    q = torch.randn((2, Hq, D), generator=g).to(torch.bfloat16)
    k_dev = torch.zeros((num_pages, page, Hkv, D), dtype=torch.bfloat16, device=cuda)
    v_dev = torch.zeros_like(k_dev)
    pages_per_seq = (max(kv_lens) + page - 1) // page
    table = torch.stack([torch.arange(num_pages - 1 - b, num_pages - 1 - b - 2 * pages_per_seq, -2)[:pages_per_seq] for b in range(2)]).int()
    used = table.flatten().long()
    k_small = torch.randn((used.numel(), page, Hkv, D), generator=g).to(torch.bfloat16)
    v_small = torch.randn((used.numel(), page, Hkv, D), generator=g).to(torch.bfloat16)
    k_dev[used.to(cuda)] = k_small.to(cuda)
    v_dev[used.to(cuda)] = v_small.to(cuda)
    lens_dev = torch.tensor(kv_lens, dtype=torch.int32, device=cuda)
    out = gqa_fwd_batch_decode(q.to(cuda), k_dev, v_dev, None, [1, 1], lens_dev, table.to(cuda), D**-0.5, kv_split=4)
    out32 = gqa_fwd_batch_decode(q.to(cuda), k_dev, v_dev, None, [1, 1], lens_dev, table.to(cuda), D**-0.5, kv_split=4,
                                 output_combine=torch.empty((2, Hq, D), dtype=torch.float32, device=cuda))
    torch.cuda.synchronize()
    small_table = torch.arange(used.numel(), dtype=torch.int32).view(2, pages_per_seq)
    exact, _ = golden.decode_exact(q, k_small, v_small, kv_lens, small_table, D**-0.5)
    assert_final_output(out, out32, exact)


def test_inter_rank_combine_and_layer(cuda):
    """One rank's shard plus synthetic peers, merged by LSE (layers/nvidia/sp_flash_decode_layer.py:142-182,
    kernels/nvidia/flash_decode.py:512-532); a peer with kv_len 0 is skipped."""
    from triton_dist.layers.nvidia import SpGQAFlashDecodeAttention
    announce("SP decode layer, 4 ranks")
    R, rank, B, Hq, Hkv, D, page = 4, 1, 3, 32, 4, 128, 16
    kv_lens = [500, 64, 1]
    g = torch.Generator().manual_seed(17)
    q = torch.randn((B, Hq, D), generator=g).to(torch.bfloat16)
    k_cache, v_cache, table = golden.make_paged_kv(B, max(kv_lens), Hkv, D, page, torch.bfloat16, g)
    global_lens = torch.tensor([[300, 0, 7], kv_lens, [0, 0, 0], [10, 20, 30]], dtype=torch.int32)
    peer_out = torch.randn((R, B, Hq, D), generator=g)
    peer_lse = torch.randn((R, B, Hq), generator=g) * 2 + math.log(100.0)
    layer = SpGQAFlashDecodeAttention(rank, 0, R, 1, Hq, Hkv, D, D, page_size=page, scale=D**-0.5, max_allowed_batch=B)
    from triton_dist.kernels.amd import gqa_fwd_batch_decode_inter_rank_combine
    all_out, all_lse = peer_out.to(cuda), peer_lse.to(cuda)
    out = layer(q.to(cuda), k_cache.to(cuda), v_cache.to(cuda), global_lens.to(cuda), table.to(cuda),
                peer_partials=(all_out, all_lse))
    # the same merge with an fp32 result (the gather buffers now hold the own shard in row `rank`)
    out32 = gqa_fwd_batch_decode_inter_rank_combine(all_out, all_lse, global_lens.to(cuda), out_dtype=torch.float32)
    torch.cuda.synchronize()
    own, own_lse = golden.decode_exact(q, k_cache, v_cache, kv_lens, table, D**-0.5)
    all_out = peer_out.double().clone()
    all_lse = peer_lse.double().clone()
    all_out[rank], all_lse[rank] = own, own_lse
    skip = (global_lens == 0)[:, :, None].expand(R, B, Hq)
    want, _ = golden.lse_merge(all_out, all_lse, skip)
    assert out.dtype == torch.bfloat16 and out.shape == (B, Hq, D)
    assert_final_output(out, out32, want)


def test_combine_all_partials_skipped_gives_zero(cuda):
    from triton_dist.kernels.amd import gqa_fwd_batch_decode_inter_rank_combine
    announce("inter-rank combine, everything skipped")
    out = gqa_fwd_batch_decode_inter_rank_combine(torch.ones((2, 1, 4, 64), device=cuda), torch.zeros((2, 1, 4), device=cuda),
                                                  torch.zeros((2, 1), dtype=torch.int32, device=cuda))
    torch.cuda.synchronize()
    assert (out == 0).all()


def test_full_size_shard_sampled(cuda):
    """BASELINE config 5 at full size (B 32, Hq 64, Hkv 8, D 128, 32768 keys, 16 splits, page 16), checked on
    two sequences against the exact closed form, and through the merge identity on all of them."""
    from triton_dist.kernels.amd.flash_decode import _split_kv, decode_combine
    announce("decode full size C5")
    B, Hq, Hkv, D, L, S, page = 32, 64, 8, 128, 32768, 16, 16
    g = torch.Generator(device="cuda").manual_seed(5)
    pages_per_seq = L // page
    num_pages = B * pages_per_seq
    k_dev = torch.randn((num_pages, page, Hkv, D), generator=g, device=cuda, dtype=torch.float32).to(torch.bfloat16)
    v_dev = torch.randn((num_pages, page, Hkv, D), generator=g, device=cuda, dtype=torch.float32).to(torch.bfloat16)
    q_dev = torch.randn((B, Hq, D), generator=g, device=cuda, dtype=torch.float32).to(torch.bfloat16)
    table = torch.randperm(num_pages, generator=torch.Generator().manual_seed(6)).view(B, pages_per_seq).int()
    lens_dev = torch.full((B, ), L, dtype=torch.int32, device=cuda)
    scale = D**-0.5
    out_split, lse_split, _ = _split_kv(q_dev, k_dev, v_dev, lens_dev, table.to(cuda), scale, 0.0, S)
    merged = torch.empty((B, Hq, D), dtype=torch.float32, device=cuda)
    merged_lse = torch.empty((B, Hq), dtype=torch.float32, device=cuda)
    decode_combine(out_split, lse_split, S, 1, lens_dev, B, Hq, D,
                   (out_split.stride(2), out_split.stride(0), out_split.stride(1)),
                   (lse_split.stride(2), lse_split.stride(0), lse_split.stride(1)), merged, merged_lse)
    torch.cuda.synchronize()
    # merge identity on every sequence: the closed-form merge of the GPU's partials equals the GPU's merge
    w_merged, w_lse = golden.lse_merge(out_split.cpu().permute(2, 0, 1, 3), lse_split.cpu().permute(2, 0, 1))
    assert (merged.cpu().double() - w_merged).abs().max() <= 1e-5
    assert (merged_lse.cpu().double() - w_lse).abs().max() <= 1e-4
    # exact closed form on two sequences (their pages only)
    for b in (0, 31):
        pages = table[b].long()
        k_b = k_dev[pages.to(cuda)].cpu()
        v_b = v_dev[pages.to(cuda)].cpu()
        t_b = torch.arange(pages_per_seq, dtype=torch.int32).view(1, -1)
        exact, exact_lse = golden.decode_exact(q_dev[b:b + 1].cpu(), k_b, v_b, [L], t_b, scale)
        assert (merged[b].cpu().double() - exact[0]).abs().max() <= ATOL
        assert (merged_lse[b].cpu().double() - exact_lse[0]).abs().max() <= ATOL


@pytest.mark.parametrize("S", [16, 32])
def test_full_size_shard_with_pages_of_one_token(cuda, S):
    """BASELINE config 5 at full size with the reference layer's default page size of one token
    (layers/nvidia/sp_flash_decode_layer.py:45; its test grid has block_size 1, test/nvidia/test_decode_attn.py:129)
    and with its default of 32 splits (:61) beside the config's 16: every token of every sequence at a random place of
    the cache (a 4.19 MB block table, 2 KB gather granules). Checked like the page-16 case: the merge identity on all
    32 sequences, the exact closed form on two of them, and the one-launch form bit for bit against split + combine."""
    from triton_dist.kernels.amd.flash_decode import _split_kv, decode_combine, decode_fused
    announce("decode full size C5, pages of one token, %d splits" % S)
    B, Hq, Hkv, D, L = 32, 64, 8, 128, 32768
    g = torch.Generator(device="cuda").manual_seed(5)
    k_dev = torch.randn((B * L, 1, Hkv, D), generator=g, device=cuda, dtype=torch.float32).to(torch.bfloat16)
    v_dev = torch.randn((B * L, 1, Hkv, D), generator=g, device=cuda, dtype=torch.float32).to(torch.bfloat16)
    q_dev = torch.randn((B, Hq, D), generator=g, device=cuda, dtype=torch.float32).to(torch.bfloat16)
    table = torch.randperm(B * L, generator=torch.Generator().manual_seed(8)).view(B, L).int()
    table_dev = table.to(cuda)
    lens_dev = torch.full((B, ), L, dtype=torch.int32, device=cuda)
    scale = D**-0.5
    out_split, lse_split, _ = _split_kv(q_dev, k_dev, v_dev, lens_dev, table_dev, scale, 0.0, S)
    merged = torch.empty((B, Hq, D), dtype=torch.float32, device=cuda)
    merged_lse = torch.empty((B, Hq), dtype=torch.float32, device=cuda)
    decode_combine(out_split, lse_split, S, 1, lens_dev, B, Hq, D,
                   (out_split.stride(2), out_split.stride(0), out_split.stride(1)),
                   (lse_split.stride(2), lse_split.stride(0), lse_split.stride(1)), merged, merged_lse)
    fused = torch.full((B, Hq, D), float("nan"), dtype=torch.float32, device=cuda)
    fused_lse = torch.full((B, Hq), float("nan"), dtype=torch.float32, device=cuda)
    decode_fused(q_dev, k_dev, v_dev, lens_dev, table_dev, scale, 0.0, S, fused, fused_lse)
    torch.cuda.synchronize()
    assert torch.equal(fused.view(torch.int32), merged.view(torch.int32))
    assert torch.equal(fused_lse.view(torch.int32), merged_lse.view(torch.int32))
    w_merged, w_lse = golden.lse_merge(out_split.cpu().permute(2, 0, 1, 3), lse_split.cpu().permute(2, 0, 1))
    assert (merged.cpu().double() - w_merged).abs().max() <= 1e-5
    assert (merged_lse.cpu().double() - w_lse).abs().max() <= 1e-4
    for b in (0, 31):
        tokens = table[b].long().to(cuda)
        k_b, v_b = k_dev[tokens].cpu(), v_dev[tokens].cpu()
        t_b = torch.arange(L, dtype=torch.int32).view(1, -1)
        exact, exact_lse = golden.decode_exact(q_dev[b:b + 1].cpu(), k_b, v_b, [L], t_b, scale)
        assert (merged[b].cpu().double() - exact[0]).abs().max() <= ATOL
        assert (merged_lse[b].cpu().double() - exact_lse[0]).abs().max() <= ATOL


def test_config5_end_to_end_with_seven_peers(cuda):
    """BASELINE config 5 end to end at full size through the layer: split-KV over the shard (32 x 32768 keys, page 16),
    merge of its splits, then the LSE merge with 7 seeded peer shards (out ~N(0,1) bf16, LSE ~N(log 32768, 2) fp32)
    into [32, 64, 128]. Checked on 8 sequences against the exact closed form (decode_exact for the own shard, lse_merge
    over the 8 shards): the fp32 form of the final output at 2e-3 absolute with no allowance, and the bf16 output
    as exactly that fp32 result rounded to bf16 (its values are O(1), so bf16 rounding alone is up to 2^-8 |x|)."""
    from triton_dist.kernels.amd import gqa_fwd_batch_decode_inter_rank_combine
    from triton_dist.layers.nvidia import SpGQAFlashDecodeAttention
    announce("decode C5 end to end, 8 shards")
    R, rank, B, Hq, Hkv, D, L, page = 8, 0, 32, 64, 8, 128, 32768, 16
    g = torch.Generator(device="cuda").manual_seed(3 + 4)
    pages_per_seq = L // page
    num_pages = B * pages_per_seq
    k_dev = torch.randn((num_pages, page, Hkv, D), generator=g, device=cuda, dtype=torch.float32).to(torch.bfloat16)
    v_dev = torch.randn((num_pages, page, Hkv, D), generator=g, device=cuda, dtype=torch.float32).to(torch.bfloat16)
    q_dev = torch.randn((B, Hq, D), generator=g, device=cuda, dtype=torch.float32).to(torch.bfloat16)
    table = torch.randperm(num_pages, generator=torch.Generator().manual_seed(6)).view(B, pages_per_seq).int()
    gp = torch.Generator().manual_seed(3 + 4 + 100)
    peer_out = torch.randn((R, B, Hq, D), generator=gp).to(torch.bfloat16)
    peer_lse = torch.randn((R, B, Hq), generator=gp) * 2 + math.log(L)
    global_lens = torch.full((R, B), L, dtype=torch.int32)
    scale = D**-0.5
    layer = SpGQAFlashDecodeAttention(rank, 0, R, 1, Hq, Hkv, D, D, page_size=page, scale=scale, max_allowed_batch=B)
    layer.kv_split = 16                                   # the config's 16 splits
    all_out = peer_out.float().to(cuda)                    # gather buffer in fp32: the own fp32 partial loses nothing
    all_lse = peer_lse.to(cuda)
    out = layer(q_dev, k_dev, v_dev, global_lens.to(cuda), table.to(cuda), peer_partials=(all_out, all_lse))
    # the same merge with an fp32 result (all_out / all_lse now hold the own shard in row `rank`)
    out32 = gqa_fwd_batch_decode_inter_rank_combine(all_out, all_lse, global_lens.to(cuda), out_dtype=torch.float32)
    torch.cuda.synchronize()
    assert out.dtype == torch.bfloat16 and out.shape == (B, Hq, D)
    assert torch.equal(out, out32.to(torch.bfloat16)), "the bf16 output is the fp32 result rounded to nearest even"
    seqs = [0, 3, 7, 12, 16, 21, 26, 31]
    for b in seqs:
        pages = table[b].long().to(cuda)
        k_b, v_b = k_dev[pages].cpu(), v_dev[pages].cpu()
        t_b = torch.arange(pages_per_seq, dtype=torch.int32).view(1, -1)
        own, own_lse = golden.decode_exact(q_dev[b:b + 1].cpu(), k_b, v_b, [L], t_b, scale)
        shard_out = peer_out[:, b:b + 1].double().clone()
        shard_lse = peer_lse[:, b:b + 1].double().clone()
        shard_out[rank], shard_lse[rank] = own, own_lse
        want, _ = golden.lse_merge(shard_out, shard_lse)
        err = float((out32[b].cpu().double() - want[0]).abs().max())
        assert err <= ATOL, "sequence %d: %g" % (b, err)


@pytest.mark.parametrize("D", [80, 96, 160, 8, 40, 248])
@pytest.mark.parametrize("num_heads,kv_lens,S,block_size", [((16, 16), [1320, 18, 463], 4, 16), ((32, 8), [1, 54, 293, 70], 8, 1),
                                                            ((6, 1), [777, 0, 5], 3, 16)])
@pytest.mark.parametrize("dtype,soft_cap", [(torch.bfloat16, 0), (torch.float16, 30)])
def test_head_dimensions_that_are_no_power_of_two(cuda, D, num_heads, kv_lens, S, block_size, dtype, soft_cap):
    """Head dimensions like 80, 96 and 160 (the reference takes them as BLOCK_DMODEL + BLOCK_DPE with masks,
    flash_decode.py:771-772): per-split partials and LSE, the merged 16-bit output, and the one-launch form bit for
    bit against split + combine. The cache rows are D wide and packed, so a lane that read beyond its row would
    read the next head's or token's values."""
    from triton_dist.kernels.amd.flash_decode import _split_kv, decode_combine, decode_fused
    announce("decode D=%d heads=%s kv_lens=%s S=%d page=%d %s cap=%s" % (D, num_heads, kv_lens, S, block_size, dtype, soft_cap))
    q, k_cache, v_cache, table = build_case(kv_lens, num_heads, D, block_size, dtype, seed=D + S)
    scale = D**-0.5
    B, Hq = len(kv_lens), num_heads[0]
    lens_dev = torch.tensor(kv_lens, dtype=torch.int32, device=cuda)
    qd, kd, vd, td = q.to(cuda), k_cache.to(cuda), v_cache.to(cuda), table.to(cuda)
    out_split, lse_split, _ = _split_kv(qd, kd, vd, lens_dev, td, scale, soft_cap, S)
    torch.cuda.synchronize()
    assert out_split.shape == (B, Hq, S, D)
    w_out, w_lse = golden.decode_split_exact(q, k_cache, v_cache, kv_lens, table, scale, S, soft_cap)
    got_lse = lse_split.cpu().double()
    empty = torch.isinf(w_lse)
    assert torch.equal(torch.isinf(got_lse), empty)
    assert (got_lse[~empty] - w_lse[~empty]).abs().max() <= ATOL
    assert (out_split.cpu().double() - w_out).abs().max() <= ATOL
    want = torch.empty((B, Hq, D), dtype=dtype, device=cuda)
    want_lse = torch.empty((B, Hq), dtype=torch.float32, device=cuda)
    decode_combine(out_split, lse_split, S, 1, lens_dev, B, Hq, D,
                   (out_split.stride(2), out_split.stride(0), out_split.stride(1)),
                   (lse_split.stride(2), lse_split.stride(0), lse_split.stride(1)), want, want_lse)
    got = torch.full((B, Hq, D), float("nan"), dtype=dtype, device=cuda)
    got_lse = torch.full((B, Hq), float("nan"), dtype=torch.float32, device=cuda)
    counters = torch.zeros(1024, dtype=torch.int32, device=cuda)
    decode_fused(qd, kd, vd, lens_dev, td, scale, soft_cap, S, got, got_lse, workspace=counters)
    torch.cuda.synchronize()
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    assert torch.equal(got_lse.view(torch.int32), want_lse.view(torch.int32))
    assert int(counters.abs().sum()) == 0
    exact, _ = golden.decode_exact(q, k_cache, v_cache, kv_lens, table, scale, soft_cap)
    assert_final_output(got, merged_fp32(out_split, lse_split, S, lens_dev), exact)


@pytest.mark.parametrize("D,num_heads,force", [(128, (64, 8), 2), (128, (16, 16), 2), (128, (32, 8), 2), (64, (64, 8), 4),
                                               (64, (24, 8), 2), (64, (16, 16), 4), (64, (64, 4), 2), (256, (32, 8), 2),
                                               (256, (12, 4), 2), (96, (64, 8), 2), (80, (16, 16), 2), (112, (24, 8), 2)])
@pytest.mark.parametrize("kv_lens,S,block_size", [([1320, 18, 463], 4, 16), ([1, 54, 293, 70], 8, 1), ([777, 0, 5, 2047], 3, 16),
                                                  ([100, 31], 1, 16)])
@pytest.mark.parametrize("dtype,soft_cap", [(torch.bfloat16, 0), (torch.float16, 30)])
@pytest.mark.parametrize("splits_per_team", [1, 3, 4])
def test_a_kv_head_per_wave(cuda, switches, D, num_heads, force, kv_lens, S, block_size, dtype, soft_cap, splits_per_team):
    """The form in which every wave of a workgroup takes a kv head of its own (chosen by itself only for grids that
    fill the chip; forced here on small cases): per-split partials and LSE against the oracle, the one-launch form bit
    for bit against split + combine with the counters back at zero, and both within the oracle's bar of the other
    form's results. A workgroup of this form streams through several consecutive splits of its sequence (as many as
    fill the chip best; forced here too, 4 being the most any instance takes): splits_per_team = 3 leaves a last workgroup with fewer, and empty splits
    inside a workgroup's range."""
    from triton_dist.kernels.amd.flash_decode import _split_kv, decode_combine, decode_fused
    from triton_dist import _lib
    switches(_lib.TDIST_DEBUG_DECODE_SPLITS_PER_TEAM, splits_per_team)
    announce("decode, a kv head per wave (%d), %d splits per workgroup: D=%d heads=%s kv_lens=%s S=%d page=%d %s cap=%s" % (force, splits_per_team, D, num_heads, kv_lens, S, block_size, dtype, soft_cap))
    q, k_cache, v_cache, table = build_case(kv_lens, num_heads, D, block_size, dtype, seed=D + S + num_heads[0])
    scale = D**-0.5
    B, Hq = len(kv_lens), num_heads[0]
    lens_dev = torch.tensor(kv_lens, dtype=torch.int32, device=cuda)
    qd, kd, vd, td = q.to(cuda), k_cache.to(cuda), v_cache.to(cuda), table.to(cuda)
    switches(_lib.TDIST_DEBUG_DECODE_WAVE_HEADS, 0)
    other_out, other_lse, _ = _split_kv(qd, kd, vd, lens_dev, td, scale, soft_cap, S)
    switches(_lib.TDIST_DEBUG_DECODE_WAVE_HEADS, force)   # 2: eight waves where the heads allow, 4: four
    out_split, lse_split, _ = _split_kv(qd, kd, vd, lens_dev, td, scale, soft_cap, S)
    torch.cuda.synchronize()
    w_out, w_lse = golden.decode_split_exact(q, k_cache, v_cache, kv_lens, table, scale, S, soft_cap)
    got_lse = lse_split.cpu().double()
    empty = torch.isinf(w_lse)
    assert torch.equal(torch.isinf(got_lse), empty)
    assert (got_lse[~empty] - w_lse[~empty]).abs().max() <= ATOL
    assert (out_split.cpu().double() - w_out).abs().max() <= ATOL
    assert (out_split.cpu()[empty] == 0).all()
    assert (out_split - other_out).abs().max() <= ATOL
    want = torch.empty((B, Hq, D), dtype=dtype, device=cuda)
    want_lse = torch.empty((B, Hq), dtype=torch.float32, device=cuda)
    decode_combine(out_split, lse_split, S, 1, lens_dev, B, Hq, D,
                   (out_split.stride(2), out_split.stride(0), out_split.stride(1)),
                   (lse_split.stride(2), lse_split.stride(0), lse_split.stride(1)), want, want_lse)
    counters = torch.zeros(1024, dtype=torch.int32, device=cuda)
    for _ in range(2):   # twice on the same counters
        got = torch.full((B, Hq, D), float("nan"), dtype=dtype, device=cuda)
        got_lse = torch.full((B, Hq), float("nan"), dtype=torch.float32, device=cuda)
        decode_fused(qd, kd, vd, lens_dev, td, scale, soft_cap, S, got, got_lse, workspace=counters)
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int16), want.view(torch.int16))
        assert torch.equal(got_lse.view(torch.int32), want_lse.view(torch.int32))
        assert int(counters.abs().sum()) == 0
    exact, _ = golden.decode_exact(q, k_cache, v_cache, kv_lens, table, scale, soft_cap)
    assert_final_output(got, merged_fp32(out_split, lse_split, S, lens_dev), exact)


@pytest.mark.parametrize("kind", ["even", "one long", "random"])
def test_form_follows_the_sequence_lengths(cuda, switches, kind):
    """A grid that fills the chip gets two launches: the form with a kv head per wave, which runs if the sequence
    lengths are even (mean >= 0.8 max, decided on the device by every wave from the same loads), and the form with a
    kv head per workgroup behind it, which runs if they are not. Exactly one of them must have written every partial
    result (the buffers start as NaN), for even and uneven batches alike, split and one-launch forms."""
    from triton_dist.kernels.amd.flash_decode import _split_kv, decode_combine, decode_fused
    from triton_dist import _lib
    switches(_lib.TDIST_DEBUG_DECODE_WAVE_HEADS, None)
    switches(_lib.TDIST_DEBUG_DECODE_SPLITS_PER_TEAM, None)
    B, heads, D, page, S = 32, (8, 8), 64, 16, 8      # 32 x 8 (sequence, split) pairs on one head group: 256 workgroups
    g = torch.Generator().manual_seed(5)
    if kind == "even":
        kv_lens = [2048] * B
    elif kind == "one long":
        kv_lens = [2048] + [64] * (B - 1)
    else:
        kv_lens = torch.randint(1, 2049, (B,), generator=g).tolist()
    announce("decode form by lengths: %s (sum %d, max %d)" % (kind, sum(kv_lens), max(kv_lens)))
    q, k_cache, v_cache, table = build_case(kv_lens, heads, D, page, torch.bfloat16, seed=9)
    # a block table twice as wide as the sequences need (as a server's is): what it lets a call read, 268 MB here, is
    # what the host goes by when it decides whether the form is worth its second launch
    table = torch.cat([table, torch.zeros_like(table)], dim=1).contiguous()
    scale = D**-0.5
    lens_dev = torch.tensor(kv_lens, dtype=torch.int32, device=cuda)
    qd, kd, vd, td = q.to(cuda), k_cache.to(cuda), v_cache.to(cuda), table.to(cuda)
    out_split = torch.full((B, heads[0], S, D), float("nan"), dtype=torch.float32, device=cuda)
    lse_split = torch.full((B, heads[0], S), float("nan"), dtype=torch.float32, device=cuda)
    _split_kv(qd, kd, vd, lens_dev, td, scale, 0.0, S, out_split, lse_split)
    torch.cuda.synchronize()
    w_out, w_lse = golden.decode_split_exact(q, k_cache, v_cache, kv_lens, table, scale, S)
    got_lse = lse_split.cpu().double()
    empty = torch.isinf(w_lse)
    assert not torch.isnan(out_split).any() and not torch.isnan(lse_split).any()
    assert torch.equal(torch.isinf(got_lse), empty)
    assert (got_lse[~empty] - w_lse[~empty]).abs().max() <= ATOL
    assert (out_split.cpu().double() - w_out).abs().max() <= ATOL
    want = torch.empty((B, heads[0], D), dtype=torch.bfloat16, device=cuda)
    want_lse = torch.empty((B, heads[0]), dtype=torch.float32, device=cuda)
    decode_combine(out_split, lse_split, S, 1, lens_dev, B, heads[0], D,
                   (out_split.stride(2), out_split.stride(0), out_split.stride(1)),
                   (lse_split.stride(2), lse_split.stride(0), lse_split.stride(1)), want, want_lse)
    counters = torch.zeros(1024, dtype=torch.int32, device=cuda)
    got = torch.full((B, heads[0], D), float("nan"), dtype=torch.bfloat16, device=cuda)
    got_lse = torch.full((B, heads[0]), float("nan"), dtype=torch.float32, device=cuda)
    decode_fused(qd, kd, vd, lens_dev, td, scale, 0.0, S, got, got_lse, workspace=counters)
    torch.cuda.synchronize()
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    assert torch.equal(got_lse.view(torch.int32), want_lse.view(torch.int32))
    assert int(counters.abs().sum()) == 0
