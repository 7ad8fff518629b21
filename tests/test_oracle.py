"""Pins the oracle: the torch restatement (oracle/golden.py) against the scalar C restatement (oracle/c),
against known answers worked by hand, and against what the mathematics fixes. CPU only."""
import math

import numpy as np
import pytest
import torch

from oracle import cref, golden


def bf16_bits(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


# ---- number formats ---------------------------------------------------------------------------------
def test_e4m3_table_matches_torch_float8():
    ours = cref.e4m3_table()
    theirs = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).float().numpy()
    assert np.array_equal(np.isnan(ours), np.isnan(theirs))
    assert np.array_equal(ours[~np.isnan(ours)], theirs[~np.isnan(theirs)])
    # known answers: 0x38 = 1.0, 0x7e = 448 (max), 0x01 = 2^-9 (min subnormal), 0x08 = 2^-6 (min normal), 0xc0 = -2
    assert ours[0x38] == 1.0 and ours[0x7E] == 448.0 and ours[0x01] == 2.0**-9 and ours[0x08] == 2.0**-6
    assert ours[0xC0] == -2.0 and math.isnan(ours[0x7F]) and math.isnan(ours[0xFF])


# ---- (b) reduction ------------------------------------------------------------------------------------
@pytest.mark.parametrize("R,first", [(8, 1), (8, 0), (4, 3), (2, 1), (1, 0), (5, 2)])
def test_reduce_slices_torch_vs_c_bit_exact(R, first):
    g = torch.Generator().manual_seed(11 + R)
    c = torch.randn((R, 4099), generator=g).to(torch.bfloat16)
    want = golden.reduce_slices_ordered(c, first)
    got = cref.reduce_slices_bf16(bf16_bits(c), first)
    assert np.array_equal(bf16_bits(want), got)


def test_reduce_two_slices_is_order_free_and_exactly_rounded():
    g = torch.Generator().manual_seed(5)
    c = torch.randn((2, 1000), generator=g).to(torch.bfloat16)
    a = golden.reduce_slices_ordered(c, 0)
    b = golden.reduce_slices_ordered(c, 1)
    assert torch.equal(a, b)
    assert torch.equal(a, (c[0].double() + c[1].double()).to(torch.bfloat16))  # a sum of two bf16 is exact in fp32


def test_reduce_order_matters_in_general():
    # 1 + 2^-24*... : (big + small) + (-big) != (big + -big) + small in fp32
    c = torch.tensor([[2.0**20], [2.0**-8], [-(2.0**20)]]).to(torch.bfloat16)
    assert float(golden.reduce_slices_ordered(c, 0)) == 0.0          # big + small = big, - big = 0
    assert float(golden.reduce_slices_ordered(c, 2)) == 2.0**-8      # -big + big = 0, + small


# ---- (a) GEMM -----------------------------------------------------------------------------------------
def test_gemm_torch_vs_c_exact_on_integer_inputs():
    g = torch.Generator().manual_seed(1)
    a = torch.randint(-4, 5, (48, 64), generator=g).to(torch.bfloat16)
    b = torch.randint(-4, 5, (40, 64), generator=g).to(torch.bfloat16)
    shards = [a[:16], a[16:32], a[32:]]
    want = cref.gemm_nt_f64(a.float().numpy(), b.float().numpy())
    assert np.array_equal(golden.ag_gemm_fp32(shards, b).numpy().astype(np.float64), want)
    # every entry is an integer below 2^8*... representable in bf16 only if |x| <= 256: compare in fp32 instead
    assert np.array_equal(golden.torch_ag_gemm([s.float() for s in shards], b.float()).numpy().astype(np.float64), want)


def test_gemm_bf16_golden_within_rounding_of_fp32():
    g = torch.Generator().manual_seed(2)
    a = torch.randn((64, 256), generator=g).to(torch.bfloat16)
    b = (torch.randn((32, 256), generator=g) * 0.02).to(torch.bfloat16)
    ref = golden.ag_gemm_fp32([a], b)
    out = golden.torch_ag_gemm([a], b)
    assert golden.max_rel_err(out.float(), ref) < 1e-2
    assert np.allclose(ref.numpy(), cref.gemm_nt_f64(a.float().numpy(), b.float().numpy()), rtol=1e-4, atol=1e-5)


def test_fp8_scaled_gemm_closed_form_vs_c():
    g = torch.Generator().manual_seed(3)
    a8 = torch.randn((24, 128), generator=g).to(torch.float8_e4m3fn)
    b8 = torch.randn((20, 128), generator=g).to(torch.float8_e4m3fn)
    sa = torch.rand(24, generator=g) * 0.09 + 0.01
    sb = torch.rand(20, generator=g) * 0.009 + 0.001
    want = cref.gemm_e4m3_nt_f64(a8.view(torch.uint8).numpy(), b8.view(torch.uint8).numpy(), sa.numpy(), sb.numpy())
    got = golden.fp8_scaled_gemm_fp32(a8, sa, b8, sb).numpy()
    assert np.allclose(got, want, rtol=1e-5, atol=1e-7)
    # scales factor out: C(sa, sb) == diag(sa) C(1, 1) diag(sb)
    plain = golden.fp8_scaled_gemm_fp32(a8, None, b8, None)
    assert torch.allclose(plain * sa[:, None] * sb[None, :], torch.from_numpy(got), rtol=1e-6, atol=0)


def test_gemm_rs_golden_vs_fp32_closed_form():
    g = torch.Generator().manual_seed(4)
    W, rank = 4, 1
    a = torch.randn((64, 128), generator=g).to(torch.bfloat16)
    w = (torch.randn((32, 128), generator=g) * 0.02).to(torch.bfloat16)
    peers = [None if r == rank else torch.randn((16, 32), generator=g).to(torch.bfloat16) for r in range(W)]
    out = golden.torch_gemm_rs(a, w, peers, rank, W)
    ref = golden.gemm_rs_fp32(a, w, peers, rank, W)
    assert out.shape == (16, 32) and golden.max_rel_err(out.float(), ref) < 1e-2


# ---- (c) MoE ------------------------------------------------------------------------------------------
def test_moe_preprocess_known_answer():
    # 3 tokens, topk 2, 3 experts; flat ids = [1,0, 0,1, 1,1]
    ids = torch.tensor([[1, 0], [0, 1], [1, 1]], dtype=torch.int32)
    splits, cumsum, scatter, gather, topk_idx = golden.moe_preprocess(ids, 3)
    assert splits.tolist() == [2, 4, 0]
    assert cumsum.tolist() == [0, 2, 6, 6]
    # expert 0 holds flat entries 1,2 -> positions 0,1; expert 1 holds 0,3,4,5 -> positions 2,3,4,5
    assert scatter.flatten().tolist() == [2, 0, 1, 3, 4, 5]
    assert gather.tolist() == [0, 1, 0, 1, 2, 2]
    assert topk_idx.tolist() == [1, 0, 0, 1, 0, 1]


@pytest.mark.parametrize("T,topk,G,seed", [(64, 8, 16, 0), (257, 4, 7, 1), (1, 1, 1, 2), (1000, 8, 256, 3), (33, 2, 64, 4)])
def test_moe_preprocess_torch_vs_c_and_invariants(T, topk, G, seed):
    g = torch.Generator().manual_seed(seed)
    if topk <= G:
        ids = golden.random_distinct_experts(T, G, topk, g)
    else:
        ids = torch.randint(0, G, (T, topk), generator=g).to(torch.int32)
    splits, cumsum, scatter, gather, topk_idx = golden.moe_preprocess(ids, G)
    c_splits, c_cumsum, c_scatter, c_gather, c_topk = cref.moe_preprocess(ids.numpy(), topk, G)
    assert np.array_equal(splits.numpy(), c_splits) and np.array_equal(cumsum.numpy(), c_cumsum)
    assert np.array_equal(scatter.numpy(), c_scatter) and np.array_equal(gather.numpy(), c_gather)
    assert np.array_equal(topk_idx.numpy(), c_topk)
    n = T * topk
    assert int(cumsum[-1]) == n
    assert sorted(scatter.flatten().tolist()) == list(range(n))                      # a permutation
    assert torch.equal(gather[scatter.flatten().long()], torch.arange(n).div(topk, rounding_mode="floor").int())
    flat = ids.flatten()
    sorted_ids = flat[torch.argsort(scatter.flatten())]
    assert torch.equal(sorted_ids, flat.sort(stable=True).values)                    # grouped by expert
    for e in range(G):                                                                # stable within an expert
        pos = scatter.flatten()[flat == e]
        assert torch.equal(pos, pos.sort().values)


def test_dispatch_and_post_process_torch_vs_c_and_round_trip():
    g = torch.Generator().manual_seed(7)
    T, topk, G, W, H, max_m = 96, 4, 16, 4, 48, 160
    Er = G // W
    ids = golden.random_distinct_experts(T, G, topk, g)
    x = torch.randn((T, H), generator=g)
    q, s = golden.quantize_per_token_e4m3(x)
    splits, cumsum, scatter, gather, _ = golden.moe_preprocess(ids, G)
    sorted_rows = q.view(torch.uint8)[gather.long()]
    sorted_scales = s[gather.long()]
    sp, recv, sc = golden.dispatch_slots(sorted_rows, sorted_scales, cumsum, W, Er, max_m, fill_byte=0xAB)
    c_sp, c_recv, c_sc = cref.dispatch_slots(q.view(torch.uint8).numpy(), s.numpy(), gather.numpy(), cumsum.numpy(), W, Er,
                                             max_m, fill_byte=0xAB)
    assert np.array_equal(sp.numpy(), c_sp) and np.array_equal(recv.numpy(), c_recv) and np.array_equal(sc.numpy(), c_sc)
    assert torch.equal(sp, splits)
    out, out_s = golden.all_to_all_post_process(sp, recv, sc, W, max_m)
    c_out, c_out_s = cref.post_process(recv.numpy(), sc.numpy(), sp.numpy(), W, Er, max_m)
    assert np.array_equal(out.numpy(), c_out) and np.array_equal(out_s.numpy(), c_out_s)
    # post_process(dispatch(x)) is the expert-sorted input again (test_all_to_all.py:461-475 with one sender)
    assert torch.equal(out, sorted_rows) and torch.equal(out_s, sorted_scales)


def test_weighted_combine_vs_c_and_reference_round_trip():
    g = torch.Generator().manual_seed(8)
    T, topk, G, H = 50, 4, 8, 32
    ids = golden.random_distinct_experts(T, G, topk, g)
    x = torch.randn((T, H), generator=g)
    q, s = golden.quantize_per_token_e4m3(x)
    w = torch.softmax(torch.randn((T, topk), generator=g), dim=-1)
    _, _, scatter, gather, _ = golden.moe_preprocess(ids, G)
    rows = q[gather.long()]
    scales = s[gather.long()]
    got = golden.weighted_combine(rows.float(), scales, scatter, w)
    want = cref.combine_e4m3(rows.view(torch.uint8).numpy(), scales.numpy(), scatter.numpy(), w.numpy())
    assert np.allclose(got.numpy(), want, rtol=1e-6, atol=1e-6)
    # weights sum to 1 and every copy of a token is the same row: y == dequantised x
    deq = q.float() * s[:, None]
    assert torch.allclose(got, deq, rtol=1e-5, atol=1e-5)
    # w == 1, scale == 1: the reference's check combine == topk * input (test_all_to_all.py:366-370)
    ones = golden.weighted_combine(rows.float(), None, scatter, None)
    assert torch.equal(ones, golden.combine_index_add(rows.float(), gather, T))
    assert torch.allclose(ones, q.float() * topk, rtol=1e-6, atol=0)


# ---- (d) decode ---------------------------------------------------------------------------------------
@pytest.mark.parametrize("heads,page,soft_cap,dims", [((8, 2), 1, 0.0, (64, 64)), ((4, 4), 16, 0.0, (64, 64)),
                                                      ((6, 1), 4, 30.0, (64, 64)), ((4, 2), 4, 0.0, (96, 64)),
                                                      ((2, 1), 16, 20.0, (192, 128))])
def test_decode_exact_vs_c_and_reference_golden(heads, page, soft_cap, dims):
    g = torch.Generator().manual_seed(9)
    Hq, Hkv = heads
    (D, Dv), kv_lens = dims, [37, 1, 130]
    B = len(kv_lens)
    q = torch.randn((B, Hq, D), generator=g).to(torch.bfloat16)
    k_cache, v_cache, table = golden.make_paged_kv(B, max(kv_lens), Hkv, D, page, torch.bfloat16, g, v_head_dim=Dv)
    scale = D**-0.5
    out, lse = golden.decode_exact(q, k_cache, v_cache, kv_lens, table, scale, soft_cap)
    c_out, c_lse = cref.decode_range(q.float().numpy(), k_cache.float().numpy(), v_cache.float().numpy(), table.numpy(),
                                     [0] * B, kv_lens, scale, soft_cap)
    assert np.allclose(out.numpy(), c_out, rtol=1e-10, atol=1e-12) and np.allclose(lse.numpy(), c_lse, rtol=1e-12)
    ref = golden.ref_paged_attn(q, k_cache, v_cache, [1] * B, kv_lens, table, scale, soft_cap)
    assert torch.allclose(ref.float(), out.float(), atol=1e-2, rtol=1e-2)   # the reference test's own tolerance
    # kv_len == 1: softmax is 1, the output is that key's value row and LSE its score
    n0 = int(table[1, 0]) * page
    v_row = v_cache.view(-1, Hkv, Dv)[n0]
    assert torch.allclose(out[1].float(), torch.repeat_interleave(v_row, Hq // Hkv, dim=0).float(), atol=1e-6)
    # the extra key dimensions take part in the scores: dropping them changes the LSE
    if D != Dv:
        _, lse_cut = golden.decode_exact(q[..., :Dv], k_cache[..., :Dv].contiguous(), v_cache, kv_lens, table, scale, soft_cap)
        assert not torch.allclose(lse_cut, lse, atol=1e-3)


def test_split_partials_merge_to_the_full_result():
    g = torch.Generator().manual_seed(10)
    B, Hq, Hkv, D, S = 3, 8, 2, 64, 6
    kv_lens = [100, 3, 0]      # 3 keys over 6 splits leaves empty splits; 0 keys: everything empty
    q = torch.randn((B, Hq, D), generator=g).to(torch.bfloat16)
    k_cache, v_cache, table = golden.make_paged_kv(B, 100, Hkv, D, 4, torch.bfloat16, g)
    scale = D**-0.5
    full, full_lse = golden.decode_exact(q, k_cache, v_cache, kv_lens, table, scale)
    part, part_lse = golden.decode_split_exact(q, k_cache, v_cache, kv_lens, table, scale, S)
    assert golden.split_ranges(3, 6) == [(0, 1), (1, 2), (2, 3), (3, 3), (4, 3), (5, 3)]
    merged, merged_lse = golden.lse_merge(part.permute(2, 0, 1, 3), part_lse.permute(2, 0, 1))
    assert torch.allclose(merged, full, atol=1e-12) and torch.allclose(merged_lse[:2], full_lse[:2], atol=1e-12)
    assert torch.isinf(merged_lse[2]).all() and (merged[2] == 0).all()
    # skipping a partial == merging without it
    skip = torch.zeros((S, B, Hq), dtype=torch.bool)
    skip[0] = True
    m2, _ = golden.lse_merge(part.permute(2, 0, 1, 3), part_lse.permute(2, 0, 1), skip)
    m3, _ = golden.lse_merge(part.permute(2, 0, 1, 3)[1:], part_lse.permute(2, 0, 1)[1:])
    assert torch.allclose(m2, m3, atol=1e-12)


# ---- MoE align / sort ------------------------------------------------------------------------------------
def test_align_sort_reference_examples():
    """The two worked examples the reference itself documents."""
    # kernels/nvidia/allgather_group_gemm.py:82-93 (expert ids 1..4 there; 0-based here)
    ids = torch.tensor([[2, 3, 4], [1, 2, 4], [1, 3, 4], [1, 2, 3]]) - 1
    s, e, b, r, n = golden.sort_topk_ids_align_block_size(ids, 4, 1, 4, 4)
    assert n == 16 and s[:n].tolist() == [3, 6, 9, 12, 0, 4, 10, 12, 1, 7, 11, 12, 2, 5, 8, 12]
    assert e.tolist() == [0, 1, 2, 3] and b.tolist() == [0, 0, 0, 0] and r.tolist() == [4]
    # csrc/lib/moe_utils.cu:136-142: [0,1,2,1,2,3,0,3,4], block 4 -> [0,6,*,*,1,3,*,*,2,4,*,*,5,7,*,*,8,*,*,*]
    ids = torch.tensor([0, 1, 2, 1, 2, 3, 0, 3, 4]).view(-1, 1)
    s, e, b, r, n = golden.sort_topk_ids_align_block_size(ids, 5, 1, 9, 4)
    P = 9
    assert s[:n].tolist() == [0, 6, P, P, 1, 3, P, P, 2, 4, P, P, 5, 7, P, P, 8, P, P, P]
    assert e.tolist() == [0, 1, 2, 3, 4]


def test_align_sort_invariants():
    g = torch.Generator().manual_seed(5)
    R, T, topk, E, BS = 3, 37, 4, 11, 8
    ids = torch.stack([torch.randperm(E, generator=g)[:topk] for _ in range(R * T)])
    s, e, b, r, n = golden.sort_topk_ids_align_block_size(ids, E, R, T, BS)
    flat = ids.reshape(-1)
    valid = s[:n][s[:n] < flat.numel()].long()
    assert sorted(valid.tolist()) == list(range(flat.numel()))           # every entry placed exactly once
    assert n % BS == 0 and int(r.sum()) * BS == n and e.numel() == n // BS
    per = T * topk
    for blk in range(n // BS):                                            # a block holds one expert of one segment
        ent = s[blk * BS:(blk + 1) * BS]
        ent = ent[ent < flat.numel()].long()
        assert torch.all(flat[ent] == e[blk]) and torch.all(ent // per == b[blk])
        assert torch.all(ent[1:] > ent[:-1])                              # flat order kept inside a group
    assert torch.all(s[n:] == flat.numel())


# ---- group quantisation ----------------------------------------------------------------------------------
def test_group_quantisation_closed_form_and_round_trip():
    g = torch.Generator().manual_seed(8)
    x = (torch.randn((6, 384), generator=g) * torch.tensor([1e-3, 0.1, 1.0, 7.0, 300.0, 5e4])[:, None]).to(torch.bfloat16)
    q, s = golden.quantize_groups_e4m3(x)
    xf = x.float().view(6, 3, 128)
    amax = xf.abs().amax(-1)
    # the scale maps the group's largest magnitude onto 448, the largest finite e4m3
    assert torch.allclose(s, amax / 448, rtol=2e-7, atol=0)
    qf = q.float().view(6, 3, 128)
    assert qf.abs().amax(-1).eq(448).all()
    # round trip: every element within half an e4m3 step (relative 2^-4 of its own size, or half the smallest
    # subnormal step 2^-10, in units of the scale)
    d = golden.dequantize_groups(q, s).float().view(6, 3, 128)
    step = torch.maximum(xf.abs() * 2.0**-4, s[..., None] * 2.0**-10) + xf.abs() * 2.0**-8
    assert ((d - xf).abs() <= step).all()
    # exact cases: powers of two times the scale are representable
    x2 = torch.zeros((1, 128)); x2[0, 0] = 448.0; x2[0, 1] = 1.0; x2[0, 2] = -0.5; x2[0, 3] = 2.0**-9
    q2, s2 = golden.quantize_groups_e4m3(x2.to(torch.bfloat16))
    assert s2.item() == 1.0 and q2.float()[0, :4].tolist() == [448.0, 1.0, -0.5, 2.0**-9]


def test_group_gemm_golden_is_the_per_row_product():
    """torch_moe_scatter_group_gemm (the reference's golden) against its definition, row by row, and against the
    dense product when every token goes to one expert."""
    g = torch.Generator().manual_seed(21)
    M, K, N, E, topk = 12, 16, 8, 5, 3
    x = torch.randint(-3, 4, (M, K), generator=g).float()
    w = torch.randint(-3, 4, (E, K, N), generator=g).float()
    ids = golden.random_distinct_experts(M, E, topk, g)
    out = golden.torch_moe_scatter_group_gemm(x, w, ids)
    assert out.shape == (M * topk, N)
    for t in range(M):
        for k in range(topk):
            assert torch.equal(out[t * topk + k], x[t] @ w[int(ids[t, k])])
    one = golden.torch_moe_scatter_group_gemm(x, w, torch.full((M, 1), 2))
    assert torch.equal(one, x @ w[2])
    halves = golden.ag_group_gemm_fp32([x[:6].bfloat16(), x[6:].bfloat16()], w, ids)
    assert torch.equal(halves, out)


def test_group_gemm_reduce_rs_golden_by_brute_force():
    g = torch.Generator().manual_seed(33)
    M, K, H, E, topk, W, rank = 8, 6, 5, 4, 2, 2, 1
    states = torch.randint(-3, 4, (M * topk, K), generator=g).float()
    w = torch.randint(-3, 4, (E, K, H), generator=g).float()
    ids = golden.random_distinct_experts(M, E, topk, g)
    wt = torch.randint(1, 4, (M, topk), generator=g).float()
    peers = [torch.randint(-5, 6, (M // W, H), generator=g).float() for _ in range(W)]
    got = golden.torch_group_gemm_reduce_rs(states, w, ids, wt, peers, rank, W)
    for i, t in enumerate(range(rank * M // W, (rank + 1) * M // W)):
        want = sum(wt[t, k] * (states[t * topk + k] @ w[int(ids[t, k])]) for k in range(topk)) + peers[0][i]
        assert torch.equal(got[i], want)
