"""The committed fixtures (tests/golden/*.npz, written by tests/golden/make_fixtures.py) against the oracle on
the CPU and against the HIP path on the GPU."""
import os

import numpy as np
import pytest
import torch

from oracle import cref, golden
from tests.conftest import announce

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(name):
    return np.load(os.path.join(HERE, name), allow_pickle=False)


def bf16(bits):
    return torch.from_numpy(bits.view(np.int16).copy()).view(torch.bfloat16)


# ---- CPU: the oracle reproduces what was frozen ------------------------------------------------------
def test_e4m3_table_fixture():
    want = load("e4m3_table.npz")["table"]
    got = cref.e4m3_table()
    assert np.array_equal(np.isnan(want), np.isnan(got)) and np.array_equal(want[~np.isnan(want)], got[~np.isnan(got)])


def test_moe_fixture_against_both_oracles():
    f = load("moe_64x8x16.npz")
    T, topk, G, W, H, max_m = f["meta"].tolist()
    ids = torch.from_numpy(f["ids"])
    splits, cumsum, scatter, gather, topk_idx = golden.moe_preprocess(ids, G)
    assert np.array_equal(splits.numpy(), f["splits"]) and np.array_equal(cumsum.numpy(), f["cumsum"])
    assert np.array_equal(scatter.numpy(), f["scatter_idx"]) and np.array_equal(gather.numpy(), f["gather_idx"])
    c = cref.moe_preprocess(f["ids"], topk, G)
    assert np.array_equal(c[2], f["scatter_idx"]) and np.array_equal(c[3], f["gather_idx"])
    _, recv, recv_scale = cref.dispatch_slots(f["rows_u8"], f["scales"], f["gather_idx"], f["cumsum"], W, G // W, max_m)
    assert np.array_equal(recv, f["recv_u8"]) and np.array_equal(recv_scale, f["recv_scale"])


def test_reduce_and_gemm_fixtures():
    f = load("reduce_8x4096.npz")
    assert np.array_equal(cref.reduce_slices_bf16(f["slices"], 1), f["out"])
    g = load("gemm_small.npz")
    c = cref.gemm_nt_f64(bf16(g["a_bf16"]).float().numpy(), bf16(g["b_bf16"]).float().numpy())
    assert np.allclose(c, g["c_f32"], rtol=1e-5, atol=1e-6)
    c8 = cref.gemm_e4m3_nt_f64(g["a_e4m3"], g["b_e4m3"], g["row_scale"], g["col_scale"])
    assert np.allclose(c8, g["c8_f32"], rtol=1e-5, atol=1e-8)


def test_decode_fixture():
    f = load("decode_2seq.npz")
    Hq, Hkv, D, page, S = f["meta"].tolist()
    q, k, v = bf16(f["q"]), bf16(f["k_cache"]), bf16(f["v_cache"])
    out, lse = cref.decode_range(q.float().numpy(), k.float().numpy(), v.float().numpy(), f["block_table"], [0, 0],
                                 f["kv_lens"], D**-0.5)
    assert np.allclose(out, f["out"], atol=1e-10) and np.allclose(lse, f["lse"], atol=1e-10)


def f16(bits):
    return torch.from_numpy(bits.view(np.int16).copy()).view(torch.float16)


def test_decode_fixture_with_extra_key_dimensions():
    f = load("decode_dk192_dv128.npz")
    Hq, Hkv, Dk, Dv, page, S, cap = f["meta"].tolist()
    q, k, v = f16(f["q"]), f16(f["k_cache"]), f16(f["v_cache"])
    assert q.shape[-1] == Dk and k.shape[-1] == Dk and v.shape[-1] == Dv
    out, lse = cref.decode_range(q.float().numpy(), k.float().numpy(), v.float().numpy(), f["block_table"], [0, 0],
                                 f["kv_lens"], Dk**-0.5, float(cap))
    assert np.allclose(out, f["out"], atol=1e-10) and np.allclose(lse, f["lse"], atol=1e-10)
    # the frozen per-split partials merge to the frozen full result
    merged, merged_lse = golden.lse_merge(torch.from_numpy(f["part"]).permute(2, 0, 1, 3), torch.from_numpy(f["part_lse"]).permute(2, 0, 1))
    assert np.allclose(merged.numpy(), f["out"], atol=1e-12) and np.allclose(merged_lse.numpy(), f["lse"], atol=1e-12)


def test_align_sort_fixture_invariants():
    """The frozen align / sort output against what the layout fixes, without calling the oracle: every block holds one
    expert's entries of one rank segment in ascending flat order, padding carries the fill value, every entry
    appears exactly once."""
    f = load("moe_align_4x24x3.npz")
    R, Tr, topk, E, block, post_pad = f["meta"].tolist()
    ids = f["ids"].reshape(-1)
    n = ids.size
    sorted_ids, expert_ids, barrier_ids, rank_blocks = f["sorted_token_ids"], f["expert_ids"], f["block_barrier_ids"], f["rank_block_num"]
    assert post_pad % block == 0 and expert_ids.size == post_pad // block == barrier_ids.size == rank_blocks.sum()
    assert np.array_equal(barrier_ids, np.repeat(np.arange(R), rank_blocks))
    seen = []
    for blk in range(post_pad // block):
        entries = sorted_ids[blk * block:(blk + 1) * block]
        real = entries[entries < n]
        assert (entries[len(real):] == n).all(), "padding sits at the end of a block"
        assert (np.diff(real) > 0).all() and (ids[real] == expert_ids[blk]).all()
        assert (real // (Tr * topk) == barrier_ids[blk]).all()
        seen.append(real)
    assert np.array_equal(np.sort(np.concatenate(seen)), np.arange(n))
    assert (sorted_ids[post_pad:] == n).all()
    got = golden.sort_topk_ids_align_block_size(torch.from_numpy(f["ids"]), E, R, Tr, block)
    assert np.array_equal(got[0].numpy(), sorted_ids) and np.array_equal(got[1].numpy(), expert_ids)


def test_group_quant_fixture_closed_form():
    f = load("quant_groups_6x384.npz")
    x = bf16(f["x"]).float().view(6, 3, 128)
    scales = torch.from_numpy(f["scales"])
    assert torch.equal(scales, x.abs().amax(-1) * torch.tensor(1.0 / 448.0))
    q = torch.from_numpy(f["q_u8"]).view(torch.float8_e4m3fn).float().view(6, 3, 128)
    assert (q[1, 1] == 0).all() or torch.isnan(q[1, 1]).all()          # an all-zero group: 0 / 0
    live = scales > 0
    assert (q.abs().amax(-1)[live] == 448).all()                       # the largest element of a group maps to 448
    deq = q * scales[..., None]
    # half an e4m3 step (3 mantissa bits) of the magnitude, or half the smallest subnormal step (2^-9) times the scale
    bound = torch.maximum(2.0**-4 * x.abs(), 2.0**-10 * scales[..., None].expand_as(x))
    assert ((deq - x).abs()[live] <= bound[live] * 1.0001).all()


# ---- GPU: the HIP path against the frozen vectors ------------------------------------------------------
@pytest.mark.gpu
def test_gpu_against_fixtures(cuda):
    from triton_dist.kernels.amd import (create_all_to_all_context, fast_all_to_all, gated_gemm, moe_dispatch_preprocess,
                                         moe_weighted_combine)
    from triton_dist.kernels.amd.flash_decode import _split_kv
    from triton_dist.kernels.amd.gemm_reduce_scatter import ring_reduce_after_scatter
    announce("fixtures: moe")
    f = load("moe_64x8x16.npz")
    T, topk, G, W, H, max_m = f["meta"].tolist()
    ids = torch.from_numpy(f["ids"]).to(cuda)
    splits, cumsum, scatter, gather = moe_dispatch_preprocess(ids, G)
    assert np.array_equal(splits.cpu().numpy(), f["splits"]) and np.array_equal(cumsum.cpu().numpy(), f["cumsum"])
    assert np.array_equal(scatter.cpu().numpy(), f["scatter_idx"]) and np.array_equal(gather.cpu().numpy(), f["gather_idx"])
    ctx = create_all_to_all_context(max_m, H, 0, G, W, G // W, dtype=torch.float8_e4m3fn)
    ctx.recv_buf.view(torch.uint8).zero_()
    ctx.scale_recv_buf.zero_()
    rows = torch.from_numpy(f["rows_u8"]).to(cuda).view(torch.float8_e4m3fn)
    _, recv, recv_scale = fast_all_to_all(ctx, rows, cumsum, torch.from_numpy(f["scales"]).to(cuda), scatter_index=scatter)
    y = moe_weighted_combine(ctx, recv, recv_scale, scatter, torch.from_numpy(f["weights"]).to(cuda), cumsum)
    torch.cuda.synchronize()
    assert np.array_equal(recv.view(torch.uint8).cpu().numpy(), f["recv_u8"])
    assert np.array_equal(recv_scale.cpu().numpy(), f["recv_scale"])
    assert golden.max_rel_err(y.float().cpu(), torch.from_numpy(f["combined_f32"])) <= 1e-2
    announce("fixtures: reduce, gemm")
    r = load("reduce_8x4096.npz")
    out = ring_reduce_after_scatter(0, 8, bf16(r["slices"]).view(8 * 64, 64).to(cuda), torch.cuda.current_stream())
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().view(torch.int16).numpy().view(np.uint16).reshape(-1), r["out"])
    g = load("gemm_small.npz")
    a, b = bf16(g["a_bf16"]).to(cuda), bf16(g["b_bf16"]).to(cuda)
    c = torch.empty((a.shape[0], b.shape[0]), dtype=torch.bfloat16, device=cuda)
    gated_gemm(a, None, 0, b, c, None, 0, 0, 1)
    a8 = torch.from_numpy(g["a_e4m3"]).to(cuda).view(torch.float8_e4m3fn)
    b8 = torch.from_numpy(g["b_e4m3"]).to(cuda).view(torch.float8_e4m3fn)
    c8 = torch.empty((a8.shape[0], b8.shape[0]), dtype=torch.bfloat16, device=cuda)
    gated_gemm(a8, None, 0, b8, c8, None, 0, 0, 1, row_scale=torch.from_numpy(g["row_scale"]).to(cuda),
               col_scale=torch.from_numpy(g["col_scale"]).to(cuda))
    torch.cuda.synchronize()
    assert golden.max_rel_err(c.float().cpu(), torch.from_numpy(g["c_f32"])) <= 1e-2
    assert golden.max_rel_err(c8.float().cpu(), torch.from_numpy(g["c8_f32"])) <= 1e-2
    announce("fixtures: decode")
    d = load("decode_2seq.npz")
    Hq, Hkv, D, page, S = d["meta"].tolist()
    out_split, lse_split, _ = _split_kv(bf16(d["q"]).to(cuda), bf16(d["k_cache"]).to(cuda), bf16(d["v_cache"]).to(cuda),
                                        torch.from_numpy(d["kv_lens"]).to(cuda), torch.from_numpy(d["block_table"]).to(cuda),
                                        D**-0.5, 0.0, S)
    torch.cuda.synchronize()
    assert np.abs(out_split.cpu().numpy() - d["part"]).max() <= 2e-3
    finite = np.isfinite(d["part_lse"])
    assert np.array_equal(np.isfinite(lse_split.cpu().numpy()), finite)
    assert np.abs(lse_split.cpu().numpy()[finite] - d["part_lse"][finite]).max() <= 2e-3
    announce("fixtures: decode with extra key dimensions, align / sort, group quantiser")
    d = load("decode_dk192_dv128.npz")
    Hq, Hkv, Dk, Dv, page, S, cap = d["meta"].tolist()
    out_split, lse_split, _ = _split_kv(f16(d["q"]).to(cuda), f16(d["k_cache"]).to(cuda), f16(d["v_cache"]).to(cuda),
                                        torch.from_numpy(d["kv_lens"]).to(cuda), torch.from_numpy(d["block_table"]).to(cuda),
                                        Dk**-0.5, float(cap), S)
    torch.cuda.synchronize()
    assert np.abs(out_split.cpu().numpy() - d["part"]).max() <= 2e-3
    finite = np.isfinite(d["part_lse"])
    assert np.array_equal(np.isfinite(lse_split.cpu().numpy()), finite)
    assert np.abs(lse_split.cpu().numpy()[finite] - d["part_lse"][finite]).max() <= 2e-3
    from triton_dist.kernels.amd import quant_bf16_fp8, sort_topk_ids_align_block_size
    a = load("moe_align_4x24x3.npz")
    R, Tr, topk, E, block, post_pad = a["meta"].tolist()
    got = sort_topk_ids_align_block_size(torch.from_numpy(a["ids"]).to(cuda), E, R, Tr, block)
    torch.cuda.synchronize()
    assert int(got[4]) == post_pad
    assert np.array_equal(got[0].cpu().numpy()[:a["sorted_token_ids"].size], a["sorted_token_ids"])
    nb = post_pad // block
    assert np.array_equal(got[1].cpu().numpy()[:nb], a["expert_ids"]) and np.array_equal(got[2].cpu().numpy()[:nb], a["block_barrier_ids"])
    assert np.array_equal(got[3].cpu().numpy(), a["rank_block_num"])
    qf = load("quant_groups_6x384.npz")
    qx, sx = quant_bf16_fp8(bf16(qf["x"]).to(cuda))
    torch.cuda.synchronize()
    assert np.array_equal(sx.cpu().numpy(), qf["scales"])
    want_q, got_q = qf["q_u8"].reshape(6, 3, 128), qx.view(torch.uint8).cpu().numpy().reshape(6, 3, 128)
    live = qf["scales"] > 0
    assert np.array_equal(got_q[live], want_q[live])      # (an all-zero group is 0 / 0: NaN on both sides, payload free)
