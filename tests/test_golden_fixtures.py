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
