"""Writes the small committed fixtures under tests/golden/ from the oracle (oracle/golden.py), in this
container, on the CPU:

    python tests/golden/make_fixtures.py

The reference keeps no stored vectors for this path (its goldens are computed at run time), so these are the
oracle's outputs on seeded inputs, frozen so that a later change to the oracle or to a kernel shows up as a
diff against data rather than against code. Inputs and expected outputs only — no reference source.
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
from oracle import golden  # noqa: E402


def bits16(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def main():
    # OCP e4m3fn decode table: all 256 byte values (NaN at 0x7f / 0xff stored as NaN)
    table = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).float().numpy()
    np.savez_compressed(os.path.join(HERE, "e4m3_table.npz"), table=table)

    # MoE: 64 tokens x top-8 over 16 experts, 4 destinations, hidden 64 (e4m3 rows + fp32 scales)
    g = torch.Generator().manual_seed(101)
    T, topk, G, W, H, max_m = 64, 8, 16, 4, 64, 192
    ids = golden.random_distinct_experts(T, G, topk, g)
    q, s = golden.quantize_per_token_e4m3(torch.randn((T, H), generator=g))
    w = torch.softmax(torch.randn((T, topk), generator=g), dim=-1).float()
    splits, cumsum, scatter, gather, topk_idx = golden.moe_preprocess(ids, G)
    rows = q.view(torch.uint8)[gather.long()]
    scales = s[gather.long()]
    _, recv, recv_scale = golden.dispatch_slots(rows, scales, cumsum, W, G // W, max_m, fill_byte=0)
    y = golden.weighted_combine(q[gather.long()].float(), scales, scatter, w)
    np.savez_compressed(os.path.join(HERE, "moe_64x8x16.npz"), ids=ids.numpy(), rows_u8=q.view(torch.uint8).numpy(),
                        scales=s.numpy(), weights=w.numpy(), splits=splits.numpy(), cumsum=cumsum.numpy(),
                        scatter_idx=scatter.numpy(), gather_idx=gather.numpy(), topk_idx=topk_idx.numpy(),
                        recv_u8=recv.numpy(), recv_scale=recv_scale.numpy(), combined_f32=y.numpy(),
                        meta=np.array([T, topk, G, W, H, max_m]))

    # GEMM: bf16 [192,128] x [160,128]^T and e4m3 [128,128] x [96,128]^T with scales; fp32 references
    g = torch.Generator().manual_seed(102)
    a = torch.randn((192, 128), generator=g).to(torch.bfloat16)
    b = (torch.randn((160, 128), generator=g) * 0.02).to(torch.bfloat16)
    c = golden.ag_gemm_fp32([a[:64], a[64:128], a[128:]], b)
    a8 = torch.randn((128, 128), generator=g).to(torch.float8_e4m3fn)
    b8 = torch.randn((96, 128), generator=g).to(torch.float8_e4m3fn)
    sa = torch.rand(128, generator=g) * 0.09 + 0.01
    sb = torch.rand(96, generator=g) * 0.009 + 0.001
    c8 = golden.fp8_scaled_gemm_fp32(a8, sa, b8, sb)
    np.savez_compressed(os.path.join(HERE, "gemm_small.npz"), a_bf16=bits16(a), b_bf16=bits16(b), c_f32=c.numpy(),
                        a_e4m3=a8.view(torch.uint8).numpy(), b_e4m3=b8.view(torch.uint8).numpy(), row_scale=sa.numpy(),
                        col_scale=sb.numpy(), c8_f32=c8.numpy())

    # slice reduction: 8 x 4096 bf16, first slice 1 (rank 0), bit patterns of the result
    g = torch.Generator().manual_seed(103)
    sl = torch.randn((8, 4096), generator=g).to(torch.bfloat16)
    np.savez_compressed(os.path.join(HERE, "reduce_8x4096.npz"), slices=bits16(sl),
                        out=bits16(golden.reduce_slices_ordered(sl, 1)))

    # decode: 2 sequences (293 and 70 keys), 16 query heads over 2 kv heads, D 128, page 16, 4 splits, bf16
    g = torch.Generator().manual_seed(104)
    kv_lens, Hq, Hkv, D, page, S = [293, 70], 16, 2, 128, 16, 4
    qd = torch.randn((2, Hq, D), generator=g).to(torch.bfloat16)
    k_cache, v_cache, table = golden.make_paged_kv(2, max(kv_lens), Hkv, D, page, torch.bfloat16, g)
    scale = D**-0.5
    out, lse = golden.decode_exact(qd, k_cache, v_cache, kv_lens, table, scale)
    part, part_lse = golden.decode_split_exact(qd, k_cache, v_cache, kv_lens, table, scale, S)
    np.savez_compressed(os.path.join(HERE, "decode_2seq.npz"), q=bits16(qd), k_cache=bits16(k_cache), v_cache=bits16(v_cache),
                        block_table=table.numpy(), kv_lens=np.array(kv_lens, dtype=np.int32), out=out.numpy(), lse=lse.numpy(),
                        part=part.numpy(), part_lse=part_lse.numpy(), meta=np.array([Hq, Hkv, D, page, S]))

    # decode with extra key dimensions: 2 sequences (100 and 37 keys), 4 query heads over 1 kv head, key dim 192,
    # value dim 128, page 4, 3 splits, f16, soft cap 30
    g = torch.Generator().manual_seed(105)
    kv_lens, Hq, Hkv, Dk, Dv, page, S, cap = [100, 37], 4, 1, 192, 128, 4, 3, 30.0
    qd = torch.randn((2, Hq, Dk), generator=g).to(torch.float16)
    k_cache, v_cache, table = golden.make_paged_kv(2, max(kv_lens), Hkv, Dk, page, torch.float16, g, v_head_dim=Dv)
    scale = Dk**-0.5
    out, lse = golden.decode_exact(qd, k_cache, v_cache, kv_lens, table, scale, cap)
    part, part_lse = golden.decode_split_exact(qd, k_cache, v_cache, kv_lens, table, scale, S, cap)
    np.savez_compressed(os.path.join(HERE, "decode_dk192_dv128.npz"), q=bits16(qd), k_cache=bits16(k_cache),
                        v_cache=bits16(v_cache), block_table=table.numpy(), kv_lens=np.array(kv_lens, dtype=np.int32),
                        out=out.numpy(), lse=lse.numpy(), part=part.numpy(), part_lse=part_lse.numpy(),
                        meta=np.array([Hq, Hkv, Dk, Dv, page, S, int(cap)]))

    # align / sort for the grouped GEMM: 4 rank segments x 24 tokens x top-3 over 10 experts, block 8
    g = torch.Generator().manual_seed(106)
    R, Tr, topk, E, block = 4, 24, 3, 10, 8
    ids = golden.random_distinct_experts(R * Tr, E, topk, g)
    sorted_ids, expert_ids, barrier_ids, rank_blocks, post_pad = golden.sort_topk_ids_align_block_size(ids, E, R, Tr, block)
    np.savez_compressed(os.path.join(HERE, "moe_align_4x24x3.npz"), ids=ids.numpy(), sorted_token_ids=sorted_ids.numpy(),
                        expert_ids=expert_ids.numpy(), block_barrier_ids=barrier_ids.numpy(),
                        rank_block_num=rank_blocks.numpy(), meta=np.array([R, Tr, topk, E, block, int(post_pad)]))

    # e4m3 quantisation in groups of 128 columns: 6 rows x 384 columns bf16 (one all-zero group, one with a huge entry)
    g = torch.Generator().manual_seed(107)
    x = torch.randn((6, 384), generator=g)
    x[1, 128:256] = 0.0
    x[2, 5] = 3.0e4
    x = x.to(torch.bfloat16)
    qx, sx = golden.quantize_groups_e4m3(x)
    np.savez_compressed(os.path.join(HERE, "quant_groups_6x384.npz"), x=bits16(x), q_u8=qx.view(torch.uint8).numpy(),
                        scales=sx.numpy())

    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")


if __name__ == "__main__":
    main()
