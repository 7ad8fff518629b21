"""CPU restatements (torch / numpy) of the reference's golden computations for the four hot-path ops.

TEST INFRASTRUCTURE ONLY. Nothing under oracle/ is imported by the product (triton-distributed_amd/): only
tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg use it, and only as the checker.

Every function cites the reference lines (paths relative to python/triton_dist of Triton-distributed) it
follows. Collectives in the reference's goldens are replaced by their closed forms on one process:
all_gather = concatenation, reduce_scatter = sum then slice, all_to_all = split and concatenate.

Pinning (what keeps each restatement honest) is listed per function; the cross-checks live in
tests/test_oracle.py. "parity unpinned" marks a function no reference test covers.
"""
import math
from typing import List, Optional, Sequence

import numpy as np
import torch

# ---------------------------------------------------------------------------------------------------
# (a) AG-GEMM
# ---------------------------------------------------------------------------------------------------


def torch_ag_gemm(shards: Sequence[torch.Tensor], weight: torch.Tensor) -> torch.Tensor:
    """test/amd/test_ag_gemm_intra_node.py:45-69 (torch_ag_gemm) with all_gather_into_tensor replaced by
    torch.cat: output = cat(shards) @ weight.T in the input dtype. weight is [N, K].
    Pinned by: ag_gemm_fp32 (closed form in fp32) within bf16 rounding; brute-force C triple loop on small
    integer-valued inputs (exact)."""
    full_input = torch.cat(list(shards), dim=0)
    return torch.matmul(full_input, weight.T)


def ag_gemm_fp32(shards: Sequence[torch.Tensor], weight: torch.Tensor) -> torch.Tensor:
    """The fp32 reference the GEMM outputs are judged against: cat(shards).float() @ weight.float().T."""
    return torch.cat([s.float() for s in shards], dim=0) @ weight.float().T


def fp8_scaled_gemm_fp32(a8: torch.Tensor, row_scale: Optional[torch.Tensor], b8: torch.Tensor,
                         col_scale: Optional[torch.Tensor]) -> torch.Tensor:
    """C = (A8 . B8^T) * sa[m] * sb[n] in fp32; a8 [M,K], b8 [N,K] float8_e4m3fn.
    PARITY UNPINNED: the reference has no scaled fp8 GEMM (fp8 is a dtype passthrough,
    kernels/nvidia/allgather_gemm.py:313). Pinned only by mathematics: the e4m3 decode table (all 256
    bytes) and the C triple loop on small inputs."""
    c = a8.float() @ b8.float().T
    if row_scale is not None:
        c = c * row_scale.float()[:, None]
    if col_scale is not None:
        c = c * col_scale.float()[None, :]
    return c


def max_rel_err(out: torch.Tensor, ref: torch.Tensor) -> float:
    """max |out-ref| / max|ref|: the 'max relative error' the GEMM bar (<= 1e-2) is stated in."""
    ref = ref.double()
    return float((out.double() - ref).abs().max() / ref.abs().max().clamp_min(1e-30))


# ---------------------------------------------------------------------------------------------------
# (b) GEMM-RS
# ---------------------------------------------------------------------------------------------------


def reduce_slices_ordered(c: torch.Tensor, first: int) -> torch.Tensor:
    """kernels/amd/gemm_reduce_scatter.py:246-258 (kernel_consumer_reduce): sum of the R slices c[R, ...] in
    the order first, first+1, ... (the kernel's cur_rank = (i + rank + 1) % R), but accumulated in fp32 and
    rounded once to c's dtype — bit-exact target for the HIP reduction.
    Pinned by: the scalar C loop (oracle/c); equality with a plain fp32 sum when R <= 2 (order-free);
    linearity checks."""
    R = c.shape[0]
    acc = torch.zeros(c.shape[1:], dtype=torch.float32)
    for i in range(R):
        acc = acc + c[(first + i) % R].float()
    return acc.to(c.dtype)


def torch_gemm_rs(a: torch.Tensor, weight: torch.Tensor, peer_partials: Sequence[Optional[torch.Tensor]], rank: int,
                  world_size: int) -> torch.Tensor:
    """test/amd/test_gemm_rs_intra_node.py:46-62 (torch_gemm_rs): output = a @ weight.T (input dtype), then
    reduce_scatter_tensor = sum over ranks of each rank's output, rows of ``rank`` kept. Peers contribute their
    partial slices [M/world, N] directly (peer_partials[r], entry ``rank`` ignored). The sum runs in fp32 in
    the kernel's slice order and is rounded once."""
    M = a.shape[0]
    m_per = M // world_size
    own = torch.matmul(a, weight.T)[rank * m_per:(rank + 1) * m_per]
    slices = [own if r == rank else peer_partials[r] for r in range(world_size)]
    return reduce_slices_ordered(torch.stack(slices, 0), (rank + 1) % world_size)


def gemm_rs_fp32(a, weight, peer_partials, rank, world_size) -> torch.Tensor:
    """fp32 closed form: (a.float() @ w.float().T)[rank rows] + sum of peers (no intermediate rounding)."""
    M = a.shape[0]
    m_per = M // world_size
    acc = (a.float() @ weight.float().T)[rank * m_per:(rank + 1) * m_per].clone()
    for r in range(world_size):
        if r != rank:
            acc += peer_partials[r].float()
    return acc


# ---------------------------------------------------------------------------------------------------
# (c) MoE dispatch / combine
# ---------------------------------------------------------------------------------------------------


def splits_to_cumsum(splits: torch.Tensor) -> torch.Tensor:
    """test/nvidia/test_all_to_all.py:42-46."""
    out = torch.empty(splits.shape[0] + 1, dtype=splits.dtype)
    out[0] = 0
    torch.cumsum(splits, 0, out=out[1:])
    return out


def calc_scatter_index_stable(choosed_experts: torch.Tensor) -> torch.Tensor:
    """test/nvidia/test_all_to_all.py:95-96."""
    return choosed_experts.flatten().argsort(stable=True).argsort().int().view(choosed_experts.shape)


def calc_gather_index(scatter_index: torch.Tensor, row_start: int, row_end: int):
    """test/nvidia/test_all_to_all.py:49-92 (the Triton helper restated with numpy indexing): for every flat
    entry whose sorted position p lies in [row_start, row_end): gather_index[p-row_start] = entry // topk,
    topk_index[p-row_start] = entry % topk."""
    ntokens, topk = scatter_index.shape
    flat = scatter_index.flatten().numpy().astype(np.int64)
    gather = np.zeros(row_end - row_start, dtype=np.int32)
    topk_index = np.zeros(row_end - row_start, dtype=np.int32)
    entry = np.arange(ntokens * topk, dtype=np.int64)
    sel = (flat >= row_start) & (flat < row_end)
    gather[flat[sel] - row_start] = (entry[sel] // topk).astype(np.int32)
    topk_index[flat[sel] - row_start] = (entry[sel] % topk).astype(np.int32)
    return torch.from_numpy(gather), torch.from_numpy(topk_index)


def moe_preprocess(exp_indices: torch.Tensor, num_experts: int):
    """test/nvidia/test_all_to_all.py:314-320 (perf_triton's index preparation).
    Pinned by: the sequential C counting sort (oracle/c), and the invariants cumsum[-1] == T*topk,
    gather_idx[scatter_idx[t,k]] == t, positions of one expert increasing with the flat index."""
    splits = torch.bincount(exp_indices.view(-1).long(), minlength=num_experts).to(torch.int32)
    cumsum = splits_to_cumsum(splits)
    scatter_idx = calc_scatter_index_stable(exp_indices)
    gather_idx, topk_idx = calc_gather_index(scatter_idx, 0, exp_indices.numel())
    return splits, cumsum, scatter_idx, gather_idx, topk_idx


def dispatch_slots(sorted_rows: torch.Tensor, sorted_scales: Optional[torch.Tensor], cumsum: torch.Tensor,
                   world_size: int, experts_per_rank: int, max_m: int, fill_byte: int = 0):
    """kernels/nvidia/low_latency_all_to_all.py:56-103 (all_to_all_kernel) with every destination's receive
    slot for this sender kept side by side: rows [cumsum[d*Er], cumsum[(d+1)*Er]) go to
    recv[d*max_m : d*max_m + n_d]; splits_out[g] = cumsum[g+1]-cumsum[g] (:70-74). Untouched slot rows keep
    ``fill_byte``. Returns (splits, recv_bytes [W*max_m, row_bytes] uint8, scales [W*max_m] | None)."""
    rows_u8 = sorted_rows.contiguous().view(torch.uint8).reshape(sorted_rows.shape[0], -1)
    recv = torch.full((world_size * max_m, rows_u8.shape[1]), fill_byte, dtype=torch.uint8)
    scales = torch.zeros(world_size * max_m, dtype=torch.float32) if sorted_scales is not None else None
    for d in range(world_size):
        st, ed = int(cumsum[d * experts_per_rank]), int(cumsum[(d + 1) * experts_per_rank])
        n = min(ed - st, max_m)
        recv[d * max_m:d * max_m + n] = rows_u8[st:st + n]
        if scales is not None:
            scales[d * max_m:d * max_m + n] = sorted_scales[st:st + n]
    splits = (cumsum[1:] - cumsum[:-1]).to(torch.int32)
    return splits, recv, scales


def all_to_all_post_process(input_splits: torch.Tensor, recv_buffer: torch.Tensor, scale_buffer, world_size: int,
                            max_m: int):
    """kernels/nvidia/low_latency_all_to_all.py:251-270."""
    num_tokens_from_each_rank = input_splits.reshape(world_size, -1).sum(dim=1)
    data_vec, scale_vec = [], []
    for i in range(world_size):
        n = int(num_tokens_from_each_rank[i])
        data_vec.append(recv_buffer[i * max_m:i * max_m + n])
        if scale_buffer is not None:
            scale_vec.append(scale_buffer[i * max_m:i * max_m + n])
    return torch.concat(data_vec), (torch.concat(scale_vec) if scale_buffer is not None else None)


def combine_index_add(combine_token: torch.Tensor, gather_idx: torch.Tensor, n_tokens: int) -> torch.Tensor:
    """test/nvidia/test_all_to_all.py:366-367: zeros.index_add_(0, gather_idx, combine_token) (in fp32)."""
    out = torch.zeros((n_tokens, combine_token.shape[1]), dtype=torch.float32)
    out.index_add_(0, gather_idx.long(), combine_token.float())
    return out


def weighted_combine(sorted_rows_f32: torch.Tensor, sorted_scales: Optional[torch.Tensor], scatter_idx: torch.Tensor,
                     topk_weight: Optional[torch.Tensor]) -> torch.Tensor:
    """test/nvidia/test_moe_reduce_rs.py:117-122 (out[mask] = (x @ w) * topk_weight[mask, None]; sum over topk)
    with the identity expert: y[t] = sum_k w[t,k] * (scale[p] * row[p]), p = scatter_idx[t,k], fp32, k in
    order 0..topk-1. Returns fp32 [T, H].
    Pinned by: combine_index_add when w == 1 and scales == 1 (reference round trip == topk * x,
    test_all_to_all.py:370), and the scalar C loop."""
    T, topk = scatter_idx.shape
    out = torch.zeros((T, sorted_rows_f32.shape[1]), dtype=torch.float32)
    for k in range(topk):
        p = scatter_idx[:, k].long()
        coef = torch.ones(T, dtype=torch.float32) if topk_weight is None else topk_weight[:, k].float()
        if sorted_scales is not None:
            coef = coef * sorted_scales[p].float()
        out += coef[:, None] * sorted_rows_f32[p]
    return out


def quantize_per_token_e4m3(x: torch.Tensor):
    """Input generator only (both sides consume its output): s = max|x| / 448 per token, q = (x / s) as e4m3.
    Follows the per-group quantiser of tutorials/04-deepseek-infer-all2all.py:309-329 with one group per token."""
    s = x.abs().amax(dim=1).clamp_min(1e-12) / 448.0
    q = (x / s[:, None]).to(torch.float8_e4m3fn)
    return q, s.float()


def random_distinct_experts(n_tokens: int, num_experts: int, topk: int, generator: torch.Generator) -> torch.Tensor:
    """test/nvidia/test_all_to_all.py:175-181 (random.sample per token) with torch's generator: topk distinct
    uniformly random experts per token, int32 [T, topk]."""
    scores = torch.rand((n_tokens, num_experts), generator=generator)
    return scores.argsort(dim=1)[:, :topk].to(torch.int32).contiguous()


# ---------------------------------------------------------------------------------------------------
# (d) flash decode
# ---------------------------------------------------------------------------------------------------


def ref_paged_attn(query: torch.Tensor, key_cache: torch.Tensor, value_cache: torch.Tensor, query_lens: List[int],
                   kv_lens: List[int], block_tables: torch.Tensor, scale: float, soft_cap: Optional[float] = None):
    """test/nvidia/test_decode_attn.py:70-120 (ref_paged_attn; the sliding-window branch, unused by the decode
    tests, is left out). Does not scale ``query`` in place (the reference's ``q *= scale`` mutates its input)."""
    num_seqs = len(query_lens)
    block_tables = block_tables.cpu().numpy()
    _, block_size, num_kv_heads, head_size = key_cache.shape
    outputs = []
    start_idx = 0
    for i in range(num_seqs):
        query_len = query_lens[i]
        kv_len = kv_lens[i]
        q = query[start_idx:start_idx + query_len] * scale
        num_kv_blocks = (kv_len + block_size - 1) // block_size
        block_indices = block_tables[i, :num_kv_blocks]
        k = key_cache[block_indices].view(-1, num_kv_heads, head_size)[:kv_len]
        v = value_cache[block_indices].view(-1, num_kv_heads, value_cache.shape[-1])[:kv_len]   # (the reference: head_size)
        if q.shape[1] != k.shape[1]:
            k = torch.repeat_interleave(k, q.shape[1] // k.shape[1], dim=1)
            v = torch.repeat_interleave(v, q.shape[1] // v.shape[1], dim=1)
        attn = torch.einsum("qhd,khd->hqk", q, k).float()
        empty_mask = torch.ones(query_len, kv_len)
        mask = torch.triu(empty_mask, diagonal=kv_len - query_len + 1).bool()
        if soft_cap is not None and soft_cap > 0.0:
            attn = soft_cap * torch.tanh(attn / soft_cap)
        attn.masked_fill_(mask, float("-inf"))
        attn = torch.softmax(attn, dim=-1).to(v.dtype)
        out = torch.einsum("hqk,khd->qhd", attn, v)
        outputs.append(out)
        start_idx += query_len
    return torch.cat(outputs, dim=0)


def _gather_kv(cache: torch.Tensor, table_row: np.ndarray, lo: int, hi: int) -> torch.Tensor:
    """Keys lo..hi-1 of one sequence: token n lives in page table[n // page_size], slot n % page_size
    (kernels/nvidia/flash_decode.py:203-205)."""
    page_size = cache.shape[1]
    n = np.arange(lo, hi)
    pages = table_row[n // page_size].astype(np.int64)
    return cache[torch.from_numpy(pages), torch.from_numpy(n % page_size)]  # [hi-lo, Hkv, D]


def decode_exact(query, key_cache, value_cache, kv_lens, block_tables, scale, soft_cap=0.0, lo_hi=None):
    """Exact (fp64) decode attention and log-sum-exp over keys [lo, hi) of every sequence: the closed form
    softmax(q.k*scale [soft-capped]) . v and LSE = logsumexp(scores) the split / combine kernels are checked
    against (kernels/nvidia/flash_decode.py:207-239 without its online-softmax bookkeeping).
    Returns (out fp64 [B,Hq,Dv], lse fp64 [B,Hq]); an empty range gives out = 0, lse = -inf.
    Pinned by: ref_paged_attn above (agreement within its bf16 rounding) and the scalar C loop."""
    B, Hq, D = query.shape
    Hkv = key_cache.shape[2]
    group = Hq // Hkv
    tables = block_tables.cpu().numpy()
    outs = torch.zeros((B, Hq, value_cache.shape[-1]), dtype=torch.float64)
    lses = torch.full((B, Hq), float("-inf"), dtype=torch.float64)
    for b in range(B):
        lo, hi = (0, int(kv_lens[b])) if lo_hi is None else lo_hi[b]
        if hi <= lo:
            continue
        k = _gather_kv(key_cache, tables[b], lo, hi).double()    # [n, Hkv, D]
        v = _gather_kv(value_cache, tables[b], lo, hi).double()
        k = torch.repeat_interleave(k, group, dim=1)
        v = torch.repeat_interleave(v, group, dim=1)
        s = torch.einsum("hd,nhd->hn", query[b].double(), k) * scale
        if soft_cap and soft_cap > 0.0:
            s = soft_cap * torch.tanh(s / soft_cap)
        lse = torch.logsumexp(s, dim=-1)
        p = torch.exp(s - lse[:, None])
        outs[b] = torch.einsum("hn,nhd->hd", p, v)
        lses[b] = lse
    return outs, lses


def split_ranges(kv_len: int, num_splits: int):
    """kernels/nvidia/flash_decode.py:193-195: per = cdiv(len, S); split s covers [per*s, min(per*s+per, len))."""
    per = (kv_len + num_splits - 1) // num_splits
    return [(per * s, min(per * s + per, kv_len)) for s in range(num_splits)]


def decode_split_exact(query, key_cache, value_cache, kv_lens, block_tables, scale, num_splits, soft_cap=0.0):
    """Per-split exact partials: out [B,Hq,S,Dv], lse [B,Hq,S] (fp64)."""
    B, Hq, _ = query.shape
    Dv = value_cache.shape[-1]
    out = torch.zeros((B, Hq, num_splits, Dv), dtype=torch.float64)
    lse = torch.full((B, Hq, num_splits), float("-inf"), dtype=torch.float64)
    ranges = [split_ranges(int(kv_lens[b]), num_splits) for b in range(B)]
    for s in range(num_splits):
        o, l = decode_exact(query, key_cache, value_cache, kv_lens, block_tables, scale, soft_cap,
                            lo_hi=[ranges[b][s] for b in range(B)])
        out[:, :, s] = o
        lse[:, :, s] = l
    return out, lse


def lse_merge(parts: torch.Tensor, lses: torch.Tensor, skip: Optional[torch.Tensor] = None):
    """kernels/nvidia/flash_decode.py:423-449 and :512-532 as a closed form: partials along dim 0 are merged
    with weights exp(lse_j - max); skipped partials (bool mask, dim-0 aligned) get weight 0.
    parts [P, ..., Dv], lses [P, ...]. Returns (out fp64 [..., Dv], lse fp64 [...]).
    Pinned by: merging the exact partials of any partition of the keys must reproduce decode_exact over all
    keys (the log-sum-exp identity)."""
    lses = lses.double().clone()
    if skip is not None:
        lses[skip] = float("-inf")
    m = lses.max(dim=0).values
    m_safe = torch.where(torch.isinf(m), torch.zeros_like(m), m)
    w = torch.exp(lses - m_safe)
    w = torch.where(torch.isinf(lses), torch.zeros_like(w), w)
    denom = w.sum(dim=0)
    out = (w[..., None] * parts.double()).sum(dim=0) / denom.clamp_min(1e-300)[..., None]
    out = torch.where((denom == 0)[..., None], torch.zeros_like(out), out)
    lse = torch.where(denom == 0, torch.full_like(m, float("-inf")), m_safe + torch.log(denom.clamp_min(1e-300)))
    return out, lse


def make_paged_kv(batch: int, kv_len_max: int, kv_heads: int, head_dim: int, page_size: int, dtype,
                  generator: torch.Generator, extra_pages: int = 3, v_head_dim: Optional[int] = None):
    """Random K/V caches [num_pages, page_size, Hkv, D] and a block table that maps every sequence to a random,
    disjoint set of pages (the data layout of test/nvidia/test_decode_attn.py:148-156, with a permutation
    instead of randint so that no two sequences alias)."""
    pages_per_seq = (kv_len_max + page_size - 1) // page_size
    num_pages = batch * pages_per_seq + extra_pages
    k_cache = torch.randn((num_pages, page_size, kv_heads, head_dim), generator=generator).to(dtype)
    v_cache = torch.randn((num_pages, page_size, kv_heads, v_head_dim or head_dim), generator=generator).to(dtype)
    perm = torch.randperm(num_pages, generator=generator)[:batch * pages_per_seq]
    block_table = perm.view(batch, pages_per_seq).to(torch.int32).contiguous()
    return k_cache, v_cache, block_table


# ---------------------------------------------------------------------------------------------------
# MoE align / sort for the grouped GEMM (the step after the dispatch)
# ---------------------------------------------------------------------------------------------------
def sort_topk_ids_align_block_size(topk_ids, num_experts, num_ranks, num_tokens_per_rank, block_size):
    """Restates moe_ag_scatter_align_block_size_kernel (csrc/lib/moe_utils.cu:60-165) as called by
    sort_topk_ids_align_block_size (kernels/nvidia/allgather_group_gemm.py:54-135).

    topk_ids [num_ranks * num_tokens_per_rank, topk]. Per rank segment (``iter`` in the kernel), in order: the
    flat entries of the segment are grouped by expert, stably (:144-158); every expert's group is padded to a
    multiple of ``block_size`` (:115-121); the padded groups are laid end to end, segment after segment (:72-75).
    Returns (sorted_token_ids int32 [capacity] pre-filled with topk_ids.numel() (:115-116 of the Python),
    expert_ids int32 [n_blocks], block_barrier_ids int32 [n_blocks], rank_block_num int32 [num_ranks],
    num_tokens_post_pad int). expert_ids / block_barrier_ids are returned at their valid length (the reference
    leaves the tail of its torch.empty buffers unwritten)."""
    topk = topk_ids.shape[1]
    flat = topk_ids.reshape(-1).to(torch.int64)
    per = num_tokens_per_rank * topk
    assert flat.numel() == per * num_ranks
    capacity = (per + num_experts * (block_size - 1)) * num_ranks
    sorted_ids = torch.full((capacity, ), flat.numel(), dtype=torch.int32)
    expert_ids, barrier_ids, rank_block_num = [], [], []
    base = 0
    for it in range(num_ranks):
        seg = flat[it * per:(it + 1) * per]
        counts = torch.bincount(seg, minlength=num_experts)
        padded = (counts + block_size - 1) // block_size * block_size
        cum = torch.zeros(num_experts + 1, dtype=torch.int64)
        cum[1:] = torch.cumsum(padded, 0)
        order = torch.argsort(seg, stable=True)              # entries grouped by expert, original order kept
        sorted_e = seg[order]
        first = torch.zeros(num_experts + 1, dtype=torch.int64)
        first[1:] = torch.cumsum(counts, 0)
        within = torch.arange(per) - first[sorted_e]          # rank of each entry inside its expert's group
        sorted_ids[base + cum[sorted_e] + within] = (order + it * per).to(torch.int32)
        for e in range(num_experts):
            nb = int(padded[e]) // block_size
            expert_ids += [e] * nb
            barrier_ids += [it] * nb
        rank_block_num.append(int(cum[-1]) // block_size)
        base += int(cum[-1])
    return (sorted_ids, torch.tensor(expert_ids, dtype=torch.int32), torch.tensor(barrier_ids, dtype=torch.int32),
            torch.tensor(rank_block_num, dtype=torch.int32), base)


# ---------------------------------------------------------------------------------------------------
# e4m3 quantisation in groups of 128 columns (the fused form of the dispatch)
# ---------------------------------------------------------------------------------------------------
def torch_moe_scatter_group_gemm(in_features, expert_weights, topk_ids):
    """test/nvidia/test_ag_moe.py:20-38: every (token, k) row is the token's features times the weights of its k-th
    expert. in_features [M, K], expert_weights [E, K, N], topk_ids [M, topk] → [M * topk, N] in the input dtype."""
    M, K = in_features.shape
    in_features = in_features.view(M, -1, K).repeat(1, topk_ids.shape[1], 1).reshape(-1, K)
    out = torch.zeros(M * topk_ids.shape[1], expert_weights.shape[2], dtype=in_features.dtype, device=in_features.device)
    topk_ids = topk_ids.reshape(-1)
    for i in range(expert_weights.shape[0]):
        mask = topk_ids == i
        if mask.sum():
            out[mask] = in_features[mask] @ expert_weights[i]
    return out


def ag_group_gemm_fp32(shards, expert_weights, full_topk_ids):
    """Closed form of the AG + grouped GEMM (test/nvidia/test_ag_moe.py:41-56: all-gather of the ranks' token rows,
    then torch_moe_scatter_group_gemm) with fp32 operands and result: the reference the 1e-2 bar is taken against.
    Pinned by: row (t, k) of the result equals (cat(shards)[t].float() @ W[ids[t, k]].float()) by definition."""
    a = torch.cat([s.float() for s in shards], dim=0)
    return torch_moe_scatter_group_gemm(a, expert_weights.float(), full_topk_ids)


def torch_group_gemm_reduce_rs(intermediate_states, w, topk_ids, topk_weight, peer_partials, rank, world_size):
    """TorchGroupGemmReduceRS.forward (test/nvidia/test_moe_reduce_rs.py:103-133) in fp32, with its
    reduce_scatter_tensor written out: intermediate_states [M * topk, K] (row t*topk + k), w [E, K, hidden], topk_ids /
    topk_weight [M, topk]; out[t] = sum_k weight[t,k] * (states[t*topk+k] @ w[ids[t,k]]); this rank keeps rows
    [rank*M/W, (rank+1)*M/W) and adds the other ranks' partial results for them (``peer_partials``: list with one
    [M/W, hidden] tensor per rank, the own entry ignored), in the order rank+1, rank+2, ... Returns fp32.
    Pinned by: the per-row definition (brute force in tests/test_oracle.py)."""
    n_rows, _ = intermediate_states.shape
    topk = topk_ids.shape[1]
    M = n_rows // topk
    ids = topk_ids.reshape(-1)
    wt = topk_weight.reshape(-1).float()
    out = torch.zeros(n_rows, w.shape[2], dtype=torch.float32)
    for i in range(w.shape[0]):
        mask = ids == i
        if mask.sum():
            out[mask] = (intermediate_states[mask].float() @ w[i].float()) * wt[mask, None]
    out = out.reshape(M, topk, -1).sum(dim=1)
    m_per = M // world_size
    acc = None
    for step in range(world_size):
        r = (rank + 1 + step) % world_size
        part = out[rank * m_per:(rank + 1) * m_per] if r == rank else peer_partials[r].float()
        acc = part.clone() if acc is None else acc + part
    return acc


def quantize_groups_e4m3(x, group=128):
    """Restates _quant_kernel (tutorials/04-deepseek-infer-all2all.py:309-329; fused in the dispatch kernel at
    :180-200): per group, scale = max|x| as fp32 times fp32(1/448), q = e4m3(float(x) / scale). PARITY UNPINNED by
    the reference: tutorial code, no test or stored vector holds its outputs; pinned here by the closed form and by
    dequantise(quantise(x)) staying within half an e4m3 step of x."""
    m, N = x.shape
    g = x.float().view(m, N // group, group)
    scale = g.abs().amax(-1, keepdim=True) * torch.tensor(1.0 / 448.0, dtype=torch.float32)
    q = (g / scale).to(torch.float8_e4m3fn).view(m, N)
    return q, scale.view(m, N // group)


def dequantize_groups(q, scale, group=128):
    """_dequant_kernel (tutorials/04-deepseek-infer-all2all.py:333-351): bf16(float(q) * scale)."""
    m, N = q.shape
    return (q.float().view(m, N // group, group) * scale[..., None]).view(m, N).to(torch.bfloat16)
