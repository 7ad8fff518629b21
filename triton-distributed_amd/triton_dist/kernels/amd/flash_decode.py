"""Split-KV GQA flash decode on one MI355X and the LSE-weighted merges.

Keeps the launcher signatures of the reference's kernels/nvidia/flash_decode.py:
``gqa_fwd_batch_decode`` (:763-844), ``gqa_fwd_batch_decode_intra_rank`` (:847-928) and
``gqa_fwd_batch_decode_persistent`` (:931-1004). The per-split partial results are kept as an fp32
``[B, Hq, S, Dv]`` tensor plus an fp32 ``[B, Hq, S]`` LSE tensor (the reference packs the LSE into column
Dv of a ``[.., Dv+1]`` buffer of the query dtype, :235-239).
"""
from typing import Optional

import torch

from triton_dist import _lib

DEFAULT_KV_SPLITS = 32  # reference :777, :861


# (q/k head dim, v head dim) with compiled shapes of their own; beside them every equal pair that is a multiple of 8
# up to 256 runs on the shape of the next power of two (the reference splits a head into BLOCK_DMODEL + BLOCK_DPE and
# masks, kernels/nvidia/flash_decode.py:771-772)
SUPPORTED_HEAD_DIMS = ((64, 64), (128, 128), (256, 256), (192, 128), (576, 512))


def head_dims_supported(dk, dv):
    return (dk, dv) in SUPPORTED_HEAD_DIMS or (dk == dv and 0 < dk <= 256 and dk % 8 == 0)


def _check_inputs(q, k_cache, v_cache, kv_lens, block_table):
    _lib.require_cuda(q, k_cache, v_cache, kv_lens, block_table)
    batch, q_heads, q_head_dim = q.shape
    _, page_size, kv_heads, k_head_dim = k_cache.shape
    assert page_size == v_cache.shape[1] and kv_heads == v_cache.shape[2] and k_head_dim == q_head_dim
    v_head_dim = v_cache.shape[-1]
    assert q_heads % kv_heads == 0
    if not head_dims_supported(q_head_dim, v_head_dim):
        raise NotImplementedError("head dims (%d, %d); supported: equal ones that are a multiple of 8 up to 256 and %s" %
                                  (q_head_dim, v_head_dim, SUPPORTED_HEAD_DIMS[3:]))
    if q.dtype != k_cache.dtype or q.dtype != v_cache.dtype:
        raise TypeError("q, k_cache and v_cache must share one dtype")
    if q.stride(-1) != 1 or k_cache.stride(-1) != 1 or v_cache.stride(-1) != 1:
        raise ValueError("the head dimension must be contiguous")
    if kv_lens.dtype != torch.int32:
        kv_lens = kv_lens.to(torch.int32)
    if block_table.dtype != torch.int32:
        block_table = block_table.to(torch.int32)
    assert block_table.stride(-1) == 1
    return kv_lens, block_table


def _decode_args(q, k_cache, v_cache, out_split, lse_split, scale, soft_cap, block_table, kv_lens, num_splits):
    batch, q_heads, q_head_dim = q.shape
    _, page_size, kv_heads, _ = k_cache.shape
    return [q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), out_split.data_ptr(), lse_split.data_ptr(),
            float(scale), float(soft_cap), block_table.data_ptr(), kv_lens.data_ptr(), batch, q_heads, kv_heads,
            q_head_dim, v_cache.shape[-1], page_size, num_splits, q.stride(0), q.stride(1), k_cache.stride(0),
            k_cache.stride(1), k_cache.stride(2), v_cache.stride(0), v_cache.stride(1), v_cache.stride(2),
            block_table.stride(0), _lib.dtype_code(q.dtype)]


def _split_buffers(q, v_cache, num_splits, out_split, lse_split):
    batch, q_heads, _ = q.shape
    if out_split is None:
        out_split = torch.empty((batch, q_heads, num_splits, v_cache.shape[-1]), dtype=torch.float32, device=q.device)
    if lse_split is None:
        lse_split = torch.empty((batch, q_heads, num_splits), dtype=torch.float32, device=q.device)
    return out_split, lse_split


def _split_kv(q, k_cache, v_cache, kv_lens, block_table, scale, soft_cap, num_splits, out_split=None, lse_split=None):
    kv_lens, block_table = _check_inputs(q, k_cache, v_cache, kv_lens, block_table)
    out_split, lse_split = _split_buffers(q, v_cache, num_splits, out_split, lse_split)
    _lib.call("tdist_decode_split_kv",
              *_decode_args(q, k_cache, v_cache, out_split, lse_split, scale, soft_cap, block_table, kv_lens, num_splits),
              _lib.stream_ptr())
    return out_split, lse_split, kv_lens


_fused_counters = {}   # (device index, stream handle) -> zero-initialised int32 counters (the kernel leaves them zero)


def _counters_for(q, kv_heads, counters):
    """Arrival counters of the fused launch. ``counters`` (an explicit opt-in of this module's own callers: the layer,
    the tests): a contiguous int32 device tensor of at least tdist_decode_fused_counters(...) entries that is ALL ZERO
    and shared with no launch that may overlap this one; the kernel leaves it zero. None: a zeroed buffer cached per
    (device, current stream): launches on one stream are ordered, so they may share it, and launches on different
    streams never do."""
    batch, q_heads, _ = q.shape
    need = _lib.load().tdist_decode_fused_counters(batch, q_heads, kv_heads)
    if counters is not None:
        if not (isinstance(counters, torch.Tensor) and counters.is_cuda and counters.dtype == torch.int32
                and counters.is_contiguous() and counters.numel() >= need):
            raise ValueError("counters: a contiguous int32 device tensor of at least %d zeroed entries" % need)
        return counters, counters.numel()
    key = (q.device.index, torch.cuda.current_stream(q.device).cuda_stream)
    buf = _fused_counters.get(key)
    if buf is None or buf.numel() < need:
        buf = torch.zeros(max(int(need), 4096), dtype=torch.int32, device=q.device)
        _fused_counters[key] = buf
    return buf, buf.numel()


def decode_fused(q, k_cache, v_cache, kv_lens, block_table, scale, soft_cap, num_splits, out, lse_out=None,
                 workspace=None, out_split=None, lse_split=None):
    """tdist_decode_fused: split-KV decode and the merge of the splits in one launch. ``out`` [B,Hq,Dv]
    (bf16 / f16 / fp32), ``lse_out`` fp32 [B,Hq] or None. ``workspace``: None, or zeroed arrival counters of the
    caller's own (see _counters_for; anything else is an error). Returns (out, out_split, lse_split)."""
    kv_lens, block_table = _check_inputs(q, k_cache, v_cache, kv_lens, block_table)
    out_split, lse_split = _split_buffers(q, v_cache, num_splits, out_split, lse_split)
    assert out.stride(-1) == 1 and (lse_out is None or (lse_out.dtype == torch.float32 and lse_out.is_contiguous()))
    counters, n_counters = _counters_for(q, k_cache.shape[2], workspace)
    _lib.call("tdist_decode_fused",
              *_decode_args(q, k_cache, v_cache, out_split, lse_split, scale, soft_cap, block_table, kv_lens, num_splits),
              counters.data_ptr(), n_counters, out.data_ptr(), _lib.dtype_code(out.dtype), out.stride(0), out.stride(1),
              _lib.ptr(lse_out), _lib.stream_ptr())
    return out, out_split, lse_split


def decode_combine(part, lse, num_partials, mode, lens, batch, q_heads, dv, part_strides, lse_strides, out,
                   lse_out=None):
    """tdist_decode_combine with explicit element strides (p, b, h) for ``part`` and ``lse``."""
    _lib.call("tdist_decode_combine", part.data_ptr(), _lib.dtype_code(part.dtype), lse.data_ptr(), num_partials, mode,
              _lib.ptr(lens), batch, q_heads, dv, part_strides[0], part_strides[1], part_strides[2], lse_strides[0],
              lse_strides[1], lse_strides[2], out.data_ptr(), _lib.dtype_code(out.dtype), out.stride(0), out.stride(1),
              _lib.ptr(lse_out), _lib.stream_ptr())
    return out


def gqa_fwd_batch_decode(q, k_cache, v_cache, workspace, q_lens, kv_lens, block_table, scale, soft_cap=0.0,
                         output_split=None, output_combine=None, kv_split=-1):
    """Decode attention of one query token per sequence over a paged KV cache (reference :763-844).

    q [B,Hq,D]; k_cache / v_cache [num_pages, page_size, Hkv, D]; kv_lens int32[B]; block_table int32
    [B, max_pages]. ``workspace`` and ``q_lens`` are accepted and unused, as in the reference.
    ``output_split`` is ignored (partials are fp32 internally). Returns ``output_combine`` [B,Hq,Dv]
    (default dtype: q's; the reference hard-codes float16, :784)."""
    num_splits = DEFAULT_KV_SPLITS if kv_split == -1 else kv_split
    out_split, lse_split, kv_lens = _split_kv(q, k_cache, v_cache, kv_lens, block_table, scale, soft_cap, num_splits)
    batch, q_heads, _ = q.shape
    dv = v_cache.shape[-1]
    if output_combine is None:
        output_combine = torch.empty((batch, q_heads, dv), dtype=q.dtype, device=q.device)
    assert output_combine.stride(-1) == 1
    decode_combine(out_split, lse_split, num_splits, 1, kv_lens, batch, q_heads, dv,
                   (out_split.stride(2), out_split.stride(0), out_split.stride(1)),
                   (lse_split.stride(2), lse_split.stride(0), lse_split.stride(1)), output_combine)
    return output_combine


def gqa_fwd_batch_decode_persistent(q, k_cache, v_cache, workspace, q_lens, kv_lens, block_table, scale, soft_cap=0.0,
                                    output_split=None, output_combine=None, kv_split=-1):
    """Same result as gqa_fwd_batch_decode in one launch (reference :931-1004: split-KV, a grid barrier on
    ``workspace``, then the combine). Here the last workgroup to finish a (sequence, head block) merges its splits.
    ``workspace`` (the reference's barrier buffer) and ``q_lens`` are accepted and unused: nothing says what a
    caller's buffer holds or who else uses it, and a counter that does not start at zero makes a merge fire early or
    never, so the arrival counters are the library's own (zeroed, cached per device and stream, left zero by every
    call). ``output_split`` is ignored (partials are fp32 internally)."""
    num_splits = DEFAULT_KV_SPLITS if kv_split == -1 else kv_split
    batch, q_heads, _ = q.shape
    if output_combine is None:
        output_combine = torch.empty((batch, q_heads, v_cache.shape[-1]), dtype=q.dtype, device=q.device)
    decode_fused(q, k_cache, v_cache, kv_lens, block_table, scale, soft_cap, num_splits, output_combine)
    return output_combine


def gqa_fwd_batch_decode_intra_rank(q, k_cache, v_cache, workspace, q_lens, kv_lens, block_table, scale, soft_cap=0.0,
                                    output_split=None, output_combine=None, kv_split=-1, return_lse=False, counters=None):
    """One rank's KV shard: split-KV decode, then the merge of its splits keeping the LSE (reference
    :847-928). Returns ``output_combine`` [B,Hq,Dv+1] with the LSE in column Dv, fp32 unless the caller
    passes a buffer of another dtype (the reference uses q's dtype). With ``return_lse`` also returns the
    fp32 (out [B,Hq,Dv], lse [B,Hq]) pair the merge produced. ``workspace`` and ``q_lens`` are accepted and unused, as
    in the reference; ``counters`` (keyword only in spirit: an addition) hands in zeroed arrival counters of the
    caller's own, see _counters_for."""
    num_splits = DEFAULT_KV_SPLITS if kv_split == -1 else kv_split
    batch, q_heads, _ = q.shape
    dv = v_cache.shape[-1]
    if output_combine is None:
        output_combine = torch.empty((batch, q_heads, dv + 1), dtype=torch.float32, device=q.device)
    out32 = torch.empty((batch, q_heads, dv), dtype=torch.float32, device=q.device)
    lse32 = torch.empty((batch, q_heads), dtype=torch.float32, device=q.device)
    # split-KV and the merge of the splits (keeping the LSE) in one launch
    decode_fused(q, k_cache, v_cache, kv_lens, block_table, scale, soft_cap, num_splits, out32, lse32,
                 workspace=counters)
    output_combine[..., :dv].copy_(out32)
    output_combine[..., dv].copy_(lse32)
    if return_lse:
        return output_combine, out32, lse32
    return output_combine


def gqa_fwd_batch_decode_inter_rank_combine(all_ranks_out, all_ranks_lse, global_kv_lens, final_output=None,
                                            out_dtype=None):
    """Merge of the ranks' partial results by LSE (reference kernel :481-532, call shape
    layers/nvidia/sp_flash_decode_layer.py:172-182): all_ranks_out [R,B,Hq,Dv] (fp32 / bf16 / f16),
    all_ranks_lse fp32 [R,B,Hq], global_kv_lens int32 [R,B] (a rank whose length is 0 is skipped,
    :513-515). Returns [B,Hq,Dv]."""
    _lib.require_cuda(all_ranks_out, all_ranks_lse, global_kv_lens)
    R, B, Hq, dv = all_ranks_out.shape
    assert all_ranks_lse.shape == (R, B, Hq) and all_ranks_lse.dtype == torch.float32
    assert all_ranks_out.stride(-1) == 1
    if global_kv_lens.dtype != torch.int32:
        global_kv_lens = global_kv_lens.to(torch.int32)
    global_kv_lens = global_kv_lens.contiguous()
    assert global_kv_lens.shape == (R, B)
    if final_output is None:
        final_output = torch.empty((B, Hq, dv), dtype=out_dtype or all_ranks_out.dtype, device=all_ranks_out.device)
    decode_combine(all_ranks_out, all_ranks_lse, R, 2, global_kv_lens, B, Hq, dv,
                   (all_ranks_out.stride(0), all_ranks_out.stride(1), all_ranks_out.stride(2)),
                   (all_ranks_lse.stride(0), all_ranks_lse.stride(1), all_ranks_lse.stride(2)), final_output)
    return final_output
