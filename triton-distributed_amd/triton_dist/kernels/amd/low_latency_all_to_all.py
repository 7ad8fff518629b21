"""Low-latency MoE dispatch / combine on one MI355X.

Keeps the interface of the reference's kernels/nvidia/low_latency_all_to_all.py (``AllToAllContext``
:125-164, ``create_all_to_all_context`` :167-186, ``fast_all_to_all`` :189-248,
``all_to_all_post_process`` :251-270) and moves the index preprocessing the reference does in its test
(test/nvidia/test_all_to_all.py:42-96,314-329) onto the GPU as ``moe_dispatch_preprocess``.

One GPU stands for the sender ``rank`` and keeps, for every destination d, the slot this sender would
fill in d's receive buffer: rows of destination d (experts d*E_r .. d*E_r+E_r-1) are contiguous in the
expert-sorted order and land in ``recv[d*max_m : d*max_m + n_d]`` — the reference's
``recv[rank*MAX_M + i]`` on destination d (:63-86), stored side by side. The NVSHMEM puts become 16-byte
vector copies; there is no signal to wait for.
"""
from typing import Optional

import torch

from triton_dist import _lib


def dtype_size_in_bytes(dtype: torch.dtype) -> int:
    return torch.tensor([], dtype=dtype).element_size()


class AllToAllContext:

    def __init__(
        self,
        max_m: int,
        hidden: int,
        rank: int,
        num_tot_experts: int,
        WORLD_SIZE: int,
        experts_per_rank: int,
        dtype=torch.bfloat16,
        scale_dtype=torch.float,
        fp8_group_size: int = 0,
    ):
        """
        max_m: capacity, in rows, of one destination slot
        fp8_group_size: 0 = one scale per row (the reference's layout, :143); 128 = one scale per group of 128
            columns, [rows, hidden/128], the layout of the reference's tutorial 04 (its NUM_GROUPS, :138,175)
        """
        if not torch.cuda.is_available():
            raise RuntimeError("AllToAllContext needs a GPU")
        if scale_dtype != torch.float:
            raise NotImplementedError("scales are fp32")
        if num_tot_experts != WORLD_SIZE * experts_per_rank:
            raise ValueError("num_tot_experts must equal WORLD_SIZE * experts_per_rank")
        _lib.check(_lib.load().tdist_init())
        device = torch.device("cuda", torch.cuda.current_device())
        # double-buffered like the reference (:141-147): a call fills half call_count % 2
        self.recv_buf = torch.empty([WORLD_SIZE * max_m * 2, hidden], dtype=dtype, device=device)
        if fp8_group_size:
            if dtype != torch.float8_e4m3fn or hidden % fp8_group_size != 0:
                raise ValueError("group scales need e4m3 rows and a hidden size that is a multiple of the group size")
            self.scale_recv_buf = torch.empty([WORLD_SIZE * max_m * 2, hidden // fp8_group_size], dtype=scale_dtype,
                                              device=device)
        else:
            self.scale_recv_buf = torch.empty([WORLD_SIZE * max_m * 2], dtype=scale_dtype, device=device)
        self.fp8_group_size = fp8_group_size
        self.split_recv_buf = torch.zeros([num_tot_experts * 2], dtype=torch.int32, device=device)
        self.signal_buf = torch.zeros([WORLD_SIZE * 2], dtype=torch.int64, device=device)

        self.max_m = max_m
        self.hidden = hidden
        self.dtype = dtype
        self.scale_dtype = scale_dtype
        self.ele_size = dtype_size_in_bytes(self.dtype)
        self.scale_ele_size = dtype_size_in_bytes(self.scale_dtype)

        self.num_tot_experts = num_tot_experts
        self.experts_per_rank = experts_per_rank

        self.WORLD_SIZE = WORLD_SIZE
        self.rank = rank

        # start from 1, as the reference does (:161-163)
        self.call_count = 1
        self.MOD_VALUE = 1000000
        # index tensors of moe_dispatch_preprocess(..., ctx=self): two sets, allocated on first use for a shape
        self.index_sets, self.index_key, self.index_calls = None, None, 0
        self.index_workspace, self.index_args, self.index_ids = None, None, None
        self.last_index = None   # (splits, split_cumsum, scatter_idx, gather_idx) of the last fast_all_to_all(expert_ids=)


def create_all_to_all_context(
    max_m: int,
    hidden: int,
    rank: int,
    num_tot_experts: int,
    WORLD_SIZE: int,
    experts_per_rank: int,
    dtype=torch.bfloat16,
    scale_dtype=torch.float,
    fp8_group_size: int = 0,
):
    return AllToAllContext(max_m, hidden, rank, num_tot_experts, WORLD_SIZE, experts_per_rank, dtype, scale_dtype,
                           fp8_group_size)


def quant_bf16_fp8(tensor: torch.Tensor, gsize: int = 128):
    """bf16 [m, N] → (e4m3 [m, N], fp32 scales [m, N // gsize]) in groups of ``gsize`` columns: scale = max|x| / 448,
    q = e4m3(x / scale) (reference tutorials/04-deepseek-infer-all2all.py:309-360; that one returns the e4m3 bytes
    packed two to a bf16 element)."""
    _lib.require_cuda(tensor)
    if tensor.dtype != torch.bfloat16:
        raise TypeError("quant_bf16_fp8 takes bf16")
    tensor = tensor.contiguous()
    m, N = tensor.shape
    out = torch.empty((m, N), dtype=torch.float8_e4m3fn, device=tensor.device)
    out_scale = torch.empty((m, N // gsize), dtype=torch.float32, device=tensor.device)
    _lib.call("tdist_quant_e4m3_groups", tensor.data_ptr(), m, N, gsize, out.data_ptr(), out_scale.data_ptr(),
              _lib.stream_ptr())
    return out, out_scale


def splits_to_cumsum(splits: torch.Tensor):
    """[G] -> [G+1] with out[0] = 0 (reference test helper, test/nvidia/test_all_to_all.py:42-46)."""
    out = torch.empty(splits.shape[0] + 1, dtype=splits.dtype, device=splits.device)
    out[0] = 0
    _ = torch.cumsum(splits, 0, out=out[1:])
    return out


def _ensure_index_sets(ctx, T, topk, num_experts, dev):
    """The context's own index tensors for a (T, topk, num_experts) shape: two sets of (splits, cumsum, scatter_idx,
    gather_idx, topk_idx) used in turn, a zeroed workspace and an int32 staging tensor for ids of another dtype,
    allocated when the shape is first seen (the calls of one context are ordered on its stream, so they may share
    them)."""
    if ctx.index_key == (T, topk, num_experts, dev):
        return
    n = T * topk

    def alloc():
        return (torch.empty(num_experts, dtype=torch.int32, device=dev),
                torch.empty(num_experts + 1, dtype=torch.int32, device=dev),
                torch.empty((T, topk), dtype=torch.int32, device=dev),
                torch.empty(n, dtype=torch.int32, device=dev),
                torch.empty(n, dtype=torch.int32, device=dev))

    ws_bytes = _lib.load().tdist_moe_workspace_bytes(n, num_experts)
    ctx.index_sets, ctx.index_key, ctx.index_calls = [alloc(), alloc()], (T, topk, num_experts, dev), 0
    ctx.index_workspace = torch.zeros(ws_bytes, dtype=torch.uint8, device=dev)
    ctx.index_ids = torch.empty((T, topk), dtype=torch.int32, device=dev)
    ctx.index_args = [((n, topk, num_experts, t[0].data_ptr(), t[1].data_ptr(), t[2].data_ptr(), t[3].data_ptr()),
                       (ctx.index_workspace.data_ptr(), ws_bytes)) for t in ctx.index_sets]


def _staged_ids(ctx, exp_indices):
    """Ids as contiguous int32: as they are, or converted into the context's staging tensor (torch.topk gives int64):
    one copy kernel, no allocation."""
    if exp_indices.dtype != torch.int32 or not exp_indices.is_contiguous():
        ctx.index_ids.copy_(exp_indices)
        return ctx.index_ids
    return exp_indices


def moe_dispatch_preprocess(exp_indices: torch.Tensor, num_experts: int, want_topk_index: bool = False,
                            ctx: Optional[AllToAllContext] = None):
    """GPU version of the reference test's index preparation (test/nvidia/test_all_to_all.py:314-320):

        splits       int32[G]        torch.bincount(exp_indices.view(-1), minlength=G)
        split_cumsum int32[G+1]      splits_to_cumsum(splits)
        scatter_idx  int32[T, topk]  exp_indices.flatten().argsort(stable=True).argsort()
        gather_idx   int32[T*topk]   token of each expert-sorted row (calc_gather_index)

    One kernel launch. With ``ctx`` the five tensors are the context's own (allocated on the first call for a shape,
    two sets used in turn like the receive buffers, so a result stays valid until the call after next) and the call
    allocates nothing. Returns (splits, split_cumsum, scatter_idx, gather_idx[, topk_idx])."""
    _lib.require_cuda(exp_indices)
    T, topk = exp_indices.shape
    n = T * topk
    dev = exp_indices.device

    def alloc():
        return (torch.empty(num_experts, dtype=torch.int32, device=dev),
                torch.empty(num_experts + 1, dtype=torch.int32, device=dev),
                torch.empty((T, topk), dtype=torch.int32, device=dev),
                torch.empty(n, dtype=torch.int32, device=dev),
                torch.empty(n, dtype=torch.int32, device=dev))

    if ctx is not None:
        _ensure_index_sets(ctx, T, topk, num_experts, dev)
        # the context has seen this shape: its tensors' addresses are at hand and the host does next to nothing (the
        # index kernel takes ~9 us on the device; a general path costs more than that on the host). Ids that are not
        # contiguous int32 (torch.topk gives int64) are converted into the context's staging tensor: one copy kernel,
        # no allocation.
        exp_indices = _staged_ids(ctx, exp_indices)
        which = ctx.index_calls % 2
        ctx.index_calls += 1
        out = ctx.index_sets[which]
        head, tail = ctx.index_args[which]
        _lib.call("tdist_moe_scatter_index", exp_indices.data_ptr(), *head, _lib.ptr(out[4] if want_topk_index else None),
                  *tail, _lib.stream_ptr())
        return out if want_topk_index else out[:4]
    if exp_indices.dtype != torch.int32:
        exp_indices = exp_indices.to(torch.int32)
    exp_indices = exp_indices.contiguous()
    ws_bytes = _lib.load().tdist_moe_workspace_bytes(n, num_experts)
    splits, cumsum, scatter_idx, gather_idx, topk_idx = alloc()
    workspace = _lib.zeroed_scratch(ws_bytes, dev)
    if not want_topk_index:
        topk_idx = None
    _lib.call("tdist_moe_scatter_index", exp_indices.data_ptr(), n, topk, num_experts, splits.data_ptr(),
              cumsum.data_ptr(), scatter_idx.data_ptr(), gather_idx.data_ptr(), _lib.ptr(topk_idx),
              workspace.data_ptr(), workspace.numel(), _lib.stream_ptr())
    if want_topk_index:
        return splits, cumsum, scatter_idx, gather_idx, topk_idx
    return splits, cumsum, scatter_idx, gather_idx


def fast_all_to_all(
    ctx: AllToAllContext,
    send_tensor: torch.Tensor,
    send_split_cumsum: torch.Tensor,
    send_scale: Optional[torch.Tensor],
    gather_index: Optional[torch.Tensor] = None,
    scatter_index: Optional[torch.Tensor] = None,
    online_quant_fp8: bool = False,
    expert_ids: Optional[torch.Tensor] = None,
):
    """
    low-latency all-to-all communication (reference :189-248).

    send_tensor [n, hidden] rows already sorted by expert, send_split_cumsum int32[G+1], send_scale fp32[n]
    or None. With ``gather_index`` (int32[n_sorted], an addition) ``send_tensor`` is the unsorted
    [T, hidden] token tensor (``send_scale`` per token) and sorted row p is read from token
    gather_index[p], which fuses the reference's index_select (test_all_to_all.py:328-329) into the copy.
    With ``scatter_index`` (int32[T, topk], an addition) the same fusion runs token-major: every token row is
    read once and written to its topk slot rows, which is the faster form.

    With ``online_quant_fp8`` (the reference's tutorial 04, ONLINE_QUANT_FP8 :180-200; needs ``scatter_index`` and a
    context made with ``fp8_group_size=128``) ``send_tensor`` is the unsorted bf16 [T, hidden] token tensor: every
    row is quantised to e4m3 in groups of 128 columns while it is dispatched, ``send_scale`` must be None and the
    scales returned are [W*max_m, hidden/128].

    With ``expert_ids`` ([T, topk] integer tensor, an addition; ``send_split_cumsum`` may then be None) the call starts
    from the router's raw expert ids: for up to 65536 of them the index build (moe_dispatch_preprocess) runs inside the
    dispatch's one launch, beyond that in a launch of its own in front of it. ``send_tensor`` is the unsorted
    [T, hidden] token tensor. The index tensors land in the context's own (two sets in turn, as the receive buffers)
    and are kept as ``ctx.last_index`` = (splits, split_cumsum, scatter_idx, gather_idx) for the combine.

    Returns [splits int32[G], recv [W*max_m, hidden], scales [W*max_m] | None] — views into the context's
    buffers, valid until the call after next.
    """
    _lib.require_cuda(send_tensor, send_split_cumsum, send_scale, gather_index, scatter_index, expert_ids)
    if expert_ids is not None:
        if online_quant_fp8 or gather_index is not None or scatter_index is not None:
            raise ValueError("expert_ids replaces gather_index / scatter_index and does not combine with online_quant_fp8")
        return _fast_all_to_all_from_ids(ctx, send_tensor, send_scale, expert_ids)
    if online_quant_fp8:
        return _fast_all_to_all_online_quant(ctx, send_tensor, send_split_cumsum, send_scale, scatter_index)
    if ctx.fp8_group_size:
        raise ValueError("a context with group scales takes its rows through online_quant_fp8=True")
    with_scale = send_scale is not None
    act_pos = ctx.call_count % 2

    split_buf_st = act_pos * ctx.num_tot_experts
    split_buf_ed = split_buf_st + ctx.num_tot_experts
    data_buf_st = act_pos * ctx.WORLD_SIZE * ctx.max_m
    data_buf_ed = data_buf_st + ctx.WORLD_SIZE * ctx.max_m

    assert send_tensor.dim() == 2 and send_tensor.shape[1] == ctx.hidden
    assert send_tensor.dtype == ctx.dtype, "send_tensor dtype differs from the context's"
    assert send_split_cumsum.dtype == torch.int32 and send_split_cumsum.numel() == ctx.num_tot_experts + 1
    send_tensor = send_tensor.contiguous()
    if gather_index is not None:
        assert gather_index.dtype == torch.int32
        n_rows = gather_index.numel()
    else:
        n_rows = send_tensor.shape[0]
    if with_scale:
        assert send_scale.dtype == torch.float32
        send_scale = send_scale.contiguous()

    recv = ctx.recv_buf[data_buf_st:data_buf_ed, :]
    scale_recv = ctx.scale_recv_buf[data_buf_st:data_buf_ed]
    splits = ctx.split_recv_buf[split_buf_st:split_buf_ed]
    if scatter_index is not None:
        assert scatter_index.dtype == torch.int32 and scatter_index.is_contiguous()
        assert scatter_index.shape[0] == send_tensor.shape[0]
        _lib.call("tdist_moe_dispatch_tokens", send_tensor.data_ptr(), ctx.hidden * ctx.ele_size, _lib.ptr(send_scale),
                  scatter_index.data_ptr(), scatter_index.shape[1], send_split_cumsum.data_ptr(), send_tensor.shape[0],
                  ctx.WORLD_SIZE, ctx.experts_per_rank, ctx.max_m, recv.data_ptr(),
                  scale_recv.data_ptr() if with_scale else None, splits.data_ptr(), _lib.stream_ptr())
    else:
        _lib.call("tdist_moe_dispatch", send_tensor.data_ptr(), ctx.hidden * ctx.ele_size, _lib.ptr(send_scale),
                  _lib.ptr(gather_index), send_split_cumsum.data_ptr(), n_rows, ctx.WORLD_SIZE, ctx.experts_per_rank,
                  ctx.max_m, recv.data_ptr(), scale_recv.data_ptr() if with_scale else None, splits.data_ptr(),
                  _lib.stream_ptr())

    ctx.call_count = (ctx.call_count + 1) % ctx.MOD_VALUE
    out_lis = [splits, recv]
    out_lis.append(scale_recv if with_scale else None)
    return out_lis


FUSED_INDEX_MAX_IDS = 65536   # tdist_moe_dispatch_tokens_from_ids takes up to this many ids


def _fast_all_to_all_from_ids(ctx, send_tensor, send_scale, expert_ids):
    if ctx.fp8_group_size:
        raise ValueError("a context with group scales takes its rows through online_quant_fp8=True")
    assert send_tensor.dim() == 2 and send_tensor.shape[1] == ctx.hidden and send_tensor.dtype == ctx.dtype
    T, topk = expert_ids.shape
    assert T == send_tensor.shape[0]
    G = ctx.num_tot_experts
    row_bytes = ctx.hidden * ctx.ele_size
    windows = -(-row_bytes // 8192)
    fused = (T * topk <= FUSED_INDEX_MAX_IDS and windows in (1, 2, 4, 8, 16) and topk <= 64
             and (4 * G + 16 * topk + 8) * 4 <= 160 * 1024 - 256)
    if not fused:
        splits_i, cumsum, scatter, gather = moe_dispatch_preprocess(expert_ids, G, ctx=ctx)
        ctx.last_index = (splits_i, cumsum, scatter, gather)
        return fast_all_to_all(ctx, send_tensor, cumsum, send_scale, scatter_index=scatter)
    _ensure_index_sets(ctx, T, topk, G, send_tensor.device)
    ids = _staged_ids(ctx, expert_ids)
    which = ctx.index_calls % 2
    ctx.index_calls += 1
    splits_i, cumsum, scatter, gather, _ = ctx.index_sets[which]
    send_tensor = send_tensor.contiguous()
    with_scale = send_scale is not None
    if with_scale:
        assert send_scale.dtype == torch.float32
        send_scale = send_scale.contiguous()
    act_pos = ctx.call_count % 2
    rows = ctx.WORLD_SIZE * ctx.max_m
    recv = ctx.recv_buf[act_pos * rows:(act_pos + 1) * rows, :]
    scale_recv = ctx.scale_recv_buf[act_pos * rows:(act_pos + 1) * rows]
    splits = ctx.split_recv_buf[act_pos * G:(act_pos + 1) * G]
    _lib.call("tdist_moe_dispatch_tokens_from_ids", send_tensor.data_ptr(), row_bytes, _lib.ptr(send_scale), ids.data_ptr(),
              topk, T, ctx.WORLD_SIZE, ctx.experts_per_rank, ctx.max_m, recv.data_ptr(),
              scale_recv.data_ptr() if with_scale else None, splits.data_ptr(), splits_i.data_ptr(), cumsum.data_ptr(),
              scatter.data_ptr(), gather.data_ptr(), _lib.stream_ptr())
    ctx.last_index = (splits_i, cumsum, scatter, gather)
    ctx.call_count = (ctx.call_count + 1) % ctx.MOD_VALUE
    return [splits, recv, scale_recv if with_scale else None]


def _fast_all_to_all_online_quant(ctx, send_tensor, send_split_cumsum, send_scale, scatter_index):
    if scatter_index is None or send_scale is not None:
        raise ValueError("online_quant_fp8 takes the unsorted bf16 tokens with scatter_index and no send_scale")
    if not ctx.fp8_group_size or ctx.dtype != torch.float8_e4m3fn:
        raise ValueError("online_quant_fp8 needs a context created with dtype=float8_e4m3fn, fp8_group_size=128")
    if send_tensor.dtype != torch.bfloat16:
        raise TypeError("online_quant_fp8 quantises bf16 tokens")
    assert send_tensor.dim() == 2 and send_tensor.shape[1] == ctx.hidden
    assert send_split_cumsum.dtype == torch.int32 and send_split_cumsum.numel() == ctx.num_tot_experts + 1
    assert scatter_index.dtype == torch.int32 and scatter_index.is_contiguous()
    assert scatter_index.shape[0] == send_tensor.shape[0]
    send_tensor = send_tensor.contiguous()
    act_pos = ctx.call_count % 2
    rows = ctx.WORLD_SIZE * ctx.max_m
    recv = ctx.recv_buf[act_pos * rows:(act_pos + 1) * rows, :]
    scale_recv = ctx.scale_recv_buf[act_pos * rows:(act_pos + 1) * rows, :]
    splits = ctx.split_recv_buf[act_pos * ctx.num_tot_experts:(act_pos + 1) * ctx.num_tot_experts]
    _lib.call("tdist_moe_dispatch_tokens_quant", send_tensor.data_ptr(), ctx.hidden, ctx.fp8_group_size,
              scatter_index.data_ptr(), scatter_index.shape[1], send_split_cumsum.data_ptr(), send_tensor.shape[0],
              ctx.WORLD_SIZE, ctx.experts_per_rank, ctx.max_m, recv.data_ptr(), scale_recv.data_ptr(), splits.data_ptr(),
              _lib.stream_ptr())
    ctx.call_count = (ctx.call_count + 1) % ctx.MOD_VALUE
    return [splits, recv, scale_recv]


def all_to_all_post_process(
    ctx: AllToAllContext,
    input_splits: torch.Tensor,
    recv_buffer: torch.Tensor,
    scale_buffer: Optional[torch.Tensor] = None,
):
    """Compacts the slots into one tensor in destination order (reference :251-270). The row count is read
    back from the device, as the reference's slicing by tensor values does."""
    _lib.require_cuda(input_splits, recv_buffer, scale_buffer)
    with_scale = scale_buffer is not None
    total = int(input_splits.sum().item())
    row_bytes = recv_buffer.shape[1] * recv_buffer.element_size()
    output = torch.empty((total, recv_buffer.shape[1]), dtype=recv_buffer.dtype, device=recv_buffer.device)
    output_scale = torch.empty((total, ), dtype=scale_buffer.dtype, device=recv_buffer.device) if with_scale else None
    if total > 0:
        _lib.call("tdist_moe_post_process", recv_buffer.data_ptr(), row_bytes, _lib.ptr(scale_buffer),
                  input_splits.data_ptr(), total, ctx.WORLD_SIZE, ctx.experts_per_rank, ctx.max_m, output.data_ptr(),
                  _lib.ptr(output_scale), _lib.stream_ptr())
    return output, output_scale


def moe_weighted_combine(ctx: Optional[AllToAllContext], rows: torch.Tensor, row_scale: Optional[torch.Tensor],
                         scatter_idx: torch.Tensor, topk_weight: Optional[torch.Tensor],
                         split_cumsum: Optional[torch.Tensor] = None, from_slots: bool = True):
    """y[t] = sum_k w[t,k] * scale[p] * rows[p], p = scatter_idx[t,k]: fp32 accumulation in k order, bf16
    output [T, hidden]. Restates the reduce step of the reference test
    (``index_add_(0, gather_idx, combine_token)``, test/nvidia/test_all_to_all.py:366-367) with the top-k
    weighting of TorchGroupGemmReduceRS (test/nvidia/test_moe_reduce_rs.py:117-122).

    ``rows`` is the slot layout returned by fast_all_to_all (from_slots=True, needs ``ctx`` and
    ``split_cumsum``) or a compact expert-sorted [n, hidden] tensor (from_slots=False)."""
    _lib.require_cuda(rows, row_scale, scatter_idx, topk_weight, split_cumsum)
    T, topk = scatter_idx.shape
    hidden = rows.shape[1]
    assert scatter_idx.dtype == torch.int32 and scatter_idx.is_contiguous()
    if topk_weight is not None:
        assert topk_weight.dtype == torch.float32 and topk_weight.is_contiguous() and topk_weight.shape == (T, topk)
    if rows.dtype == torch.float8_e4m3fn:
        code = _lib.TDIST_F8E4M3
    elif rows.dtype == torch.bfloat16:
        code = _lib.TDIST_BF16
    else:
        raise TypeError("combine takes e4m3 or bf16 rows, got %s" % rows.dtype)
    out = torch.empty((T, hidden), dtype=torch.bfloat16, device=rows.device)
    if from_slots:
        assert ctx is not None and split_cumsum is not None
        W, Er, max_m = ctx.WORLD_SIZE, ctx.experts_per_rank, ctx.max_m
    else:
        W, Er, max_m = 1, 1, 0
    scale_group = 0
    if row_scale is not None and row_scale.dim() == 2:   # one scale per group of columns
        assert row_scale.is_contiguous() and hidden % row_scale.shape[1] == 0
        scale_group = hidden // row_scale.shape[1]
    _lib.call("tdist_moe_combine", rows.data_ptr(), code, _lib.ptr(row_scale), scatter_idx.data_ptr(),
              _lib.ptr(topk_weight), _lib.ptr(split_cumsum), T, topk, hidden, W, Er, max_m, scale_group, out.data_ptr(),
              _lib.stream_ptr())
    return out
