"""AG-GEMM on one MI355X: the consumer GEMM gated per chunk on HBM flag words, with the all-gather's
arrivals played by copy streams of the same GPU.

Keeps the interface of the reference's kernels/amd/all_gather_gemm.py
(``create_ag_gemm_intra_node_context`` :360-429, ``ag_gemm_intra_node`` :432-464, context dataclass
:327-357). What differs is where the peers' rows come from: with one GPU there is no IPC workspace a peer
pushes into, so the shards of the other ranks are handed to the context (``ctx.set_peer_shards``) and the
producer copies them chunk by chunk into the workspace and then releases the chunk's flag, exactly the
per-chunk protocol of the reference's copy-engine producer (:41-100). The GEMM reads the caller's own
shard directly and never waits for it (:201-218).
"""
import dataclasses
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from triton_dist import _lib
from triton_dist.kernels.amd.common_ops import fill_flags


def cp_engine_producer_all_gather_full_mesh_push_multi_stream(
    rank,
    num_ranks,
    peer_shards: Dict[int, torch.Tensor],
    workspace: torch.Tensor,
    one: torch.Tensor,
    M_PER_CHUNK: int,
    ag_stream_pool: List[torch.cuda.Stream],
    barrier: torch.Tensor,
    arrival_order: Optional[Sequence[Tuple[int, int]]] = None,
    held_chunks: Sequence[int] = (),
    use_sdma: bool = True,
    link_gbps: float = 0.0,
    start_stamp: Optional[torch.Tensor] = None,
):
    """Delivers the peers' shards into ``workspace`` chunk by chunk: data copy, then a 4-byte copy of
    ``one`` into the chunk's flag on the same stream (reference :80-100). ``arrival_order`` is a list of
    (peer_rank, chunk_in_rank); the default is the reference's (:54-66): peers rank+1, rank+2, ... each
    on its own stream, chunks in order. Chunks listed in ``held_chunks`` (global chunk ids) are never
    delivered — a test hook for the bounded wait. With ``link_gbps`` > 0 every peer's n-th chunk is held back
    until n * chunk_bytes / link rate after ``start_stamp`` (a device time stamp taken when the op started): the
    pace at which a peer's copy engine would deliver it over one xGMI link."""
    some = next(iter(peer_shards.values()))
    M_per_rank, K = some.shape
    chunk_num_per_rank = M_per_rank // M_PER_CHUNK
    esz = some.element_size()
    nbytes = M_PER_CHUNK * K * esz
    if arrival_order is None:
        arrival_order = []
        for idx in range(1, num_ranks):
            r = (rank + idx) % num_ranks
            arrival_order += [(r, c) for c in range(chunk_num_per_rank)]
    held = set(int(c) for c in held_chunks)
    n_streams = len(ag_stream_pool)
    sent: Dict[int, int] = {}
    for r, c in arrival_order:
        if r == rank:
            continue
        chunk_pos = r * chunk_num_per_rank + c
        if chunk_pos in held:
            continue
        stream = ag_stream_pool[r % n_streams]
        src = peer_shards[r]
        src_ptr = src.data_ptr() + c * M_PER_CHUNK * K * esz
        dst_ptr = workspace.data_ptr() + (r * M_per_rank + c * M_PER_CHUNK) * K * esz
        flag_ptr = barrier.data_ptr() + chunk_pos * 4
        if link_gbps > 0:
            sent[r] = sent.get(r, 0) + 1
            _lib.call("tdist_producer_wait_until", start_stamp.data_ptr(), int(sent[r] * nbytes / link_gbps),
                      stream.cuda_stream)
        _lib.call("tdist_producer_push_chunk", dst_ptr, src_ptr, nbytes, flag_ptr, one.data_ptr(),
                  1 if use_sdma else 0, stream.cuda_stream)


def kernel_producer_all_gather_push(rank, num_ranks, ctx, workspace, M_PER_CHUNK, stream, barrier):
    """The peers' pushes as ONE launch of tdist_producer_push_peers (a block row per peer, pacing inside the kernel):
    the same data-then-flag protocol as the copy-engine producer above with a single host call, and light enough
    on registers to share compute units with the GEMM."""
    some = next(iter(ctx.peer_shards.values()))
    M_per_rank, K = some.shape
    esz = some.element_size()
    n_chunks = num_ranks * (M_per_rank // M_PER_CHUNK)
    if ctx.arrival_order is not None:
        raise ValueError("the kernel producer delivers every peer's chunks in order; arrival_order needs the copy producer")
    if ctx.producer_counters is None or ctx.producer_counters.numel() < n_chunks:
        ctx.producer_counters = torch.zeros(n_chunks, dtype=torch.int32, device=some.device)
    held = None
    if ctx.held_chunks or ctx.late_chunks_us:
        key = (tuple(ctx.held_chunks), tuple(sorted(ctx.late_chunks_us.items())), n_chunks)
        if ctx.held_mask_key != key:
            held = torch.zeros(n_chunks, dtype=torch.int32)
            for c, us in ctx.late_chunks_us.items():
                held[int(c)] = -min(int(us), 100000)
            held[list(int(c) for c in ctx.held_chunks)] = 1
            ctx.held_mask, ctx.held_mask_key = held.to(some.device), key
        held = ctx.held_mask
    else:
        ctx.held_mask, ctx.held_mask_key = None, None
    paced = ctx.link_gbps > 0
    nbytes = M_PER_CHUNK * K * esz
    # race provocation: a new seed per call, so every call sees another pattern of late chunks
    delay_ns = int(ctx.random_delay_us * 1000)
    if delay_ns > 0:
        ctx.delay_calls += 1
    seed = (ctx.delay_seed * 0x9E3779B1 + ctx.delay_calls) & 0xFFFFFFFF
    _lib.call("tdist_producer_push_peers", workspace.data_ptr(), ctx.peer_ptrs.data_ptr(), num_ranks, rank,
              M_per_rank * K * esz, nbytes, barrier.data_ptr(), 1, ctx.producer_counters.data_ptr(), _lib.ptr(held),
              ctx.start_stamp.data_ptr() if paced else None, int(nbytes / ctx.link_gbps) if paced else 0,
              seed, delay_ns, int(ctx.producer_workgroups), stream.cuda_stream)


@dataclasses.dataclass
class AllGatherGEMMTensorParallelContext:
    rank: int
    num_ranks: int
    workspace_tensors: List[Optional[torch.Tensor]]
    barrier_tensors: List[Optional[torch.Tensor]]
    comm_bufs: List[Optional[torch.Tensor]]
    one: torch.Tensor
    comm_buf_ptr: Optional[torch.Tensor]
    ag_streams: Optional[List[torch.cuda.streams.Stream]] = None
    gemm_stream: Optional[torch.cuda.streams.Stream] = None
    serial: bool = False
    M_PER_CHUNK: int = 1024
    BLOCK_M: int = 128
    BLOCK_N: int = 256
    BLOCK_K: int = 64
    stages: int = 3
    autotune: bool = False
    # ---- one-GPU additions -------------------------------------------------------------------
    output_dtype: torch.dtype = torch.bfloat16
    peer_shards: Dict[int, torch.Tensor] = dataclasses.field(default_factory=dict)
    arrival_order: Optional[List[Tuple[int, int]]] = None
    held_chunks: Tuple[int, ...] = ()
    spin_limit: int = 0          # 0 = library default (seconds of polling)
    # int32[4]: [0:2] error code and chunk of the current call's expired flag wait, [2:4] the first one of earlier
    # calls that nobody has looked at yet (every call retires its predecessor's, so a timeout slows down one launch)
    status: Optional[torch.Tensor] = None
    # True: chunk copies go to the copy engines (hipMemcpyDeviceToDeviceNoCU), as the reference's cp-engine
    # producer does across GPUs. On one GPU the engines move ~55 GB/s each, far below a kernel copy inside HBM, so
    # the default is the blit path.
    use_sdma: bool = False
    preset_flags: bool = False   # debug: release every flag before the GEMM starts (no overlap)
    # > 0: pace the arrivals like one xGMI link per peer (GB/s; a link of MI355X moves ~153): a peer's n-th chunk is
    # copied no earlier than n * chunk_bytes / rate after the op started. 0: chunks are copied as fast as this GPU can.
    link_gbps: float = 0.0
    start_stamp: Optional[torch.Tensor] = None   # int64[1], device wall-clock stamp of the current call
    # True: the peers' pushes are one launch of a small kernel (a block row per peer) instead of two async copies
    # per chunk on the copy streams. Its waves fit beside the GEMM's on a SIMD, so no compute units are set aside
    # (producer_cus is ignored) and the host queues three launches per call, however many chunks there are.
    producer_kernel: bool = False
    producer_workgroups: int = 8   # workgroups per peer of that kernel
    # > 0 (kernel producer only): about 7 of 10 chunks, chosen by a hash of (delay_seed, call number, chunk), are held
    # back by a pseudo-random time below this many microseconds before they are copied: the reference's race
    # provocation (its producer sleeps with probability 0.7 when run "for correctness",
    # kernels/nvidia/allgather.py:72-77,118-121), seeded so that a failing pattern can be replayed.
    random_delay_us: float = 0.0
    delay_seed: int = 0
    delay_calls: int = 0
    producer_counters: Optional[torch.Tensor] = None
    peer_ptrs: Optional[torch.Tensor] = None   # int64[num_ranks] device array of the peer shards' addresses
    held_mask: Optional[torch.Tensor] = None
    held_mask_key: Optional[tuple] = None
    # kernel producer only: global chunk id -> microseconds by which that chunk is copied late (a straggler: the same
    # peer's later chunks follow behind it)
    late_chunks_us: Dict[int, float] = dataclasses.field(default_factory=dict)
    # Compute units the gated GEMM leaves to the producer's copies. On one GPU those copies need compute
    # units of this GPU; measured on MI355X they make no progress next to a full-chip persistent grid
    # unless 32 units stay free. A peer's copy engine pushing over xGMI would need none.
    producer_cus: int = 32
    # The context's workspace for the GEMM (tdist_gemm_split_k_workspace_bytes() bytes, zero-filled once): with it a
    # last round of tiles that fills at most half of the grid is cut along K. It belongs to this context, so contexts
    # on different streams share no state. None: whole tiles only.
    sk_workspace: Optional[torch.Tensor] = None

    def update(self, rank, num_ranks, BLOCK_M=128, BLOCK_N=256, BLOCK_K=64, stages=3, ag_streams=None, gemm_stream=None,
               serial=False, autotune=False):
        self.rank = rank
        self.num_ranks = num_ranks
        self.BLOCK_M = BLOCK_M
        self.BLOCK_N = BLOCK_N
        self.BLOCK_K = BLOCK_K
        self.stages = stages
        self.ag_streams = ag_streams
        self.gemm_stream = gemm_stream
        self.serial = serial
        self.autotune = autotune

    def set_peer_shards(self, shards):
        """``shards``: dict rank -> [M_per_rank, K] tensor, or a list of num_ranks tensors (the entry of
        ``rank`` is ignored). They stand for the A shards living on the other ranks."""
        if not isinstance(shards, dict):
            shards = {r: t for r, t in enumerate(shards) if t is not None}
        for r, t in shards.items():
            if r == self.rank:
                continue
            _lib.require_cuda(t)
            if not t.is_contiguous():
                raise ValueError("peer shard of rank %d must be contiguous" % r)
        self.peer_shards = {r: t for r, t in shards.items() if r != self.rank}
        ptrs = [self.peer_shards[r].data_ptr() if r in self.peer_shards else 0 for r in range(self.num_ranks)]
        self.peer_ptrs = torch.tensor(ptrs, dtype=torch.int64).to(self.one.device)

    def check_status(self):
        """Synchronises and raises TdistError if a bounded flag wait expired in an earlier call (the earliest one
        since the last check)."""
        torch.cuda.synchronize()
        code, chunk, first_code, first_chunk = self.status.tolist()
        if first_code != 0:
            code, chunk = first_code, first_chunk
        if code != 0:
            self.status.zero_()
            raise _lib.TdistError(code, "flag wait expired for chunk %d" % chunk)


def create_ag_gemm_intra_node_context(max_M, N, K, input_dtype, output_dtype, rank, num_ranks, tp_group,
                                      ag_streams=None, gemm_stream=None, M_PER_CHUNK=1024, BLOCK_M=128, BLOCK_N=256,
                                      BLOCK_K=64, stages=3, serial=False, autotune=False, split_k=True,
                                      ragged_chunks=False):
    """create context for allgather gemm intra-node (reference :360-429).

    ``tp_group`` may be None: one GPU holds the only real rank. BLOCK_*/stages/autotune are accepted for
    signature compatibility; the HIP kernel picks its own tiling. ``split_k``: give the context a workspace
    (64 MiB) with which a last round of tiles that fills at most half of the grid is cut along K.
    ``ragged_chunks``: M_PER_CHUNK need not be a multiple of BLOCK_M (the reference asserts that it is, :375); a
    tile of the GEMM then waits for every chunk its rows touch, and the own shard goes through the workspace.
    """
    assert ragged_chunks or M_PER_CHUNK % BLOCK_M == 0
    assert max_M % num_ranks == 0
    M_per_rank = max_M // num_ranks
    assert M_per_rank % M_PER_CHUNK == 0
    if not torch.cuda.is_available():
        raise RuntimeError("create_ag_gemm_intra_node_context needs a GPU")
    _lib.check(_lib.load().tdist_init())
    device = torch.device("cuda", torch.cuda.current_device())
    sk_workspace = _lib.new_split_k_workspace(device) if split_k else None
    workspace = torch.empty([max_M, K], dtype=input_dtype, device=device)
    m_chunk_num = (max_M + M_PER_CHUNK - 1) // M_PER_CHUNK
    barrier = torch.zeros([m_chunk_num], dtype=torch.int32, device=device)
    workspaces: List[Optional[torch.Tensor]] = [None] * num_ranks
    barriers: List[Optional[torch.Tensor]] = [None] * num_ranks
    workspaces[rank] = workspace
    barriers[rank] = barrier

    current_stream = torch.cuda.current_stream()
    # default priority on purpose (the reference asks for priority -1)
    # two copy streams by default (the reference makes one per rank): with the GEMM stream that stays within the 4
    # hardware queues of a process, so no stream waits behind another one's packets
    _ag_streams = [torch.cuda.Stream() for _ in range(min(num_ranks, 2))] if ag_streams is None else ag_streams
    _gemm_stream = current_stream if gemm_stream is None else gemm_stream
    one = torch.ones((1024, ), dtype=torch.int32, device=device)
    status = torch.zeros((4, ), dtype=torch.int32, device=device)
    start_stamp = torch.zeros((1, ), dtype=torch.int64, device=device)
    torch.cuda.synchronize()

    return AllGatherGEMMTensorParallelContext(
        rank=rank,
        num_ranks=num_ranks,
        workspace_tensors=workspaces,
        barrier_tensors=barriers,
        comm_bufs=[None] * num_ranks,
        one=one,
        comm_buf_ptr=None,
        ag_streams=_ag_streams,
        gemm_stream=_gemm_stream,
        serial=serial,
        M_PER_CHUNK=M_PER_CHUNK,
        BLOCK_M=BLOCK_M,
        BLOCK_N=BLOCK_N,
        BLOCK_K=BLOCK_K,
        stages=stages,
        autotune=autotune,
        output_dtype=output_dtype,
        status=status,
        start_stamp=start_stamp,
        sk_workspace=sk_workspace,
    )


_GEMM_ENTRY = {
    torch.bfloat16: "tdist_gemm_chunk_gated_bf16",
    torch.float16: "tdist_gemm_chunk_gated_f16",
    torch.float8_e4m3fn: "tdist_gemm_chunk_gated_fp8e4m3",
}


def gated_gemm(a_ws, a_local, local_row_begin, b, c, flags, m_per_chunk, rank, num_ranks, *, row_scale=None,
               col_scale=None, chunk_order=None, wait_value=1, spin_limit=0, status=None, max_workgroups=0,
               sk_workspace=None, stream=None):
    """Thin wrapper over tdist_gemm_chunk_gated_*: C[M,N] = A[M,K] @ B[N,K]^T with per-chunk gating.
    ``a_ws`` [M,K] gathered rows, ``a_local`` own shard or None, ``b`` [N,K]. ``max_workgroups`` > 0 caps the
    persistent grid (leave compute units to a producer that copies on this same GPU). ``sk_workspace``: an optional
    zero-initialised uint8 tensor of tdist_gemm_split_k_workspace_bytes() bytes (_lib.new_split_k_workspace); launches
    that share one must be ordered."""
    _lib.require_cuda(a_ws, b, c)
    M, K = a_ws.shape
    N = b.shape[0]
    if a_ws.dtype not in _GEMM_ENTRY:
        raise TypeError("unsupported GEMM dtype %s" % a_ws.dtype)
    if a_ws.stride(1) != 1 or b.stride(1) != 1 or c.stride(1) != 1:
        raise ValueError("A, B and C must be row-major with a contiguous last dimension")
    args = [
        a_ws.data_ptr(), a_ws.stride(0),
        _lib.ptr(a_local), a_local.stride(0) if a_local is not None else 0,
        int(local_row_begin), a_local.shape[0] if a_local is not None else 0,
        b.data_ptr(), b.stride(0), c.data_ptr(), c.stride(0), M, N, K,
    ]
    if a_ws.dtype == torch.float8_e4m3fn:
        args += [_lib.ptr(row_scale), _lib.ptr(col_scale)]
    elif row_scale is not None or col_scale is not None:
        raise ValueError("scales are only defined for fp8 inputs")
    args += [
        _lib.ptr(flags), int(m_per_chunk), int(wait_value), _lib.ptr(chunk_order), int(rank), int(num_ranks),
        int(spin_limit), _lib.ptr(status), int(max_workgroups), *_lib.workspace_args(sk_workspace),
        _lib.stream_ptr(stream),
    ]
    _lib.call(_GEMM_ENTRY[a_ws.dtype], *args)
    return c


def ag_gemm_intra_node_op(a, b, c, rank, num_ranks, workspace_tensors, one, barrier_tensors, comm_buf_ptr, ag_streams,
                          gemm_stream, serial=False, M_PER_CHUNK=1024, BLOCK_M=128, BLOCK_N=256, BLOCK_K=64, stages=3,
                          autotune=False, use_persistent_gemm=True, *, ctx=None, row_scale=None, col_scale=None):
    """Reference :257-324: start the producer on the all-gather streams, then the gated GEMM on the GEMM
    stream; the caller's stream waits for the GEMM."""
    assert a.shape[1] == b.shape[1], "Incompatible dimensions"
    assert a.dtype == b.dtype, "Incompatible dtypes"
    if not use_persistent_gemm:
        raise NotImplementedError("Non-perisitent gemm is not yet supported")
    M_per_rank, K = a.shape
    M = M_per_rank * num_ranks
    workspace = workspace_tensors[rank]
    barrier = barrier_tensors[rank]
    peer_shards = ctx.peer_shards if ctx is not None else {}
    if num_ranks > 1:
        missing = [r for r in range(num_ranks) if r != rank and r not in peer_shards]
        if missing:
            raise RuntimeError(
                "one GPU holds a single rank: hand the other ranks' A shards to the context first "
                "(ctx.set_peer_shards); missing ranks %s" % missing)

    current_stream = torch.cuda.current_stream()
    paced = ctx is not None and ctx.link_gbps > 0 and num_ranks > 1
    if paced:
        _lib.call("tdist_producer_mark", ctx.start_stamp.data_ptr(), current_stream.cuda_stream)
    use_kernel = ctx is not None and ctx.producer_kernel
    # Fork: one event on the caller's stream, waited for by the GEMM stream and by the producer streams that this
    # call really uses (the kernel producer needs one; the copy producer stream r % n for every peer r). The host
    # cost of a call is what bounds the small shapes, so nothing is forked, joined or entered that is not used.
    if num_ranks <= 1:
        used_ag_streams = []
    elif use_kernel:
        used_ag_streams = [ag_streams[0]]
    else:
        used = sorted(set(r % len(ag_streams) for r in range(num_ranks) if r != rank))
        used_ag_streams = [ag_streams[i] for i in used]
    fork = current_stream.record_event()
    gemm_stream.wait_event(fork)
    for ag_stream in used_ag_streams:
        ag_stream.wait_event(fork)

    def call_ag():
        if num_ranks > 1 and use_kernel:
            kernel_producer_all_gather_push(rank, num_ranks, ctx, workspace, M_PER_CHUNK, ag_streams[0], barrier)
        elif num_ranks > 1:
            cp_engine_producer_all_gather_full_mesh_push_multi_stream(
                rank, num_ranks, peer_shards, workspace, one, M_PER_CHUNK, ag_streams, barrier,
                arrival_order=ctx.arrival_order if ctx is not None else None,
                held_chunks=ctx.held_chunks if ctx is not None else (),
                use_sdma=ctx.use_sdma if ctx is not None else True,
                link_gbps=ctx.link_gbps if paced else 0.0, start_stamp=ctx.start_stamp if paced else None)

    # Chunks that are not whole 128-row tiles: a tile may hold rows of the own shard and of a neighbour's, so the
    # own rows are copied into the workspace and released through their flags like everyone else's (what the
    # reference's producer does with every local shard, :268-272).
    local = a
    if M_PER_CHUNK % 128 != 0 or (rank * M_per_rank) % 128 != 0 or M_per_rank % 128 != 0:
        local = None

    def call_gemm(max_wgs):
        if ctx is not None:
            # the launch before may have given up on a flag: keep what it reported, start this one clean
            _lib.call("tdist_status_retire", ctx.status.data_ptr(), ctx.status.data_ptr() + 8, gemm_stream.cuda_stream)
        if local is None:
            if not a.is_contiguous():
                raise ValueError("the local shard must be contiguous")
            first, per_rank = rank * M_per_rank, M_per_rank // M_PER_CHUNK
            own_flags = barrier.data_ptr() + rank * per_rank * 4
            _lib.call("tdist_producer_push_chunk", workspace.data_ptr() + first * K * a.element_size(), a.data_ptr(),
                      a.numel() * a.element_size(), own_flags, one.data_ptr(), 0, gemm_stream.cuda_stream)
            if per_rank > 1:
                _lib.call("tdist_flag_fill", own_flags, per_rank, 1, gemm_stream.cuda_stream)
        # (the launch names its stream; nothing here runs on torch's current stream)
        gated_gemm(workspace[:M], local, rank * M_per_rank, b, c, barrier, M_PER_CHUNK, rank, num_ranks,
                   row_scale=row_scale, col_scale=col_scale, wait_value=1,
                   spin_limit=ctx.spin_limit if ctx is not None else 0,
                   status=ctx.status if ctx is not None else None, max_workgroups=max_wgs,
                   sk_workspace=ctx.sk_workspace if ctx is not None else None, stream=gemm_stream)

    if serial or (ctx is not None and ctx.preset_flags):
        # every chunk delivered before the GEMM starts
        call_ag()
        for ag_stream in used_ag_streams:
            gemm_stream.wait_stream(ag_stream)
        if serial:
            torch.cuda.synchronize()
        call_gemm(0)
    else:
        max_wgs = 0
        if ctx is not None and num_ranks > 1 and ctx.producer_cus > 0 and not use_kernel:
            max_wgs = max(1, _lib.load().tdist_num_cus() - ctx.producer_cus)
        # The reference's order (:300-304): producer first. (Queuing the GEMM first would let it start on the own
        # rows while the host still queues copies, but a copy that lands behind the spinning GEMM on a shared
        # hardware queue can never run, and which streams share a queue is not under the caller's control.)
        call_ag()
        call_gemm(max_wgs)
    current_stream.wait_stream(gemm_stream)
    for ag_stream in used_ag_streams:
        current_stream.wait_stream(ag_stream)
    # (c and the operands are used on gemm_stream by kernels queued before this join; the caller's stream owns them)
    return None


def ag_gemm_intra_node(a, b, transe_b, ctx, *, row_scale=None, col_scale=None):
    """allgather gemm for intra-node (reference :432-464)

    Allgather global matrix A and do matmul with local matrix B, produces local matrix C

    Args:
        a (torch.Tensor): local matmul A matrix. shape: [M_per_rank, K]
        b (torch.Tensor): local matmul B matrix. shape: [N_per_rank, K]
        transe_b (bool): indicates whether tensor b is transposed (not supported, as in the reference)
        ctx (AllGatherGEMMTensorParallelContext)
        row_scale / col_scale: fp8 inputs only — fp32 per-row scales of the gathered A ([M]) and per-column
            scales of B ([N_per_rank]); no counterpart in the reference.

    Returns:
        c (torch.Tensor): local matmul C matrix. shape: [M, N_per_rank]; a.dtype for 16-bit inputs,
        ctx.output_dtype (bf16) for fp8 inputs.
    """
    if ctx is None:
        raise RuntimeError("requires ctx for ipc handle")
    if transe_b:
        raise NotImplementedError("transpose weight is not yet supported")
    _lib.require_cuda(a, b)
    M_per_rank, K = a.shape
    N_per_rank = b.shape[0]
    out_dtype = a.dtype if a.dtype in (torch.bfloat16, torch.float16) else torch.bfloat16
    C = torch.empty([ctx.num_ranks * M_per_rank, N_per_rank], dtype=out_dtype, device=a.device)

    ag_gemm_intra_node_op(a, b, C, ctx.rank, ctx.num_ranks, ctx.workspace_tensors, ctx.one, ctx.barrier_tensors,
                          ctx.comm_buf_ptr, ag_streams=ctx.ag_streams, gemm_stream=ctx.gemm_stream, serial=ctx.serial,
                          M_PER_CHUNK=ctx.M_PER_CHUNK, autotune=ctx.autotune, use_persistent_gemm=True, ctx=ctx,
                          row_scale=row_scale, col_scale=col_scale)
    # reset (reference :459-462); stream-ordered after the GEMM and after every producer copy
    fill_flags(ctx.barrier_tensors[ctx.rank], 0)
    return C
