"""Benchmark of the hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--only c2]

Headline (one JSON line on stdout): BASELINE config 2, the GEMM-RS one-rank share at the Llama-70B TP=8
MLP-down shape — a "step" is one gemm_rs_intra_node call: the scatter-epilogue GEMM
A[8192,3584] x B[8192,3584]^T plus the fp32 reduction of 8 partial slices [1024,8192]. ``value`` is the
algorithmic GEMM work (2*M*N*K) over the whole step time. The same line carries
  roofline      the dominant kernel (the GEMM) against the bf16 dense MFMA peak, its launch time measured
                with HIP events on the launch stream,
  cpu_baseline  the oracle's torch golden for the same step timed on the host cores,
  kernels       every other hot-path kernel at its BASELINE config with its own roofline fraction.
Inputs are synthetic, seeded, and resident in HBM before any timed region. Every timed region is preceded by
``--settle-seconds`` (1.5 s) of the same launches, untimed, and then by the ``--warmup`` launches: after an idle
gap the GPU spends its first ~0.7 s of work at a lower core clock than the one it then sustains, and it is the
sustained rate that is reported.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "triton-distributed_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

PEAK = {"bf16": 2.5e15, "fp8": 5.0e15, "hbm": 8.0e12}  # MI355X published dense MFMA peaks (FLOP/s) and HBM3E B/s
# HBM-side bytes per launch, read off two rocprofv3 counter passes over this same script (FETCH_SIZE, then
# WRITE_SIZE, KiB per dispatch, each scaled by what the counter reads for the 1 GiB copy kernel: x2.000 and
# x1.000). Counters cannot be collected inside a timed run, so the figures are carried here as constants;
# the summaries are kept under profiles/. Each figure names the kernel sources it was measured on, and
# MEASURED_SOURCE_DIGEST holds those sources' digests at the time: a figure whose sources have changed since is
# reported as null, not as a measurement (tests/test_bench_constants.py fails until it is measured again).
MEASURED_TRAFFIC_BYTES = {
    "c2_gemm": (840.0e6, ("gemm.hip", "common.h")), "c2_reduce": (151.0e6, ("reduce.hip", "common.h")),
    "c1_gemm": (130.4e6, ("gemm.hip", "common.h")), "c3_gemm": (1646.0e6, ("gemm.hip", "common.h")),
    "c4_dispatch": (265.8e6, ("moe.hip", "common.h")), "c4_dispatch_from_ids": (267.4e6, ("moe.hip", "common.h")),
    "c4_combine": (296.7e6, ("moe.hip", "common.h")), "c5_split_kv": (4318.1e6, ("decode.hip", "common.h")),
}
MEASURED_SOURCE_DIGEST = {
    "common.h": "29a71d5d51010d68",
    "decode.hip": "5f65cc9c7465e64c",
    "gemm.hip": "5b1de058c7b76344",
    "moe.hip": "3ab3dfd4ffc67cea",
    "reduce.hip": "469689d34df1b205",
}
CSRC = os.path.join(ROOT, "triton-distributed_amd", "csrc")


def source_digest(name):
    """sha256 (first 16 hex digits) of a kernel source with comments and white space taken out, so that only a
    change of code makes a measurement stale."""
    import hashlib
    import re
    text = open(os.path.join(CSRC, name)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"//[^\n]*", "", text)
    return hashlib.sha256("".join(text.split()).encode()).hexdigest()[:16]


def measured_traffic(key):
    """The measured HBM-side bytes of one launch, or None when a source the figure was measured on has changed."""
    value, sources = MEASURED_TRAFFIC_BYTES[key]
    for name in sources:
        if source_digest(name) != MEASURED_SOURCE_DIGEST.get(name):
            log("traffic of %s: %s has changed since the counters were read; reporting null" % (key, name))
            return None
    return value


LIVE_PRODUCER = True  # --no-live-producer clears it
METRIC = "AG-GEMM/GEMM-RS TFLOPS (% MFMA peak); decode & A2A GB/s (% HBM peak)"


def log(*a):
    print(*a, file=sys.stderr, flush=True)


SETTLE_SECONDS = 1.5  # --settle-seconds


def settle(fn, seconds=None):
    """Keeps the GPU busy with ``fn`` for ``seconds`` so that the timed region starts at the sustained clock: after
    an idle gap this GPU runs its first ~0.7 s of work at a lower core clock than it then holds for good."""
    import torch
    seconds = SETTLE_SECONDS if seconds is None else seconds
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(20):
            fn()
        torch.cuda.synchronize()


def time_launches(fn, steps, warmup):
    """Average duration in seconds of ``fn`` (which launches on torch's current stream), HIP events on that
    stream around ``steps`` back-to-back calls, after the settle period and ``warmup`` untimed calls."""
    import torch
    settle(fn)
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(steps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) * 1e-3 / steps


def time_live_ag_gemm(call, ctx, steps, warmup):
    """Times the AG-GEMM with its producer running, in the reference's order (producer queued first, then the gated
    GEMM); a bounded flag wait that expired is an error. Returns (seconds, order)."""
    call()
    ctx.check_status()
    s = time_launches(call, steps, warmup)
    ctx.check_status()
    return s, "copies_first"


XGMI_LINK_GBPS = 153.0   # one xGMI link of MI355X: the rate at which one peer's rows arrive


def paced_ag_gemm(make_call, world, rank, mpr, N, K, in_dtype, peer_shards, chunk_rows, pre_s, steps, warmup):
    """AG-GEMM with every peer's chunks held back to the pace of one xGMI link per peer (the one-GPU producer kernel
    copies chunk c of every peer no earlier than (c+1) chunk times of a link after the call started), for several
    chunk sizes. Overlap efficiency = time with every flag pre-set / time with paced arrivals; the time includes
    the host's queueing of the call (three streams, their events), which is what bounds the small config.
    ``straggler``: on top of the pacing, the peer that the static order expects first is late, so that chunks arrive out
    of the order the static schedule walks them in: timed with the tiles taken in arrival order (the default) and in
    the static order."""
    import torch
    from triton_dist import _lib
    from triton_dist.kernels.amd import create_ag_gemm_intra_node_context
    out = {}
    for rows in chunk_rows:
        ctx = create_ag_gemm_intra_node_context(world * mpr, N, K, in_dtype, torch.bfloat16, rank, world, None,
                                                M_PER_CHUNK=rows)
        ctx.set_peer_shards(peer_shards)
        ctx.link_gbps = XGMI_LINK_GBPS
        ctx.producer_kernel, ctx.producer_workgroups = True, 16   # every peer in one launch, pacing inside the kernel
        s, order = time_live_ag_gemm(make_call(ctx), ctx, max(steps // 2, 1), warmup)
        arrive_us = mpr * K * peer_shards[(rank + 1) % world].element_size() / XGMI_LINK_GBPS / 1e3
        out["m_per_chunk_%d" % rows] = {"us": round(s * 1e6, 2), "order": order,
                                        "overlap_efficiency": round(pre_s / s, 4),
                                        "last_chunk_arrives_us": round(arrive_us, 1)}
        if rows == chunk_rows[-1]:
            # a straggler: the peer the static order expects first delivers its first chunk `late` us late (a third of
            # the call's time with every flag set), its other chunks behind it
            late = round(pre_s * 1e6 / 3)
            ctx.late_chunks_us = {((rank + 1) % world) * (mpr // rows): late}
            res = {"first_peer_late_by_us": late}
            for name, static in (("arrival_order", False), ("static_order", True)):
                old = _lib.load().tdist_debug_get(_lib.TDIST_DEBUG_GEMM_SCHEDULE)
                if static:
                    _lib.check(_lib.load().tdist_debug_set(_lib.TDIST_DEBUG_GEMM_SCHEDULE, 0))
                try:
                    js, _ = time_live_ag_gemm(make_call(ctx), ctx, max(steps // 2, 1), warmup)
                finally:
                    _lib.check(_lib.load().tdist_debug_set(_lib.TDIST_DEBUG_GEMM_SCHEDULE, old))
                res[name + "_us"] = round(js * 1e6, 2)
            out["m_per_chunk_%d" % rows]["straggler"] = res
    return out


def cpu_time(fn):
    """Wall time of one call of ``fn`` on the host cores (torch's thread pool at its default width)."""
    import torch
    t0 = time.perf_counter()
    fn()
    return time.perf_counter() - t0, torch.get_num_threads()


def roof(bound, work, seconds, peak_key, traffic=None):
    achieved = work / seconds
    unit = "TFLOP/s" if bound == "mfma" else "GB/s"
    scale = 1e12 if bound == "mfma" else 1e9
    return {
        "bound": bound,
        "achieved": round(achieved / scale, 2),
        "peak": PEAK[peak_key] / scale,
        "unit": unit,
        "frac": round(achieved / PEAK[peak_key], 4),
        "traffic": traffic,
        "us_per_launch": round(seconds * 1e6, 2),
    }


# ---- workloads ------------------------------------------------------------------------------------------
def bench_c2(dev, steps, warmup):
    """GEMM-RS: returns (step seconds, gemm roofline, reduce roofline, cpu baseline)."""
    import torch
    from oracle import golden
    from triton_dist.kernels.amd import create_gemm_rs_intra_node_context, gemm_rs_intra_node
    from triton_dist.kernels.amd.gemm_reduce_scatter import matmul_fuse_scatter, ring_reduce_after_scatter
    W, rank, M, N, K = 8, 0, 8192, 8192, 3584
    g = torch.Generator().manual_seed(3 + 1)
    a = torch.randn((M, K), generator=g).to(torch.bfloat16)
    b = (torch.randn((N, K), generator=g) * 0.02).to(torch.bfloat16)
    peers = [None if r == rank else torch.randn((M // W, N), generator=g).to(torch.bfloat16) for r in range(W)]
    ctx = create_gemm_rs_intra_node_context(M, N, torch.bfloat16, rank, W, None)
    ctx.set_peer_partials(peers)
    a_d, b_d = a.to(dev), b.to(dev)
    flops = 2.0 * M * N * K

    # whole step: settle, `warmup` untimed steps, then sync on both sides of exactly `steps` steps
    settle(lambda: gemm_rs_intra_node(a_d, b_d, ctx))
    for _ in range(warmup):
        out = gemm_rs_intra_node(a_d, b_d, ctx)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        out = gemm_rs_intra_node(a_d, b_d, ctx)
    torch.cuda.synchronize()
    step_s = (time.perf_counter() - t0) / steps

    err = golden.max_rel_err(out.float().cpu(), golden.gemm_rs_fp32(a, b, peers, rank, W))
    assert err <= 1e-2, "GEMM-RS result off: max rel err %g" % err

    stream = torch.cuda.current_stream()
    gemm_s = time_launches(lambda: matmul_fuse_scatter(a_d, b_d, ctx.scatter_bufs_ptr, rank, W, False, stream=stream),
                           steps, warmup)
    scatter_out = ctx.scatter_bufs[rank][:M]
    red_s = time_launches(lambda: ring_reduce_after_scatter(rank, W, scatter_out, stream), steps, warmup)
    red_bytes = (W + 1) * (M // W) * N * 2

    # CPU baseline: the oracle's golden for the same step (bf16 up-cast to fp32, as the torch golden runs on
    # a CPU), timed on the host cores. A 1/8 row sample first; the full problem if that is quick.
    torch.set_num_threads(max(1, min(os.cpu_count() or 1, 64)))
    cores = torch.get_num_threads()
    rows = M // 8
    t0 = time.perf_counter()
    (a[:rows].float() @ b.float().T)
    probe = time.perf_counter() - t0
    if probe * 8 <= 30.0:
        # the full step, repeated for about ten seconds of CPU work (at least three times): the mean is the baseline
        reps, t0 = 0, time.perf_counter()
        while reps < 3 or (time.perf_counter() - t0 < 10.0 and reps < 200):
            golden.gemm_rs_fp32(a, b, peers, rank, W).to(torch.bfloat16)
            reps += 1
        total = time.perf_counter() - t0
        cpu_s = total / reps
        cpu = {"value": round(flops / cpu_s / 1e12, 4), "unit": "TFLOP/s", "cores": cores, "kind": "port",
               "sample": "full step x %d (fp32 up-cast golden: [8192,3584]x[3584,8192] + 8-slice sum), %.1f s of CPU "
                         "work, %.2f s per step" % (reps, total, cpu_s)}
    else:
        cpu = {"value": round(flops / 8 / probe / 1e12, 4), "unit": "TFLOP/s", "cores": cores, "kind": "port",
               "sample": "1/8 of the rows (1024 of 8192) of the fp32 up-cast golden GEMM, %.2f s" % probe}
    gemm_roof = roof("mfma", flops, gemm_s, "bf16", measured_traffic("c2_gemm"))
    # The same launch on constant operands (all ones): the matrix cores then draw far less power and the clock stays
    # up, so this rate shows the schedule's cycles rather than the power limit that the seeded random operands run into.
    ones_a, ones_b = torch.ones_like(a_d), torch.ones_like(b_d)
    const_s = time_launches(lambda: matmul_fuse_scatter(ones_a, ones_b, ctx.scatter_bufs_ptr, rank, W, False, stream=stream),
                            max(steps // 2, 1), warmup)
    lib_out = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
    lib_const_s = time_launches(lambda: torch.matmul(ones_a, ones_b.t(), out=lib_out), max(steps // 2, 1), warmup)
    gemm_roof["constant_operands"] = {"us_per_launch": round(const_s * 1e6, 2), "frac": round(flops / const_s / PEAK["bf16"], 4),
                                      "hipblaslt_us_per_launch": round(lib_const_s * 1e6, 2),
                                      "hipblaslt_frac": round(flops / lib_const_s / PEAK["bf16"], 4)}
    del ones_a, ones_b, lib_out
    return (step_s, gemm_roof, roof("hbm", red_bytes, red_s, "hbm", measured_traffic("c2_reduce")), cpu, err)


def bench_c1(dev, steps, warmup):
    import torch
    from oracle import golden
    from triton_dist.kernels.amd import ag_gemm_intra_node, create_ag_gemm_intra_node_context, gated_gemm
    world, rank, mpr, K, N = 4, 0, 1024, 4096, 1536
    g = torch.Generator().manual_seed(3 + 0)
    shards = [torch.randn((mpr, K), generator=g).to(torch.bfloat16) for _ in range(world)]
    b = (torch.randn((N, K), generator=g) * 0.02).to(torch.bfloat16)
    ctx = create_ag_gemm_intra_node_context(world * mpr, N, K, torch.bfloat16, torch.bfloat16, rank, world, None, M_PER_CHUNK=1024)
    ctx.set_peer_shards({r: s.to(dev) for r, s in enumerate(shards) if r != rank})
    a_d, b_d = shards[rank].to(dev), b.to(dev)
    flops = 2.0 * world * mpr * N * K
    live_s, live_order = None, None
    if LIVE_PRODUCER:
        live_s, live_order = time_live_ag_gemm(lambda: ag_gemm_intra_node(a_d, b_d, False, ctx), ctx, steps, warmup)
        c = ag_gemm_intra_node(a_d, b_d, False, ctx)
        ctx.check_status()
        err = golden.max_rel_err(c.float().cpu(), golden.ag_gemm_fp32(shards, b))
        assert err <= 1e-2
    # kernel alone, every flag already released
    full = torch.cat(shards).to(dev)
    flags = torch.ones(world, dtype=torch.int32, device=dev)
    out = torch.empty((world * mpr, N), dtype=torch.bfloat16, device=dev)
    pre_s = time_launches(lambda: gated_gemm(full, None, 0, b_d, out, flags, 1024, rank, world, sk_workspace=ctx.sk_workspace), steps, warmup)
    r = roof("mfma", flops, pre_s, "bf16", measured_traffic("c1_gemm"))
    cs, cores = cpu_time(lambda: golden.torch_ag_gemm(shards, b))
    r["cpu_baseline"] = {"value": round(flops / cs / 1e12, 4), "unit": "TFLOP/s", "cores": cores, "kind": "port",
                         "sample": "the whole config once (torch golden: cat + matmul), %.2f s" % cs}
    r["with_live_producer_us"] = round(live_s * 1e6, 2) if live_s is not None else None
    r["live_producer_order"] = live_order
    if LIVE_PRODUCER:
        r["paced_xgmi_%dGBps" % XGMI_LINK_GBPS] = paced_ag_gemm(
            lambda c: (lambda: ag_gemm_intra_node(a_d, b_d, False, c)), world, rank, mpr, N, K, torch.bfloat16,
            ctx.peer_shards, (1024, 256), pre_s, steps, warmup)
    return r


def bench_c3(dev, steps, warmup):
    import torch
    from oracle import golden
    from triton_dist.kernels.amd import ag_gemm_intra_node, create_ag_gemm_intra_node_context, gated_gemm
    world, rank, mpr, K, N = 8, 0, 2048, 8192, 7168
    g = torch.Generator().manual_seed(3 + 2)
    shards = [torch.randn((mpr, K), generator=g).to(torch.float8_e4m3fn) for _ in range(world)]
    b = torch.randn((N, K), generator=g).to(torch.float8_e4m3fn)
    sa = (torch.rand(world * mpr, generator=g) * 0.09 + 0.01).to(dev)
    sb = (torch.rand(N, generator=g) * 0.009 + 0.001).to(dev)
    ctx = create_ag_gemm_intra_node_context(world * mpr, N, K, torch.float8_e4m3fn, torch.bfloat16, rank, world, None,
                                            M_PER_CHUNK=2048)
    ctx.set_peer_shards({r: s.to(dev) for r, s in enumerate(shards) if r != rank})
    a_d, b_d = shards[rank].to(dev), b.to(dev)
    flops = 2.0 * world * mpr * N * K
    live_s, live_order = None, None
    if LIVE_PRODUCER:
        live_s, live_order = time_live_ag_gemm(lambda: ag_gemm_intra_node(a_d, b_d, False, ctx, row_scale=sa, col_scale=sb),
                                               ctx, steps, warmup)
        c = ag_gemm_intra_node(a_d, b_d, False, ctx, row_scale=sa, col_scale=sb)
        ctx.check_status()
        rows = slice(5 * mpr + 11, 5 * mpr + 75)
        ref = golden.fp8_scaled_gemm_fp32(shards[5][11:75], sa.cpu()[rows], b, sb.cpu())
        err = golden.max_rel_err(c[rows].float().cpu(), ref)
        assert err <= 1e-2
    full = torch.cat([s.view(torch.uint8) for s in shards]).to(dev).view(torch.float8_e4m3fn)
    flags = torch.ones(world, dtype=torch.int32, device=dev)
    out = torch.empty((world * mpr, N), dtype=torch.bfloat16, device=dev)
    pre_s = time_launches(lambda: gated_gemm(full, None, 0, b_d, out, flags, 2048, rank, world, row_scale=sa, col_scale=sb,
                                             sk_workspace=ctx.sk_workspace),
                          steps, warmup)
    r = roof("mfma", flops, pre_s, "fp8", measured_traffic("c3_gemm"))
    sa_c, sb_c = sa.cpu(), sb.cpu()
    cs, cores = cpu_time(lambda: golden.fp8_scaled_gemm_fp32(shards[0][:1024], sa_c[:1024], b, sb_c))
    r["cpu_baseline"] = {"value": round(flops / 16 / cs / 1e12, 4), "unit": "TFLOP/s", "cores": cores, "kind": "port",
                         "sample": "1024 of the 16384 rows (fp32 up-cast golden with scales), %.2f s" % cs}
    r["with_live_producer_us"] = round(live_s * 1e6, 2) if live_s is not None else None
    r["live_producer_order"] = live_order
    if LIVE_PRODUCER:
        r["paced_xgmi_%dGBps" % XGMI_LINK_GBPS] = paced_ag_gemm(
            lambda c: (lambda: ag_gemm_intra_node(a_d, b_d, False, c, row_scale=sa, col_scale=sb)), world, rank, mpr, N, K,
            torch.float8_e4m3fn, ctx.peer_shards, (2048, 512), pre_s, steps, warmup)
    return r


def bench_c4(dev, steps, warmup):
    import torch
    from oracle import golden
    from triton_dist.kernels.amd import (create_all_to_all_context, fast_all_to_all, moe_dispatch_preprocess,
                                         moe_weighted_combine)
    T, topk, G, W, H, max_m = 4096, 8, 256, 32, 7168, 4096
    g = torch.Generator().manual_seed(3 + 3)
    ids = golden.random_distinct_experts(T, G, topk, g)
    q, s = golden.quantize_per_token_e4m3(torch.randn((T, H), generator=g))
    w = torch.softmax(torch.randn((T, topk), generator=g), dim=-1).float().contiguous().to(dev)
    ctx = create_all_to_all_context(max_m, H, 0, G, W, G // W, dtype=torch.float8_e4m3fn)
    ids_d, q_d, s_d = ids.to(dev), q.to(dev), s.to(dev)
    splits, cumsum, scatter, gather = moe_dispatch_preprocess(ids_d, G)
    pre_s = time_launches(lambda: moe_dispatch_preprocess(ids_d, G, ctx=ctx), steps, warmup)
    disp_s = time_launches(lambda: fast_all_to_all(ctx, q_d, cumsum, s_d, scatter_index=scatter), steps, warmup)

    def index_then_dispatch():
        _, cs, sc, _ = moe_dispatch_preprocess(ids_d, G, ctx=ctx)
        fast_all_to_all(ctx, q_d, cs, s_d, scatter_index=sc)
    two_s = time_launches(index_then_dispatch, steps, warmup)
    # the same from the raw ids in ONE launch: every workgroup of the dispatch counts the ids itself
    both_s = time_launches(lambda: fast_all_to_all(ctx, q_d, None, s_d, expert_ids=ids_d), steps, warmup)
    _, recv, recv_scale = fast_all_to_all(ctx, q_d, cumsum, s_d, scatter_index=scatter)
    comb_s = time_launches(lambda: moe_weighted_combine(ctx, recv, recv_scale, scatter, w, cumsum), steps, warmup)
    n = T * topk
    disp_bytes = T * H + n * H + T * 4 + n * 4 + n * 4          # unique row reads + row writes + scales + gather index
    comb_bytes = n * H + n * 4 + n * 4 + n * 4 + T * H * 2      # row reads + scales + weights + scatter index + bf16 out
    d = roof("hbm", disp_bytes, disp_s, "hbm", measured_traffic("c4_dispatch"))

    def cpu_dispatch():
        _, c_cumsum, _, c_gather, _ = golden.moe_preprocess(ids, G)
        rows = q.view(torch.uint8)[c_gather.long()]
        golden.dispatch_slots(rows, s[c_gather.long()], c_cumsum, W, G // W, max_m)
    cs, cores = cpu_time(cpu_dispatch)
    d["cpu_baseline"] = {"value": round(disp_bytes / cs / 1e9, 2), "unit": "GB/s", "cores": cores, "kind": "port",
                         "sample": "the whole config once (bincount, stable argsort, index_select, slot copies), %.2f s" % cs}
    d["index_build_us"] = round(pre_s * 1e6, 2)
    # the dispatch end to end: splits / cumsum / scatter index from the raw expert ids (one launch, the context's own
    # tensors, no allocation), then the row movement; the ids' 131 KB are added to the bytes
    d["with_index_build"] = {"us": round(both_s * 1e6, 2), "achieved_GBps": round((disp_bytes + n * 4) / both_s / 1e9, 1),
                             "frac": round((disp_bytes + n * 4) / both_s / PEAK["hbm"], 4),
                             "traffic": measured_traffic("c4_dispatch_from_ids"),
                             "as_two_launches_us": round(two_s * 1e6, 2)}
    # the step after the dispatch: align / sort of the same ids for the grouped GEMM (8 rank segments, block 128)
    from triton_dist.kernels.amd import sort_topk_ids_align_block_size
    ids64 = ids_d.long()
    align_s = time_launches(lambda: sort_topk_ids_align_block_size(ids64, G, 8, T // 8, 128), steps, warmup)
    d["align_sort_us"] = round(align_s * 1e6, 2)
    # dispatch with the e4m3 quantisation (groups of 128 columns) fused in: bf16 tokens read once, 8 e4m3 copies written
    ctx_q = create_all_to_all_context(max_m, H, 0, G, W, G // W, dtype=torch.float8_e4m3fn, fp8_group_size=128)
    xb = torch.randn((T, H), generator=g).to(torch.bfloat16).to(dev)
    qd_s = time_launches(lambda: fast_all_to_all(ctx_q, xb, cumsum, None, scatter_index=scatter, online_quant_fp8=True),
                         steps, warmup)
    qd_bytes = T * H * 2 + n * H + n * (H // 128) * 4 + n * 4
    d["online_quant_dispatch"] = {"us_per_launch": round(qd_s * 1e6, 2), "achieved_GBps": round(qd_bytes / qd_s / 1e9, 1),
                                  "frac": round(qd_bytes / qd_s / PEAK["hbm"], 4)}
    c = roof("hbm", comb_bytes, comb_s, "hbm", measured_traffic("c4_combine"))
    _, _, c_scatter, c_gather, _ = golden.moe_preprocess(ids, G)
    rows_f32 = q[c_gather.long()].float()
    cs, cores = cpu_time(lambda: golden.weighted_combine(rows_f32, s[c_gather.long()], c_scatter, w.cpu()))
    c["cpu_baseline"] = {"value": round(comb_bytes / cs / 1e9, 2), "unit": "GB/s", "cores": cores, "kind": "port",
                         "sample": "the whole config once (scale, gather by scatter index, weighted sum over k), %.2f s" % cs}
    return d, c


def bench_c5(dev, steps, warmup):
    import torch
    from triton_dist.kernels.amd.flash_decode import _split_kv, decode_combine, decode_fused
    B, Hq, Hkv, D, L, S, page = 32, 64, 8, 128, 32768, 16, 16
    g = torch.Generator(device="cuda").manual_seed(3 + 4)
    pages_per_seq = L // page
    num_pages = B * pages_per_seq
    k = torch.randn((num_pages, page, Hkv, D), generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16)
    v = torch.randn((num_pages, page, Hkv, D), generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16)
    q = torch.randn((B, Hq, D), generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16)
    table = torch.randperm(num_pages, generator=torch.Generator().manual_seed(6)).view(B, pages_per_seq).int().to(dev)
    lens = torch.full((B, ), L, dtype=torch.int32, device=dev)
    out_split = torch.empty((B, Hq, S, D), dtype=torch.float32, device=dev)
    lse_split = torch.empty((B, Hq, S), dtype=torch.float32, device=dev)
    scale = D**-0.5
    split_s = time_launches(lambda: _split_kv(q, k, v, lens, table, scale, 0.0, S, out_split, lse_split), steps, warmup)
    merged = torch.empty((B, Hq, D), dtype=torch.bfloat16, device=dev)
    comb_s = time_launches(
        lambda: decode_combine(out_split, lse_split, S, 1, lens, B, Hq, D,
                               (out_split.stride(2), out_split.stride(0), out_split.stride(1)),
                               (lse_split.stride(2), lse_split.stride(0), lse_split.stride(1)), merged), steps, warmup)

    def two_launches():
        _split_kv(q, k, v, lens, table, scale, 0.0, S, out_split, lse_split)
        decode_combine(out_split, lse_split, S, 1, lens, B, Hq, D,
                       (out_split.stride(2), out_split.stride(0), out_split.stride(1)),
                       (lse_split.stride(2), lse_split.stride(0), lse_split.stride(1)), merged)

    both_s = time_launches(two_launches, steps, warmup)
    # the same in one launch: the last workgroup of a (sequence, head block) merges its splits
    fused_out = torch.empty_like(merged)
    fused_s = time_launches(lambda: decode_fused(q, k, v, lens, table, scale, 0.0, S, fused_out, None,
                                                 out_split=out_split, lse_split=lse_split), steps, warmup)
    if not torch.equal(fused_out.view(torch.int16), merged.view(torch.int16)):
        raise RuntimeError("fused decode differs from split + combine")
    # the rank merge of BASELINE config 5: own (out, LSE) + 7 seeded synthetic peer shards -> [32, 64, 128] bf16
    from triton_dist.kernels.amd import gqa_fwd_batch_decode_inter_rank_combine
    g2 = torch.Generator(device="cuda").manual_seed(3 + 4 + 100)
    R = 8
    all_out = torch.randn((R, B, Hq, D), generator=g2, device=dev, dtype=torch.float32).to(torch.bfloat16)
    all_lse = torch.randn((R, B, Hq), generator=g2, device=dev, dtype=torch.float32) * 2 + 10.4
    all_lens = torch.full((R, B), L, dtype=torch.int32, device=dev)
    final = torch.empty((B, Hq, D), dtype=torch.bfloat16, device=dev)
    rank_s = time_launches(lambda: gqa_fwd_batch_decode_inter_rank_combine(all_out, all_lse, all_lens, final), steps, warmup)
    kv_bytes = 2 * B * L * Hkv * D * 2
    split_bytes = kv_bytes + q.numel() * 2 + table.numel() * 4 + out_split.numel() * 4 + lse_split.numel() * 4
    r = roof("hbm", split_bytes, split_s, "hbm", measured_traffic("c5_split_kv"))
    from oracle import golden
    pages1 = table[0].long()
    k1, v1, q1 = k[pages1].cpu(), v[pages1].cpu(), q[:1].cpu()
    t1 = torch.arange(pages_per_seq, dtype=torch.int32).view(1, -1)
    cs, cores = cpu_time(lambda: golden.ref_paged_attn(q1, k1, v1, [1], [L], t1, scale))
    r["cpu_baseline"] = {"value": round(split_bytes / B / cs / 1e9, 2), "unit": "GB/s", "cores": cores, "kind": "port",
                         "sample": "one of the 32 sequences (torch golden ref_paged_attn, 32768 keys), %.2f s" % cs}
    r["combine_us"] = round(comb_s * 1e6, 2)
    r["split_then_combine_us"] = round(both_s * 1e6, 2)
    r["fused_split_and_combine_us"] = round(fused_s * 1e6, 2)
    r["inter_rank_combine_us"] = round(rank_s * 1e6, 2)
    # the reference layer's defaults (layers/nvidia/sp_flash_decode_layer.py:45,61): 32 splits, and pages of one token
    # (the same caches seen as 1 048 576 pages of one token each, every token of a sequence at a random place: 2 KB
    # gather granules per cache and a 4.19 MB block table)
    S32 = 32
    out32 = torch.empty((B, Hq, S32, D), dtype=torch.float32, device=dev)
    lse32 = torch.empty((B, Hq, S32), dtype=torch.float32, device=dev)
    s32_s = time_launches(lambda: _split_kv(q, k, v, lens, table, scale, 0.0, S32, out32, lse32), steps, warmup)
    r32 = roof("hbm", kv_bytes + q.numel() * 2 + table.numel() * 4 + out32.numel() * 4 + lse32.numel() * 4, s32_s, "hbm")
    r32["workload"] = "C5 with 32 splits (page 16)"
    k1p, v1p = k.view(num_pages * page, 1, Hkv, D), v.view(num_pages * page, 1, Hkv, D)
    table1 = torch.randperm(B * L, generator=torch.Generator().manual_seed(7)).view(B, L).int().to(dev)
    p1_s = time_launches(lambda: _split_kv(q, k1p, v1p, lens, table1, scale, 0.0, S, out_split, lse_split), steps, warmup)
    rp1 = roof("hbm", kv_bytes + q.numel() * 2 + table1.numel() * 4 + out_split.numel() * 4 + lse_split.numel() * 4, p1_s, "hbm")
    rp1["workload"] = "C5 with pages of one token (16 splits), tokens at random places"
    p1s32_s = time_launches(lambda: _split_kv(q, k1p, v1p, lens, table1, scale, 0.0, S32, out32, lse32), steps, warmup)
    rp1["with_32_splits_us"] = round(p1s32_s * 1e6, 2)
    return r, r32, rp1


def bench_group_gemm(dev, steps, warmup):
    """AG + grouped GEMM of the MoE tensor-parallel path at the reference's Mixtral-8x7B layer shape
    (test/nvidia/test_ag_moe.py:160-171: K 14336, N 4096 over 8 ranks, 8 experts, top-2) with 8192 tokens: the step
    that consumes the align / sort output. Not a BASELINE config; reported beside them."""
    import torch
    from oracle import golden
    from triton_dist.kernels.amd import (ag_group_gemm_intra_node, create_ag_group_gemm_intra_node_context,
                                         group_gemm_gated)
    world, rank, mpr, K, N, E, topk, block = 8, 0, 1024, 14336, 512, 8, 2, 128
    g = torch.Generator().manual_seed(3 + 7)
    shards = [torch.randn((mpr, K), generator=g).to(torch.bfloat16) for _ in range(world)]
    w_nk = (torch.randn((E, N, K), generator=g) * 0.02).to(torch.bfloat16).to(dev)
    w = w_nk.transpose(1, 2)                       # [E, K, N] as the reference takes it, K-contiguous underneath
    ids = golden.random_distinct_experts(world * mpr, E, topk, g).to(dev)
    a_d = shards[rank].to(dev)
    ctx = create_ag_group_gemm_intra_node_context(None, a_d, w, ids, E, max_M=world * mpr, BLOCK_M=block, rank=rank,
                                                  num_ranks=world)
    ctx.set_peer_shards({r: s.to(dev) for r, s in enumerate(shards) if r != rank})
    flops = 2.0 * world * mpr * topk * K * N
    live_s = None
    if LIVE_PRODUCER:
        c = ag_group_gemm_intra_node(a_d, w, ctx)
        ctx.check_status()
        rows = torch.arange(5 * mpr * topk + 3, 5 * mpr * topk + 67)
        ref = golden.ag_group_gemm_fp32(shards, w.cpu(), ids.cpu())[rows]
        assert golden.max_rel_err(c[rows.to(dev)].float().cpu(), ref) <= 1e-2
        live_s = time_launches(lambda: ag_group_gemm_intra_node(a_d, w, ctx), steps, warmup)
        ctx.check_status()
    full = torch.cat(shards).to(dev)
    flags = torch.ones(world, dtype=torch.int32, device=dev)
    out = torch.empty((world * mpr * topk, N), dtype=torch.bfloat16, device=dev)
    pre_s = time_launches(
        lambda: group_gemm_gated(full, None, 0, w_nk, out, ctx.sorted_topk_ids, ctx.aligned_expert_ids,
                                 ctx.aligned_barrier_ids, ctx.aligned_num_tokens, block, ctx.full_num_tokens, topk, mpr,
                                 ctx.first_block, flags, rank, sk_workspace=ctx.sk_workspace), steps, warmup)
    r = roof("mfma", flops, pre_s, "bf16")
    r["workload"] = "8192 tokens x top-2 of 8 experts, K 14336, N 512 per rank, row blocks of 128 (128 x 256 tiles)"
    r["with_live_producer_us"] = round(live_s * 1e6, 2) if live_s is not None else None
    return r


def bench_copy(dev, steps, warmup):
    import torch
    from triton_dist import _lib
    n = 1 << 30
    src = torch.empty(n, dtype=torch.uint8, device=dev)
    dst = torch.empty(n, dtype=torch.uint8, device=dev)
    s = time_launches(lambda: _lib.bench_call("tdist_copy_bytes", dst.data_ptr(), src.data_ptr(), n, _lib.stream_ptr()), steps, warmup)
    r = roof("hbm", 2 * n, s, "hbm")
    # the one-directional streams over the same 1 GiB (four times the memory-side cache): what HBM sustains for
    # writes alone (the MoE dispatch writes 8 bytes per byte it reads) and for reads alone (combine, decode)
    sink = torch.zeros(256, dtype=torch.int32, device=dev)
    w = time_launches(lambda: _lib.bench_call("tdist_fill_bytes", dst.data_ptr(), n, _lib.stream_ptr()), steps, warmup)
    rd = time_launches(lambda: _lib.bench_call("tdist_read_bytes", src.data_ptr(), n, sink.data_ptr(), _lib.stream_ptr()), steps, warmup)
    r["write_only"] = {"achieved_GBps": round(n / w / 1e9, 1), "frac": round(n / w / PEAK["hbm"], 4)}
    r["read_only"] = {"achieved_GBps": round(n / rd / 1e9, 1), "frac": round(n / rd / PEAK["hbm"], 4)}
    return r


def bench_mfma_ceiling(dev, steps, warmup):
    """The MFMA rate the chip sustains with no memory traffic, on constant and on random register operands."""
    import torch
    from triton_dist import _lib
    cus = _lib.load().tdist_num_cus()
    sink = torch.empty(cus * 256, dtype=torch.float32, device=dev)
    iters = 1000
    out = {}
    for name, code, kstep in (("bf16", _lib.TDIST_BF16, 16), ("fp8", _lib.TDIST_F8E4M3, 64)):
        for entry, rows, ks in (("tdist_mfma_rate_probe", "", kstep), ("tdist_mfma_rate_probe_16row", "_16row_mfma", 2 * kstep)):
            for rnd in (0, 1):
                if rows and not rnd:
                    continue
                s = time_launches(lambda: _lib.bench_call(entry, code, rnd, iters, sink.data_ptr(), _lib.stream_ptr()),
                                  max(steps // 4, 5), warmup)
                tf = cus * 4 * iters * 2.0 * 128 * 128 * ks / s / 1e12
                out["%s_%s_operands%s_TFLOPs" % (name, "random" if rnd else "constant", rows)] = round(tf, 1)
    return out


def bench_library_gemm(dev, steps, warmup):
    """Yardstick, not product: the vendor library's GEMM (torch.matmul = hipBLASLt) on the headline shape and the
    same seeded operands, timed the same way. Says what fraction of the nominal peak AMD's own kernel sustains on
    this data under the same power limit."""
    import torch
    M, N, K = 8192, 8192, 3584
    g = torch.Generator().manual_seed(3 + 1)
    a = torch.randn((M, K), generator=g).to(torch.bfloat16).to(dev)
    b = (torch.randn((N, K), generator=g) * 0.02).to(torch.bfloat16).to(dev)
    bt = b.t()
    out = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
    s = time_launches(lambda: torch.matmul(a, bt, out=out), steps, warmup)
    return roof("mfma", 2.0 * M * N * K, s, "bf16")


def bench_library_fp8_gemm(dev, steps, warmup):
    """Yardstick, not product: the vendor library's e4m3 GEMM (torch._scaled_mm) on the C3 shape and the same seeded
    operands and scales: with one scale per row of A and per row of B (what the C3 kernel applies), and with one
    scale per tensor."""
    import torch
    M, N, K = 16384, 7168, 8192
    g = torch.Generator().manual_seed(3 + 2)
    a = torch.randn((M, K), generator=g).to(torch.float8_e4m3fn).to(dev)
    b = torch.randn((N, K), generator=g).to(torch.float8_e4m3fn).to(dev)
    sa = (torch.rand(M, generator=g) * 0.09 + 0.01).to(dev)
    sb = (torch.rand(N, generator=g) * 0.009 + 0.001).to(dev)
    one = torch.ones((), device=dev)
    out = {}
    for name, scale_a, scale_b in (("row_scales", sa.view(M, 1), sb.view(1, N)), ("tensor_scales", one, one)):
        try:
            call = lambda: torch._scaled_mm(a, b.t(), scale_a=scale_a, scale_b=scale_b, out_dtype=torch.bfloat16)
            call()
            r = roof("mfma", 2.0 * M * N * K, time_launches(call, max(steps // 2, 1), warmup), "fp8")
            out[name] = {k: r[k] for k in ("achieved", "frac", "us_per_launch")}
        except Exception as exc:   # (a library without this form of the call)
            out[name] = {"unavailable": repr(exc)[:120]}
    return out


def main():
    global LIVE_PRODUCER, SETTLE_SECONDS
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--settle-seconds", type=float, default=SETTLE_SECONDS,
                    help="untimed period of the same launches before each warm-up, to reach the sustained clock")
    ap.add_argument("--only", default="", help="comma list of c1,c2,c3,c4,c5,moe_gemm,copy,mfma,library (c2 always runs)")
    ap.add_argument("--no-live-producer", action="store_true",
                    help="skip the AG-GEMM legs in which a copy stream releases the flags while the GEMM spins: a "
                    "counter-collecting profiler serialises dispatches, so the producer could never run beside it")
    ap.add_argument("--static-schedule", action="store_true",
                    help="gated GEMMs walk their tiles in the static chunk-major order instead of in arrival order "
                    "(the library's TDIST_DEBUG_GEMM_SCHEDULE switch): the comparison leg of the overlap figures")
    args = ap.parse_args()
    LIVE_PRODUCER = not args.no_live_producer
    SETTLE_SECONDS = args.settle_seconds
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        log("bench.py: this build measures one GPU's share of the path; --gpus %d is not supported (every GPU box "
            "here has one GPU and the path has no cross-GPU step in it)" % args.gpus)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        log("bench.py needs a GPU")
        sys.exit(1)
    from triton_dist import _lib
    _lib.check(_lib.load().tdist_init())
    if args.static_schedule:
        _lib.check(_lib.load().tdist_debug_set(_lib.TDIST_DEBUG_GEMM_SCHEDULE, 0))
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    want = set(x for x in args.only.split(",") if x) or {"c1", "c2", "c3", "c4", "c5", "moe_gemm", "copy", "mfma", "library"}

    step_s, gemm_roof, red_roof, cpu, err = bench_c2(dev, args.steps, args.warmup)
    log("c2 step %.1f us, gemm %s, reduce %s" % (step_s * 1e6, gemm_roof, red_roof))
    kernels = {"c2_gemm_rs_scatter_gemm_bf16": dict(gemm_roof), "c2_reduce_slices_bf16": red_roof}
    if "c1" in want:
        kernels["c1_ag_gemm_bf16_gated"] = bench_c1(dev, args.steps, args.warmup)
        log("c1", kernels["c1_ag_gemm_bf16_gated"])
    if "c3" in want:
        kernels["c3_ag_gemm_fp8_gated"] = bench_c3(dev, args.steps, args.warmup)
        log("c3", kernels["c3_ag_gemm_fp8_gated"])
    if "c4" in want:
        d, c = bench_c4(dev, args.steps, args.warmup)
        kernels["c4_moe_dispatch_fp8"], kernels["c4_moe_combine"] = d, c
        log("c4", d, c)
    if "c5" in want:
        kernels["c5_decode_split_kv_bf16"], kernels["c5_decode_32splits"], kernels["c5_decode_page1"] = bench_c5(dev, args.steps, args.warmup)
        log("c5", kernels["c5_decode_split_kv_bf16"], kernels["c5_decode_32splits"], kernels["c5_decode_page1"])
    if "moe_gemm" in want:
        kernels["ag_group_gemm_bf16_mixtral_8x7b_tp8"] = bench_group_gemm(dev, args.steps, args.warmup)
        log("moe_gemm", kernels["ag_group_gemm_bf16_mixtral_8x7b_tp8"])
    if "copy" in want:
        kernels["copy_1GiB_yardstick"] = bench_copy(dev, args.steps, args.warmup)
        log("copy", kernels["copy_1GiB_yardstick"])

    if "mfma" in want:
        kernels["mfma_only_rate_yardstick"] = bench_mfma_ceiling(dev, args.steps, args.warmup)
        log("mfma", kernels["mfma_only_rate_yardstick"])
    if "library" in want:
        kernels["hipblaslt_matmul_c2_shape_yardstick"] = bench_library_gemm(dev, args.steps, args.warmup)
        log("library", kernels["hipblaslt_matmul_c2_shape_yardstick"])
        kernels["hipblaslt_scaled_mm_c3_shape_yardstick"] = bench_library_fp8_gemm(dev, args.steps, args.warmup)
        log("library fp8", kernels["hipblaslt_scaled_mm_c3_shape_yardstick"])

    flops = 2.0 * 8192 * 8192 * 3584
    line = {
        "metric": METRIC,
        "value": round(flops / step_s / 1e12, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(step_s * 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "GEMM-RS one-rank share, Llama-70B TP=8 MLP-down: A[8192,3584] x B[3584,8192] bf16 "
                               "scatter-epilogue GEMM + fp32 sum of 8 partial slices [1024,8192] (BASELINE configs[1])",
                   "rank": 0, "world_size": 8, "max_rel_err_vs_fp32": float("%.3g" % err)},
        "roofline": gemm_roof,
        "cpu_baseline": cpu,
        "kernels": kernels,
    }
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
