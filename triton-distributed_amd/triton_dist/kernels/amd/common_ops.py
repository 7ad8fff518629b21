"""Stream-ordered flag helpers for one GPU.

Mirrors the host-side part of the reference's kernels/amd/common_ops.py:76-112 (``wait_eq`` /
``set_signal``) and :66-73 (``barrier_all_on_stream``). The device-side spin (``wait_eq_sys``, :39-46)
lives inside the gated GEMM kernel. With a single GPU there is no peer to rendezvous with, so the
cross-rank barrier is a no-op that only keeps stream order.
"""
import torch

from triton_dist import _lib


def set_signal(ptr: int, val: int, stream: torch.cuda.Stream, require_i64=False):
    """Stores ``val`` into the int32 flag at device address ``ptr``, ordered on ``stream``
    (reference: hipStreamWriteValue32, kernels/amd/common_ops.py:97-112)."""
    if require_i64:
        raise NotImplementedError("64-bit flags are only used by the reference's inter-node path")
    _lib.call("tdist_flag_set", ptr, int(val), stream.cuda_stream)


def fill_flags(flags: torch.Tensor, value: int, stream: torch.cuda.Stream = None):
    """Stream-ordered ``flags.fill_(value)`` for an int32 flag tensor, by a small kernel (safe to capture
    into a HIP graph, unlike a memset node)."""
    assert flags.dtype == torch.int32 and flags.is_contiguous()
    _lib.call("tdist_flag_fill", flags.data_ptr(), flags.numel(), int(value), _lib.stream_ptr(stream))


def barrier_all_on_stream(rank, num_ranks, sync_bufs_ptr, stream):
    """Cross-rank barrier of the reference (kernels/amd/common_ops.py:66-73). One GPU has nobody to wait
    for: the call only exists so that code written against the reference keeps running."""
    return None
