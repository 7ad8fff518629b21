"""ctypes binding of libtdist_hip.so — one prototype per declaration in include/tdist.h."""
import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int64, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "_lib", "libtdist_hip.so")

TDIST_OK = 0
TDIST_ERR_INVALID = -1
TDIST_ERR_UNSUPPORTED = -2
TDIST_ERR_LAUNCH = -3
TDIST_ERR_TIMEOUT = -4
TDIST_ERR_WORKSPACE = -5
TDIST_ERR_DEVICE = -6

TDIST_BF16 = 0
TDIST_F16 = 1
TDIST_F8E4M3 = 2
TDIST_F32 = 3

# tdist_debug_key (include/tdist.h): test and measurement switches, -1 = the library decides
TDIST_DEBUG_GEMM_TILE = 0
TDIST_DEBUG_GEMM_SPLIT_K = 1
TDIST_DEBUG_GEMM_SK_COHERENT = 2
TDIST_DEBUG_GEMM_SCHEDULE = 3
TDIST_DEBUG_DECODE_WAVE_HEADS = 4
TDIST_DEBUG_DECODE_SPLITS_PER_TEAM = 5
TDIST_DEBUG_MOE_INDEX_FORM = 6

_P = c_void_p
_I = c_int
_L = c_int64
_F = c_float

# name -> (restype, argtypes); mirrors include/tdist.h in order
PROTOTYPES = {
    "tdist_version": (_I, []),
    "tdist_last_error_string": (c_char_p, []),
    "tdist_init": (_I, []),
    "tdist_num_cus": (_I, []),
    "tdist_debug_set": (_I, [_I, _I]),
    "tdist_debug_get": (_I, [_I]),
    "tdist_gemm_chunk_gated_bf16": (_I, [_P, _L, _P, _L, _I, _I, _P, _L, _P, _L, _I, _I, _I, _P, _I, _I, _P, _I, _I, _I, _P, _I, _P, _L, _P]),
    "tdist_gemm_chunk_gated_f16": (_I, [_P, _L, _P, _L, _I, _I, _P, _L, _P, _L, _I, _I, _I, _P, _I, _I, _P, _I, _I, _I, _P, _I, _P, _L, _P]),
    "tdist_gemm_chunk_gated_fp8e4m3": (_I, [_P, _L, _P, _L, _I, _I, _P, _L, _P, _L, _I, _I, _I, _P, _P, _P, _I, _I, _P, _I, _I, _I, _P, _I, _P, _L, _P]),
    "tdist_producer_push_chunk": (_I, [_P, _P, _L, _P, _P, _I, _P]),
    "tdist_producer_push_peers": (_I, [_P, _P, _I, _I, _L, _L, _P, _I, _P, _P, _P, _L, ctypes.c_uint32, _L, _I, _P]),
    "tdist_producer_mark": (_I, [_P, _P]),
    "tdist_producer_wait_until": (_I, [_P, _L, _P]),
    "tdist_flag_set": (_I, [_P, _I, _P]),
    "tdist_status_retire": (_I, [_P, _P, _P]),
    "tdist_flag_fill": (_I, [_P, _I, _I, _P]),
    "tdist_gemm_rs_scatter_bf16": (_I, [_P, _L, _P, _L, _P, _L, _I, _I, _I, _I, _I, _P, _L, _P]),
    "tdist_gemm_rs_scatter_f16": (_I, [_P, _L, _P, _L, _P, _L, _I, _I, _I, _I, _I, _P, _L, _P]),
    "tdist_gemm_rs_scatter_fp8e4m3": (_I, [_P, _L, _P, _L, _P, _L, _I, _I, _I, _P, _P, _I, _I, _P, _L, _P]),
    "tdist_reduce_slices": (_I, [_P, _L, _I, _I, _L, _P, _I, _P]),
    "tdist_moe_workspace_bytes": (_L, [_L, _I]),
    "tdist_moe_splits_cumsum": (_I, [_P, _L, _I, _P, _P, _P, _L, _P]),
    "tdist_moe_scatter_index": (_I, [_P, _L, _I, _I, _P, _P, _P, _P, _P, _P, _L, _P]),
    "tdist_moe_scatter_index_static": (_I, [_P, _L, _I, _I, _P, _P, _P, _P, _P, _P]),
    "tdist_moe_dispatch": (_I, [_P, _L, _P, _P, _P, _L, _I, _I, _I, _P, _P, _P, _P]),
    "tdist_moe_dispatch_tokens": (_I, [_P, _L, _P, _P, _I, _P, _L, _I, _I, _I, _P, _P, _P, _P]),
    "tdist_moe_dispatch_tokens_from_ids": (_I, [_P, _L, _P, _P, _I, _L, _I, _I, _I, _P, _P, _P, _P, _P, _P, _P, _P]),
    "tdist_moe_post_process": (_I, [_P, _L, _P, _P, _L, _I, _I, _I, _P, _P, _P]),
    "tdist_moe_combine": (_I, [_P, _I, _P, _P, _P, _P, _L, _I, _I, _I, _I, _I, _I, _P, _P]),
    "tdist_quant_e4m3_groups": (_I, [_P, _L, _I, _I, _P, _P, _P]),
    "tdist_moe_dispatch_tokens_quant": (_I, [_P, _I, _I, _P, _I, _P, _L, _I, _I, _I, _P, _P, _P, _P]),
    "tdist_moe_align_workspace_bytes": (_L, [_L, _I, _I]),
    "tdist_moe_align_block_size": (_I, [_P, _I, _L, _I, _I, _L, _I, _P, _L, _P, _P, _P, _P, _P, _L, _P]),
    "tdist_group_gemm_gated_bf16": (_I, [_P, _L, _P, _L, _I, _I, _P, _L, _L, _P, _L, _I, _I, _I, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _P, _I, _I, _I, _P, _I, _P, _L, _P]),
    "tdist_group_gemm_gated_f16": (_I, [_P, _L, _P, _L, _I, _I, _P, _L, _L, _P, _L, _I, _I, _I, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _P, _I, _I, _I, _P, _I, _P, _L, _P]),
    "tdist_group_gemm_gated_fp8e4m3": (_I, [_P, _L, _P, _L, _I, _I, _P, _L, _L, _P, _L, _I, _I, _I, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _P, _I, _I, _I, _P, _I, _P, _L, _P]),
    "tdist_gemm_split_k_workspace_bytes": (_L, []),
    "tdist_decode_split_kv": (_I, [_P, _P, _P, _P, _P, _F, _F, _P, _P, _I, _I, _I, _I, _I, _I, _I,
                                   _L, _L, _L, _L, _L, _L, _L, _L, _L, _I, _P]),
    "tdist_decode_fused_counters": (_L, [_I, _I, _I]),
    "tdist_decode_fused": (_I, [_P, _P, _P, _P, _P, _F, _F, _P, _P, _I, _I, _I, _I, _I, _I, _I,
                                _L, _L, _L, _L, _L, _L, _L, _L, _L, _I, _P, _L, _P, _I, _L, _L, _P, _P]),
    "tdist_decode_combine": (_I, [_P, _I, _P, _I, _I, _P, _I, _I, _I, _L, _L, _L, _L, _L, _L, _P, _I, _L, _L, _P, _P]),
}

# libtdist_bench.so (include/tdist_bench.h): measurement helpers for bench.py, kept out of the product library
BENCH_LIB_PATH = os.path.join(_HERE, "_lib", "libtdist_bench.so")
BENCH_PROTOTYPES = {
    "tdist_bench_last_error_string": (c_char_p, []),
    "tdist_copy_bytes": (_I, [_P, _P, _L, _P]),
    "tdist_fill_bytes": (_I, [_P, _L, _P]),
    "tdist_read_bytes": (_I, [_P, _L, _P, _P]),
    "tdist_mfma_rate_probe": (_I, [_I, _I, _I, _P, _P]),
    "tdist_mfma_rate_probe_16row": (_I, [_I, _I, _I, _P, _P]),
}


class TdistError(RuntimeError):
    def __init__(self, code, message):
        super().__init__("libtdist_hip error %d: %s" % (code, message))
        self.code = code


_lib = None


def load():
    """Loads the shared library (once). Raises if it has not been built: there is no fallback path."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            "libtdist_hip.so is missing at %s — build it with `python triton-distributed_amd/build.py` "
            "(hipcc, gfx950). The ops have no CPU or PyTorch fallback." % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in PROTOTYPES.items():
        fn = getattr(lib, name)  # AttributeError here means header and library disagree
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def last_error():
    msg = load().tdist_last_error_string()
    return msg.decode("utf-8", "replace") if msg else ""


def check(code):
    if code != TDIST_OK:
        raise TdistError(code, last_error())


def call(name, *args):
    """Calls an entry point that returns a tdist_status and raises TdistError on failure."""
    check(getattr(load(), name)(*args))


class debug_switch:
    """``with debug_switch(key, value): ...`` sets one of the library's test and measurement switches
    (tdist_debug_set) and puts the previous value back on exit."""

    def __init__(self, key, value):
        self.key, self.value = key, value

    def __enter__(self):
        self.old = load().tdist_debug_get(self.key)
        check(load().tdist_debug_set(self.key, -1 if self.value is None else int(self.value)))
        return self

    def __exit__(self, *exc):
        check(load().tdist_debug_set(self.key, self.old))
        return False


def ptr(t):
    """Device pointer of a tensor (None → NULL)."""
    return None if t is None else t.data_ptr()


def stream_ptr(stream=None):
    import torch
    s = torch.cuda.current_stream() if stream is None else stream
    return s.cuda_stream


def dtype_code(dtype):
    import torch
    if dtype == torch.bfloat16:
        return TDIST_BF16
    if dtype == torch.float16:
        return TDIST_F16
    if dtype == torch.float8_e4m3fn:
        return TDIST_F8E4M3
    if dtype == torch.float32:
        return TDIST_F32
    raise TypeError("unsupported dtype %s" % dtype)


_bench_lib = None


def load_bench():
    """Loads libtdist_bench.so (once): the copy and MFMA-rate yardsticks of bench.py."""
    global _bench_lib
    if _bench_lib is None:
        if not os.path.exists(BENCH_LIB_PATH):
            raise RuntimeError("libtdist_bench.so is missing at %s: build it with `python triton-distributed_amd/build.py`"
                               % BENCH_LIB_PATH)
        lib = ctypes.CDLL(BENCH_LIB_PATH)
        for name, (restype, argtypes) in BENCH_PROTOTYPES.items():
            fn = getattr(lib, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _bench_lib = lib
    return _bench_lib


def bench_call(name, *args):
    lib = load_bench()
    code = getattr(lib, name)(*args)
    if code != TDIST_OK:
        msg = lib.tdist_bench_last_error_string()
        raise TdistError(code, msg.decode("utf-8", "replace") if msg else "")


def new_split_k_workspace(device=None):
    """A zero-filled workspace for the GEMM entry points' sk_workspace argument (tdist_gemm_split_k_workspace_bytes()
    bytes: 64 MiB + 12 KiB on MI355X). Every context owns one: launches that share a workspace must be ordered, and
    contexts may run on streams of their own. Returns a uint8 tensor."""
    import torch
    dev = None if device is None else torch.device(device).index
    if dev is None:   # (no device, or "cuda" without an index: the current one)
        dev = torch.cuda.current_device()
    with torch.cuda.device(dev):
        nbytes = load().tdist_gemm_split_k_workspace_bytes()
        if nbytes <= 0:
            raise TdistError(TDIST_ERR_DEVICE, "split-K workspace: device %d is not gfx950" % dev)
        return torch.zeros(nbytes, dtype=torch.uint8, device="cuda:%d" % dev)


_zero_scratch = {}   # (device index, stream handle) -> uint8 tensor whose control words the kernels keep at zero


def zeroed_scratch(nbytes, device):
    """A scratch tensor of at least ``nbytes`` for entry points whose workspace starts with control words that must be
    zero on first use and are left zero by every call (the MoE index build, the align / sort): allocated zero-filled
    once per (device, current stream) and handed out again on later calls, so a call allocates nothing. Launches on
    one stream are ordered and may share it; launches on different streams never do."""
    import torch
    device = torch.device(device)
    if device.index is None:
        device = torch.device("cuda", torch.cuda.current_device())
    key = (device.index, torch.cuda.current_stream(device).cuda_stream)
    buf = _zero_scratch.get(key)
    if buf is None or buf.numel() < nbytes:
        buf = torch.zeros(max(int(nbytes), 1 << 20), dtype=torch.uint8, device=device)
        _zero_scratch[key] = buf
    return buf


def workspace_args(ws):
    """(pointer, bytes) of an optional workspace tensor for the sk_workspace / sk_workspace_bytes arguments."""
    return (None, 0) if ws is None else (ws.data_ptr(), ws.numel() * ws.element_size())


def require_cuda(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("tdist ops run on the GPU only; got a %s tensor" % t.device)
