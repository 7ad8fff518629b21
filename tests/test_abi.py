"""The C-ABI library loads without a GPU and exports exactly what include/tdist.h declares; argument
validation that needs no device returns error codes instead of aborting. No compute call is made here."""
import ctypes
import os
import re

import pytest

from triton_dist import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "tdist.h")
BENCH_HEADER = os.path.join(ROOT, "include", "tdist_bench.h")


def header_functions(header=HEADER):
    text = open(header).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tdist_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_functions():
    names = header_functions()
    assert "tdist_gemm_chunk_gated_bf16" in names and "tdist_decode_split_kv" in names
    assert len(names) >= 20


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    for name in header_functions():
        assert hasattr(lib, name), "libtdist_hip.so does not export %s" % name


def test_python_prototypes_cover_header():
    assert sorted(_lib.PROTOTYPES) == header_functions()


def test_bench_library_is_separate_and_complete():
    """The measurement helpers live in libtdist_bench.so: declared in tdist_bench.h, exported there, and absent from
    the product library."""
    names = header_functions(BENCH_HEADER)
    assert sorted(_lib.BENCH_PROTOTYPES) == names
    bench, product = _lib.load_bench(), _lib.load()
    for name in names:
        assert hasattr(bench, name), "libtdist_bench.so does not export %s" % name
        assert not hasattr(product, name), "libtdist_hip.so still exports %s" % name
    assert bench.tdist_copy_bytes(None, None, 16, None) == _lib.TDIST_ERR_INVALID


def test_prototype_arity_matches_header():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    for name, (_, argtypes) in _lib.PROTOTYPES.items():
        m = re.search(r"\b%s\s*\((.*?)\)\s*;" % name, text, flags=re.S)
        assert m, name
        params = m.group(1).strip()
        n = 0 if params in ("", "void") else params.count(",") + 1
        assert n == len(argtypes), "%s: header has %d parameters, binding %d" % (name, n, len(argtypes))


def test_version_and_error_string():
    lib = _lib.load()
    assert lib.tdist_version() >= 100
    assert isinstance(_lib.last_error(), str)


def test_null_pointers_are_rejected_without_touching_the_gpu():
    lib = _lib.load()
    assert lib.tdist_reduce_slices(None, 0, 8, 0, 16, None, _lib.TDIST_BF16, None) == _lib.TDIST_ERR_INVALID
    assert "null" in _lib.last_error()
    assert lib.tdist_flag_set(None, 1, None) == _lib.TDIST_ERR_INVALID
    assert lib.tdist_moe_dispatch(None, 16, None, None, None, 0, 1, 1, 1, None, None, None, None) == _lib.TDIST_ERR_INVALID
    buf = ctypes.create_string_buffer(64)
    p = ctypes.addressof(buf)
    # bad sizes are caught before any launch
    assert lib.tdist_reduce_slices(p, 0, 0, 0, 16, p, _lib.TDIST_BF16, None) == _lib.TDIST_ERR_INVALID
    assert lib.tdist_reduce_slices(p, 0, 4, 7, 16, p, _lib.TDIST_BF16, None) == _lib.TDIST_ERR_INVALID
    assert lib.tdist_reduce_slices(p, 0, 4, 0, 16, p, _lib.TDIST_F8E4M3, None) == _lib.TDIST_ERR_UNSUPPORTED
    assert lib.tdist_decode_split_kv(p, p, p, p, p, 1.0, 0.0, p, p, 1, 6, 4, 128, 128, 1, 4, 0, 0, 0, 0, 0, 0, 0, 0, 0,
                                     _lib.TDIST_BF16, None) == _lib.TDIST_ERR_INVALID  # 6 % 4 != 0
    assert lib.tdist_decode_split_kv(p, p, p, p, p, 1.0, 0.0, p, p, 1, 8, 4, 100, 100, 1, 4, 0, 0, 0, 0, 0, 0, 0, 0, 0,
                                     _lib.TDIST_BF16, None) == _lib.TDIST_ERR_UNSUPPORTED  # head_dim 100: no multiple of 8
    assert lib.tdist_decode_split_kv(p, p, p, p, p, 1.0, 0.0, p, p, 1, 8, 4, 96, 64, 1, 4, 0, 0, 0, 0, 0, 0, 0, 0, 0,
                                     _lib.TDIST_BF16, None) == _lib.TDIST_ERR_UNSUPPORTED  # 96 goes with Dv = 96
    assert lib.tdist_decode_split_kv(p, p, p, p, p, 1.0, 0.0, p, p, 1, 8, 4, 192, 64, 1, 4, 0, 0, 0, 0, 0, 0, 0, 0, 0,
                                     _lib.TDIST_BF16, None) == _lib.TDIST_ERR_UNSUPPORTED  # 192 goes with Dv = 128 or 192
    # the fused launch: 40 query heads over 2 kv heads = 2 blocks of 16 heads per kv head and sequence
    assert lib.tdist_decode_fused_counters(3, 40, 2) == 3 * 2 * 2
    assert lib.tdist_decode_fused_counters(3, 40, 3) == -1
    fused = lambda n_counters, out: lib.tdist_decode_fused(
        p, p, p, p, p, 1.0, 0.0, p, p, 3, 40, 2, 128, 128, 1, 4, 0, 0, 0, 0, 0, 0, 0, 0, 0, _lib.TDIST_BF16,
        p, n_counters, out, _lib.TDIST_BF16, 0, 0, None, None)
    assert fused(11, p) == _lib.TDIST_ERR_WORKSPACE and "counters" in _lib.last_error()
    assert fused(12, None) == _lib.TDIST_ERR_INVALID
    assert lib.tdist_producer_mark(None, None) == _lib.TDIST_ERR_INVALID
    assert lib.tdist_producer_wait_until(None, 1000, None) == _lib.TDIST_ERR_INVALID
    assert lib.tdist_producer_wait_until(p, -1, None) == _lib.TDIST_ERR_INVALID
    assert lib.tdist_producer_wait_until(p, 100000001, None) == _lib.TDIST_ERR_INVALID and "100 ms" in _lib.last_error()
    assert lib.tdist_moe_workspace_bytes(32768, 256) == (128 + 1) * 256 * 4 + 256


def test_debug_switches_default_to_automatic_and_ignore_the_environment(monkeypatch):
    """The library's test and measurement switches: -1 (the library decides) until tdist_debug_set says otherwise,
    a negative value puts a key back, unknown keys are rejected, and nothing is read from the environment."""
    lib = _lib.load()
    for name in ("TDIST_GEMM_TILE", "TDIST_GEMM_SPLIT_K", "TDIST_DECODE_WAVE_HEADS", "TDIST_MOE_INDEX_LAUNCHES"):
        monkeypatch.setenv(name, "2")
    keys = [_lib.TDIST_DEBUG_GEMM_TILE, _lib.TDIST_DEBUG_GEMM_SPLIT_K, _lib.TDIST_DEBUG_GEMM_SK_COHERENT,
            _lib.TDIST_DEBUG_GEMM_SCHEDULE, _lib.TDIST_DEBUG_DECODE_WAVE_HEADS, _lib.TDIST_DEBUG_DECODE_SPLITS_PER_TEAM,
            _lib.TDIST_DEBUG_MOE_INDEX_FORM]
    assert [lib.tdist_debug_get(k) for k in keys] == [-1] * len(keys)
    with _lib.debug_switch(_lib.TDIST_DEBUG_GEMM_TILE, 3):
        assert lib.tdist_debug_get(_lib.TDIST_DEBUG_GEMM_TILE) == 3
        assert lib.tdist_debug_get(_lib.TDIST_DEBUG_GEMM_SPLIT_K) == -1
    assert lib.tdist_debug_get(_lib.TDIST_DEBUG_GEMM_TILE) == -1
    assert lib.tdist_debug_set(_lib.TDIST_DEBUG_GEMM_TILE, -7) == 0 and lib.tdist_debug_get(_lib.TDIST_DEBUG_GEMM_TILE) == -1
    assert lib.tdist_debug_set(99, 1) == _lib.TDIST_ERR_INVALID and lib.tdist_debug_set(-1, 1) == _lib.TDIST_ERR_INVALID
    assert lib.tdist_debug_get(99) == -1
    # the header's key values are the binding's
    text = open(HEADER).read()
    for name in ("GEMM_TILE", "GEMM_SPLIT_K", "GEMM_SK_COHERENT", "GEMM_SCHEDULE", "DECODE_WAVE_HEADS",
                 "DECODE_SPLITS_PER_TEAM", "MOE_INDEX_FORM"):
        m = re.search(r"TDIST_DEBUG_%s\s*=\s*(\d+)" % name, text)
        assert m and int(m.group(1)) == getattr(_lib, "TDIST_DEBUG_" + name), name
    import glob
    for src in glob.glob(os.path.join(ROOT, "triton-distributed_amd", "csrc", "*")):
        assert "getenv" not in open(src).read(), "%s reads the environment" % src


def test_ops_fail_loudly_without_gpu():
    import torch
    if torch.cuda.is_available():
        pytest.skip("GPU present")
    from triton_dist.kernels.amd import create_gemm_rs_intra_node_context, moe_dispatch_preprocess
    with pytest.raises(RuntimeError):
        create_gemm_rs_intra_node_context(1024, 256, torch.bfloat16, 0, 8, None)
    with pytest.raises(RuntimeError):
        moe_dispatch_preprocess(torch.zeros((4, 2), dtype=torch.int32), 8)
