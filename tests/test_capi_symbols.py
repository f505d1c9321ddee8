"""The C-ABI library loads and exports exactly the entry points include/spargeattn_amd.h declares (no GPU needed)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "spargeattn_amd.h")
LIB = os.path.join(ROOT, "spargeattn_amd", "libspargeattn_amd.so")


def _declared():
    src = open(HEADER).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"\b(spg_[a-z0-9_]+)\s*\(", src)))


def test_header_declares_the_stages():
    names = _declared()
    for want in ("spg_km_mean", "spg_pool_sim_quant", "spg_block_select", "spg_map_to_lut", "spg_v_quant_fp8",
                 "spg_block_sparse_attn", "spg_block_sparse_attn_f16v", "spg_v_tiles_f16", "spg_dense_attn_f16", "spg_selftest_division", "spg_selftest_fp8_pack", "spg_last_error", "spg_version"):
        assert want in names


@pytest.mark.skipif(not os.path.exists(LIB), reason="library not built (python -m spargeattn_amd.build)")
def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(LIB)
    for name in _declared():
        assert hasattr(lib, name), name
    lib.spg_version.restype = ctypes.c_int
    assert lib.spg_version() >= 100


@pytest.mark.skipif(not os.path.exists(LIB), reason="library not built")
def test_binding_table_matches_header():
    from spargeattn_amd import _lib
    assert sorted(_lib.SIGNATURES) == _declared()
    # argument counts agree with the prototypes
    src = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    for name, (_, args) in _lib.SIGNATURES.items():
        m = re.search(r"\b" + name + r"\s*\(([^;]*?)\)\s*;", src, flags=re.S)
        assert m, name
        params = m.group(1).strip()
        n = 0 if params in ("", "void") else params.count(",") + 1
        assert n == len(args), (name, n, len(args))


@pytest.mark.skipif(not os.path.exists(LIB), reason="library not built")
def test_argument_errors_are_reported_without_a_gpu():
    """Validation happens on the host before any launch: status code + thread-local message."""
    from spargeattn_amd import _lib
    lib = _lib.load()
    rc = lib.spg_km_mean(None, None, None, None, 1, 1, 128, 96, 0, None)
    assert rc == _lib.SPG_ERR_UNSUPPORTED and b"head_dim" in lib.spg_last_error()
    rc = lib.spg_block_select(1, 1, 1, 1, None, None, 0, 0, 1, 1, None, 1, 1, 1, 1, 2, 64, 0, None)
    assert rc == _lib.SPG_ERR_INVALID and b"Only one of cdfthreshd and topk" in lib.spg_last_error()
    rc = lib.spg_block_select(1, 1, 1, 1, 1, None, 0, 0, 1, 1, None, 1, 6, 4, 1, 2, 64, 0, None)
    assert rc == _lib.SPG_ERR_INVALID and b"must be divisible by num_kv_heads" in lib.spg_last_error()
    rc = lib.spg_pool_sim_quant(None, None, None, None, None, None, None, None, 1, 1, 128, 64, 128, 128, 1, None)
    assert rc == _lib.SPG_ERR_INVALID and b"NULL" in lib.spg_last_error()
    # quantisation granularity: per block, or 32-row groups of a 128-row block without a mean
    rc = lib.spg_pool_sim_quant(1, None, None, None, None, 1, 1, None, 1, 1, 128, 64, 64, 32, 1, None)
    assert rc == _lib.SPG_ERR_UNSUPPORTED and b"quant_rows" in lib.spg_last_error()
    rc = lib.spg_pool_sim_quant(1, None, 1, None, None, 1, 1, None, 1, 1, 128, 64, 128, 32, 1, None)
    assert rc == _lib.SPG_ERR_UNSUPPORTED and b"quant_rows" in lib.spg_last_error()
    rc = lib.spg_v_quant_fp8(1, None, 1, 1, 1, 1, 128, 64, 7, None)
    assert rc == _lib.SPG_ERR_INVALID and b"dtype" in lib.spg_last_error()
    assert lib.spg_km_mean_workspace_bytes(1, 32, 32768, 128) > 0
    rc = lib.spg_block_sparse_attn(1, 1, 1, 1, None, 0, 1, 1, 1, 1, 1, 1, 1, 6, 4, 128, 128, 64, 0.125, 0, 1, 1, None, None)
    assert rc == _lib.SPG_ERR_INVALID and b"must be divisible by num_kv_heads" in lib.spg_last_error()
    rc = lib.spg_block_sparse_attn(1, 1, 1, 1, None, 0, 1, 1, 1, 1, 1, 1, 1, 4, 4, 128, 128, 64, 0.125, 0, 1, 3, None, None)
    assert rc == _lib.SPG_ERR_INVALID and b"pv_threshold_mode" in lib.spg_last_error()
    rc = lib.spg_block_sparse_attn(1, 1, 1, 1, None, 0, 1, 1, 1, 1, 1, 1, 1, 4, 4, 128, 0, 64, 0.125, 0, 1, 1, None, None)
    assert rc == _lib.SPG_ERR_INVALID and b"must be positive" in lib.spg_last_error()        # kv_len
    # qk_quant_gran: 1 and 2 are served, 3 (per thread) is refused as unsupported, anything else with the reference's
    # message (csrc/pytorch_extensions_utils.cuh:81-85)
    for fn, tail in ((lib.spg_block_sparse_attn, (1, 1, 1)), (lib.spg_block_sparse_attn_f16v, (1, 1))):
        head = (1, 1, 1, 1, None, 0, 1, 1, 1) + tail
        rc = fn(*head, 1, 4, 4, 128, 128, 64, 0.125, 0, 3, 1, None, None)
        assert rc == _lib.SPG_ERR_UNSUPPORTED and b"per thread" in lib.spg_last_error()
        rc = fn(*head, 1, 4, 4, 128, 128, 64, 0.125, 0, 0, 1, None, None)
        assert rc == _lib.SPG_ERR_INVALID and b"Unsupported qk_quant_gran: 0" in lib.spg_last_error()
    rc = lib.spg_selftest_fp8_pack(1, 1, 6, 1, None)
    assert rc == _lib.SPG_ERR_INVALID and b"multiple of 4" in lib.spg_last_error()
    # strides: {batch, head, row} in elements, positive multiples of 8, row stride >= head_dim
    import ctypes
    bad = (ctypes.c_int64 * 3)(128 * 64, 64, 60)
    rc = lib.spg_v_quant_fp8(1, bad, 1, 1, 1, 1, 128, 64, 0, None)
    assert rc == _lib.SPG_ERR_INVALID and b"multiple of 8" in lib.spg_last_error()
    bad = (ctypes.c_int64 * 3)(128 * 64, 128 * 64, 32)
    rc = lib.spg_km_mean(1, bad, 1, 1, 1, 1, 128, 64, 0, None)
    assert rc == _lib.SPG_ERR_INVALID and b"smaller than head_dim" in lib.spg_last_error()
