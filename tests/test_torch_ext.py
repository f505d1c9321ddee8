"""The PyTorch extension over the C ABI (csrc/torch_ext.cpp): it loads, registers every operator under
torch.ops.spargeattn_amd with a schema, and its meta kernels give the shapes and dtypes of the real ones.  No GPU."""
import os

import pytest
import torch

from spargeattn_amd import _lib

pytestmark = pytest.mark.skipif(not os.path.exists(_lib.TORCH_EXT_PATH), reason="extension not built (python -m spargeattn_amd.build)")

OPS = ["km_mean", "pool_sim_quant", "block_select", "map_to_lut", "v_quant_fp8", "v_tiles_f16", "block_sparse_attn",
       "block_sparse_attn_f16v", "dense_attn_f16", "selftest_fp8_pack", "selftest_division"]


def test_operators_are_registered_with_schemas():
    ops = _lib.load_torch_ext()
    for name in OPS:
        op = getattr(ops, name)
        schema = str(op.default._schema)
        assert schema.startswith(f"spargeattn_amd::{name}("), schema
    # the attention entry points mutate their output argument and say so
    assert "Tensor(a!) out" in str(ops.block_sparse_attn.default._schema)
    assert "int qk_quant_gran" in str(ops.block_sparse_attn_f16v.default._schema)


def test_meta_kernels_give_the_output_shapes():
    ops = _lib.load_torch_ext()
    B, H, Hkv, N, Nk, D = 2, 4, 2, 300, 500, 128
    nq, nk = (N + 127) // 128, (Nk + 63) // 64
    m = lambda *s, dtype=torch.bfloat16: torch.empty(*s, dtype=dtype, device="meta")
    q, k = m(B, H, N, D), m(B, Hkv, Nk, D)
    assert ops.km_mean(k).shape == (B, Hkv, 1, D) and ops.km_mean(k).dtype == torch.bfloat16
    pool, sim, xq, scale = ops.pool_sim_quant(q, None, 128, m(H, dtype=torch.float32), True, 32)
    assert (pool.shape, sim.shape, xq.shape, scale.shape) == ((B, H, nq, D), (B, H, nq), (B, H, N, D), (B, H, nq * 4))
    assert (sim.dtype, xq.dtype, scale.dtype) == (torch.bool, torch.int8, torch.float32)
    pool, sim, kq, scale = ops.pool_sim_quant(k, ops.km_mean(k), 64, None, False, 64)
    assert pool.numel() == 0 and sim.numel() == 0 and scale.shape == (B, Hkv, nk) and kq.shape == k.shape
    lut, valid, bmap = ops.block_select(m(B, H, nq, D), m(B, H, nq, dtype=torch.bool), m(B, Hkv, nk, D),
                                        m(B, Hkv, nk, dtype=torch.bool), m(H, dtype=torch.float32), None, True, False, True)
    assert (lut.shape, valid.shape, bmap.shape) == ((B, H, nq, nk), (B, H, nq), (B, H, nq, nk)) and lut.dtype == torch.int32
    lut2, valid2 = ops.map_to_lut(m(B, H, nq, nk, dtype=torch.int64))
    assert lut2.shape == lut.shape and valid2.shape == valid.shape
    v8, vs = ops.v_quant_fp8(m(B, Hkv, Nk, D))
    assert v8.shape == (B, Hkv, nk, D, 64) and v8.dtype == torch.uint8 and vs.shape == (B, Hkv, D)
    assert ops.v_tiles_f16(m(B, Hkv, Nk, D)).dtype == torch.float16
    f32 = torch.float32
    pvc = ops.block_sparse_attn(xq, m(B, Hkv, Nk, D, dtype=torch.int8), v8, m(B, H, N, D), lut, valid, m(H, dtype=f32),
                                m(B, H, nq * 4, dtype=f32), m(B, Hkv, nk, dtype=f32), vs, 0.1, False, 2, 1, True)
    assert pvc.shape == (B, H, nq * 4) and pvc.dtype == torch.int32
    with pytest.raises(ValueError, match="must divide the block size"):
        ops.pool_sim_quant(q, None, 128, None, False, 48)


def test_cpu_tensors_have_no_kernel():
    """There is no CPU implementation behind the operators: a CPU tensor fails in the dispatcher."""
    ops = _lib.load_torch_ext()
    with pytest.raises((NotImplementedError, RuntimeError)):
        ops.km_mean(torch.zeros(1, 1, 128, 64, dtype=torch.float16))


def test_binding_selector():
    assert _lib.get_binding() in ("ctypes", "torch")
    before = _lib.get_binding()
    with pytest.raises(ValueError):
        _lib.set_binding("pybind")
    _lib.set_binding("torch")
    assert _lib._torch() is _lib.load_torch_ext()
    _lib.set_binding("ctypes")
    assert _lib._torch() is None
    _lib.set_binding(before)
