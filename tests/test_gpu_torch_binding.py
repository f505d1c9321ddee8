"""The PyTorch-extension binding (torch.ops.spargeattn_amd.*) against the ctypes binding: both sit on the same C ABI,
so every stage gives the same bits, the operators give the same tensors, and the error classes agree.  The whole GPU
suite runs through either binding with SPARGEATTN_AMD_BINDING=torch; this file keeps the comparison in the default run.
"""
import numpy as np
import pytest
import torch

import spargeattn_amd as sa
from oracle import api as oapi
from spargeattn_amd import _lib, utils
from gpu_common import tag_of, to_np, rand_T
from test_gpu_attention import _check_out

pytestmark = pytest.mark.gpu


@pytest.fixture
def both():
    """Runs a callable under each binding and returns the two results."""
    before = _lib.get_binding()

    def run(fn):
        out = {}
        for name in ("ctypes", "torch"):
            _lib.set_binding(name)
            out[name] = fn()
        return out["ctypes"], out["torch"]
    yield run
    _lib.set_binding(before)


def _same(a, b):
    if a is None or b is None:
        return a is None and b is None
    if isinstance(a, (tuple, list)):
        return len(a) == len(b) and all(_same(x, y) for x, y in zip(a, b))
    return a.dtype == b.dtype and a.shape == b.shape and torch.equal(a.view(torch.uint8) if a.dtype == torch.bool else a,
                                                                     b.view(torch.uint8) if b.dtype == torch.bool else b)


@pytest.mark.parametrize("dtype,D", [(torch.bfloat16, 128), (torch.float16, 64)])
def test_every_stage_gives_the_same_bits_through_both_bindings(both, dtype, D):
    B, H, Hkv, N, Nk = 1, 4, 2, 640, 900
    q = rand_T((B, H, N, D), dtype, 1)
    k = rand_T((B, Hkv, Nk, D), dtype, 2, shift=0.3)
    v = rand_T((B, Hkv, Nk, D), dtype, 3)
    thr = torch.full((H,), 0.3, dtype=torch.float32, device="cuda")
    km_c, km_t = both(lambda: _lib.km_mean(k))
    assert _same(km_c, km_t)
    for qr in (128, 32):
        assert _same(*both(lambda: _lib.pool_sim_quant(q, None, 128, thr, quant_rows=qr)))
    assert _same(*both(lambda: _lib.pool_sim_quant(k, km_c, 64, thr[:Hkv].contiguous())))
    assert _same(*both(lambda: _lib.pool_sim_quant(k, km_c, 64, with_pool=False)))
    nhd = q.transpose(1, 2).contiguous().transpose(1, 2)                       # strided input
    assert _same(*both(lambda: _lib.pool_sim_quant(nhd, None, 128, thr)))
    pq, sq, q8, qs = _lib.pool_sim_quant(q, None, 128, thr)
    pk, sk, k8, ks = _lib.pool_sim_quant(k, km_c, 64, thr[:Hkv].contiguous())
    topk = torch.linspace(0.3, 0.8, H, device="cuda")
    for kw in (dict(topk=topk, is_causal=True, return_map=True), dict(cdfthreshd=topk, attention_sink=True)):
        assert _same(*both(lambda: _lib.block_select(pq, sq, pk, sk, **kw)))
    lut, valid, bmap = _lib.block_select(pq, sq, pk, sk, topk=topk, return_map=True)
    assert _same(*both(lambda: _lib.map_to_lut(bmap.to(torch.int32))))
    assert _same(*both(lambda: _lib.v_quant_fp8(v)))
    assert _same(*both(lambda: _lib.v_tiles_f16_swizzled(v)))
    v8, vs = _lib.v_quant_fp8(v)
    vt = _lib.v_tiles_f16_swizzled(v)
    pvt = torch.full((H,), 2.0, dtype=torch.float32, device="cuda")

    def attn(f16v):
        out = torch.zeros((B, H, N, D), dtype=dtype, device="cuda")
        if f16v:
            pvc = _lib.block_sparse_attn_f16v(q8, k8, vt, out, lut, valid, pvt, qs, ks, D ** -0.5, return_pv_count=True)
        else:
            pvc = _lib.block_sparse_attn(q8, k8, v8, out, lut, valid, pvt, qs, ks, vs, D ** -0.5, return_pv_count=True,
                                         pv_mode=_lib.PV_PER_WARP)
        return out, pvc
    assert _same(*both(lambda: attn(False)))
    assert _same(*both(lambda: attn(True)))
    x = torch.randn(4096, device="cuda") * 300
    assert _same(*both(lambda: _lib.selftest_fp8_pack(x)))
    c, t = both(lambda: _lib.selftest_division(64, seed=3))
    assert c == t and c[1] == 0


def test_operators_through_the_torch_binding_match_the_oracle(both):
    dtype, B, H, N, D = torch.bfloat16, 1, 2, 1024, 128
    q, k, v = rand_T((B, H, N, D), dtype, 11), rand_T((B, H, N, D), dtype, 12, shift=0.4), rand_T((B, H, N, D), dtype, 13)
    res = oapi.spas_sage2_attn_meansim_topk(to_np(q), to_np(k), to_np(v), tag_of(dtype), is_causal=True, topk=0.5, qk_quant_gran=2)
    oc, ot = both(lambda: sa.spas_sage2_attn_meansim_topk_cuda(q, k, v, is_causal=True, topk=0.5, qk_quant_gran=2,
                                                                tensor_layout="HND"))
    assert torch.equal(oc, ot)
    _check_out(ot, res["out"])
    mask = torch.ones((B, H, 8, 16), dtype=torch.int32, device="cuda")
    assert _same(*both(lambda: sa.block_sparse_sage2_attn_cuda(q, k, v, mask_id=mask, pvthreshd=3.0)))
    assert _same(*both(lambda: sa.spas_sage_attn_meansim_cuda(q, k, v, simthreshd1=0.3, cdfthreshd=0.9)))
    qn, kn, vn = (t.transpose(1, 2).contiguous() for t in (q, k, v))
    assert _same(*both(lambda: sa.spas_sage2_attn_meansim_topk_cuda(qn, kn, vn, topk=0.5, tensor_layout="NHD")))


def test_error_classes_agree(both):
    q = rand_T((1, 2, 256, 64), torch.float16, 1)
    km = _lib.km_mean(q)

    def classes():
        seen = []
        for fn in (lambda: _lib.pool_sim_quant(q, km, 128, with_pool=False, quant_rows=32),      # ValueError from the C ABI
                   lambda: _lib.pool_sim_quant(q, None, 128, with_pool=False, quant_rows=48),    # ValueError before it
                   lambda: utils.get_vanilla_qk_quant(q, q, km, qk_quant_gran=3),
                   lambda: _lib.km_mean(q[..., ::2])):                                            # RuntimeError: layout
            try:
                fn()
                seen.append(None)
            except Exception as e:      # noqa: BLE001
                seen.append(type(e))
        return seen
    c, t = both(classes)
    assert c == t == [ValueError, ValueError, ValueError, RuntimeError]
    # direct use of the registered operators: the checks of the shim itself
    ops = _lib.load_torch_ext()
    with pytest.raises(RuntimeError, match="must be contiguous"):
        ops.block_select(q, q[..., 0].bool(), q, q[..., 0].bool(), None, None, False, False, False) if False else \
            ops.map_to_lut(torch.ones((1, 2, 4, 8), device="cuda").transpose(2, 3))
    with pytest.raises(ValueError, match="Only one of cdfthreshd and topk"):
        pq, sq, _, _ = _lib.pool_sim_quant(q, None, 128, torch.zeros(2, device="cuda"))
        pk, sk, _, _ = _lib.pool_sim_quant(q, km, 64, torch.zeros(2, device="cuda"))
        ops.block_select(pq, sq, pk, sk, None, None, False, False, False)
