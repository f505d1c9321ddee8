"""GPU parity of the INT8-QK / FP16-PV path (spas_sage_attn_meansim[_topk]_cuda) against the oracle.

The fp16 V^T tiles are bit-exact; the attention output is compared by tolerance (cosine >= 0.999, relative L1 <= 1e-2
as for the FP8 path; measured about 1e-4, the residual being the reference-style fp16 rounding of P on both sides and
approximate exp2/rcp)."""
import numpy as np
import pytest
import torch

import spargeattn_amd as sa
from oracle import api as oapi, attention as oat
from spargeattn_amd import _lib, workloads as W
from gpu_common import tag_of, to_np, rand_T

pytestmark = pytest.mark.gpu


def _check(o_gpu, ref, cos_min=0.999, l1_max=1e-2):
    met = oat.precision_metric(to_np(o_gpu), ref)
    assert met["Cossim"] >= cos_min and met["L1"] <= l1_max, met
    return met


@pytest.mark.parametrize("dtype,D,N", [(torch.bfloat16, 128, 1024), (torch.float16, 64, 500), (torch.float32, 64, 256)])
def test_v_tiles_f16_bit_exact(dtype, D, N):
    v = rand_T((1, 3, N, D), torch.float32, 5, scale=3.0).to(dtype if dtype != torch.float32 else torch.float16)
    vt = _lib.v_tiles_f16_swizzled(v)
    nk = (N + 63) // 64
    assert vt.shape == (1, 3, nk, D, 64) and vt.dtype == torch.float16
    nat = _lib.v_tiles_f16_to_natural(vt)
    assert torch.equal(nat[:, :, :N], v.to(torch.float16)) and bool((nat[:, :, N:] == 0).all())


@pytest.mark.parametrize("dtype,D,N,causal", [(torch.bfloat16, 128, 1024, False), (torch.float16, 64, 1024, True),
                                              (torch.bfloat16, 64, 333, True), (torch.float16, 128, 700, False)])
@pytest.mark.parametrize("topk", [0.5, 1.0])
def test_f16v_kernel_on_oracle_tensors(dtype, D, N, causal, topk):
    B, H = 1, 2
    q = rand_T((B, H, N, D), dtype, 60)
    k = rand_T((B, H, N, D), dtype, 61, shift=0.4)
    v = rand_T((B, H, N, D), dtype, 62)
    res = oapi.spas_sage_attn_meansim_topk(to_np(q), to_np(k), to_np(v), tag_of(dtype), topk=topk, is_causal=causal)
    dev = "cuda"
    vt = _lib.v_tiles_f16_swizzled(v)
    assert np.array_equal(to_np(_lib.v_tiles_f16_to_natural(vt)), res["v16"])
    out = torch.zeros((B, H, N, D), dtype=dtype, device=dev)
    pvt = torch.full((H,), 50.0, dtype=torch.float32, device=dev)
    pvc = _lib.block_sparse_attn_f16v(torch.from_numpy(res["q8"]).to(dev), torch.from_numpy(res["k8"]).to(dev), vt, out,
                                      torch.from_numpy(res["lut"]).to(dev), torch.from_numpy(res["valid"]).to(dev), pvt,
                                      torch.from_numpy(res["q_scale"]).to(dev), torch.from_numpy(res["k_scale"]).to(dev),
                                      1.0 / D ** 0.5, is_causal=causal, return_pv_count=True)
    torch.cuda.synchronize()
    met = _check(out, res["out"])
    print(f"f16v {dtype} D{D} N{N} causal={causal} topk={topk}: {met}", flush=True)
    assert np.array_equal(pvc.view(B, H, -1, 4).cpu().numpy(), np.repeat(res["pv_count"][..., None], 4, axis=-1))


def test_f16v_pv_threshold_skips_like_the_oracle():
    dtype, D, N, B, H = torch.float16, 64, 768, 1, 2
    q = (rand_T((B, H, N, D), dtype, 50).float().abs() + 0.5).to(dtype)
    k = rand_T((B, H, N, D), dtype, 51, scale=0.05)
    k[:, :, :64] += 6.0
    v = rand_T((B, H, N, D), dtype, 52)
    for thr in (5.0, -1e6):
        res = oapi.spas_sage_attn_meansim_topk(to_np(q), to_np(k), to_np(v), tag_of(dtype), topk=1.0, pvthreshd=thr)
        o = sa.spas_sage_attn_meansim_topk_cuda(q, k, v, topk=1.0, pvthreshd=thr)
        _check(o, res["out"])
    assert res["pv_count"].max() <= 3          # first block + the two final blocks


@pytest.mark.parametrize("name,shrink,causal", [("cfg1", None, False), ("cfg4", dict(H=2, N=2048), True),
                                                ("cfg3", dict(H=2, grid=(4, 12, 15), text_tokens=50), False)])
def test_sage1_topk_operator_vs_oracle(name, shrink, causal):
    cfg = W.CONFIGS[name]
    q, k, v = W.make_qkv(cfg, device="cuda", shrink=shrink)
    res = oapi.spas_sage_attn_meansim_topk(to_np(q), to_np(k), to_np(v), tag_of(cfg.dtype), is_causal=causal,
                                           topk=cfg.topk, pvthreshd=cfg.pvthreshd)
    o, sparsity = sa.spas_sage_attn_meansim_topk_cuda(q, k, v, is_causal=causal, topk=cfg.topk, pvthreshd=cfg.pvthreshd,
                                                      return_sparsity=True)
    assert o.dtype == cfg.dtype and abs(sparsity - res["sparsity"]) < 1e-6
    _check(o, res["out"])
    # NHD layout and the CDF entry point
    o2 = sa.spas_sage_attn_meansim_topk_cuda(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), is_causal=causal,
                                             topk=cfg.topk, pvthreshd=cfg.pvthreshd, tensor_layout="NHD")
    assert torch.equal(o2.transpose(1, 2), o)
    res_c = oapi.spas_sage_attn_meansim_topk(to_np(q), to_np(k), to_np(v), tag_of(cfg.dtype), is_causal=causal, topk=None,
                                             cdfthreshd=0.9, simthreshd1=0.3)
    o3 = sa.spas_sage_attn_meansim_cuda(q, k, v, is_causal=causal, cdfthreshd=0.9, simthreshd1=0.3)
    _check(o3, res_c["out"])


def test_sage1_against_sdpa_and_fp8_path():
    """Same selection, two PV precisions: both near dense attention under the block mask; the fp16-PV output is the
    closer one."""
    cfg = W.CONFIGS["cfg1"]
    q, k, v = W.make_qkv(cfg, device="cuda")
    o1 = sa.spas_sage_attn_meansim_topk_cuda(q, k, v, topk=1.0)
    o2 = sa.spas_sage2_attn_meansim_topk_cuda(q, k, v, topk=1.0)
    ref = torch.nn.functional.scaled_dot_product_attention(q.float(), k.float(), v.float())
    m1 = oat.precision_metric(to_np(o1), to_np(ref))
    m2 = oat.precision_metric(to_np(o2), to_np(ref))
    assert m1["Cossim"] > 0.999 and m2["Cossim"] > 0.999 and m1["L1"] <= m2["L1"] * 1.05, (m1, m2)
