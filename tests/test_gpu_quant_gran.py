"""GPU parity of the per-warp INT8 granularity (qk_quant_gran = 2) against the oracle, through the C ABI.

Codes and scales of the 32-row quantiser bit for bit; the attention kernels (FP8 PV and FP16 PV) at the output
tolerance of the other attention tests with equal PV-skip counts; the operators' opt-in keyword.
"""
import numpy as np
import pytest
import torch

import spargeattn_amd as sa
from oracle import api as oapi, attention as oat, maskpred as mp
from spargeattn_amd import _lib, utils
from gpu_common import tag_of, to_np, bits_equal_T, rand_T
from test_gpu_attention import _check_out

pytestmark = pytest.mark.gpu


def _grouped_q(B, H, N, D, dtype, seed):
    """Q whose 32-row groups differ in magnitude (1, 10, 0.1, 3): the four scales of a block differ by up to 100x."""
    mags = torch.tensor([1.0, 10.0, 0.1, 3.0])[(torch.arange(N) // 32) % 4]
    g = torch.Generator().manual_seed(seed)
    return (torch.randn((B, H, N, D), generator=g) * mags[None, None, :, None] * 0.3).to(dtype).cuda()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,H,N,D", [(1, 2, 1024, 64), (2, 2, 333, 128), (1, 3, 1100, 128), (1, 2, 128 + 40, 64),
                                     (1, 1, 130, 128)])
def test_quantiser_with_32_row_groups(dtype, B, H, N, D):
    tag = tag_of(dtype)
    q = _grouped_q(B, H, N, D, dtype, 2)
    thr = torch.tensor([0.5] * H, dtype=torch.float32, device="cuda")
    pool, sim, xq, scale = _lib.pool_sim_quant(q, None, 128, thr, quant_rows=32)
    ref = mp.pool_sim_quant(to_np(q), None, 128, thr.cpu().numpy(), tag, quant_rows=32)
    nb = (N + 127) // 128
    assert scale.shape == (B, H, nb * 4)
    assert np.array_equal(xq.cpu().numpy(), ref["q"])
    assert np.array_equal(scale.cpu().numpy().view(np.uint32), ref["scale"].view(np.uint32))
    assert bits_equal_T(pool, ref["pool"], dtype) and np.array_equal(sim.cpu().numpy(), ref["sim"])
    # pooled blocks and flags do not depend on the granularity; the quant-only entry gives the same codes
    pool1, sim1, _, scale1 = _lib.pool_sim_quant(q, None, 128, thr)
    assert torch.equal(pool1, pool) and torch.equal(sim1, sim)
    assert torch.equal(scale.view(B, H, nb, 4).amax(dim=-1), scale1)
    _, _, xq2, scale2 = _lib.pool_sim_quant(q, None, 128, with_pool=False, quant_rows=32)
    assert torch.equal(xq2, xq) and torch.equal(scale2, scale)
    # NHD input read in place
    qn = q.transpose(1, 2).contiguous().transpose(1, 2)
    _, _, xq3, scale3 = _lib.pool_sim_quant(qn, None, 128, thr, quant_rows=32)
    assert torch.equal(xq3, xq) and torch.equal(scale3, scale)


def test_quantiser_refuses_other_group_sizes():
    q = rand_T((1, 1, 256, 64), torch.float16, 1)
    km = _lib.km_mean(q)
    with pytest.raises(ValueError, match="quant_rows"):
        _lib.pool_sim_quant(q, None, 64, with_pool=False, quant_rows=32)        # K blocks: a warp spans the block
    with pytest.raises(ValueError, match="quant_rows"):
        _lib.pool_sim_quant(q, km, 128, with_pool=False, quant_rows=32)
    with pytest.raises(ValueError, match="quant_rows"):
        _lib.pool_sim_quant(q, None, 128, with_pool=False, quant_rows=64)
    with pytest.raises(ValueError):
        utils.get_vanilla_qk_quant(q, q, km, qk_quant_gran=3)
    with pytest.raises(ValueError, match="Unsupported qk_quant_gran"):
        utils.get_vanilla_qk_quant(q, q, km, qk_quant_gran="per_token")


def _run_kernel(res, out_dtype, H, N, D, pvthreshd, fp16v=False, is_causal=False, pv_mode=_lib.PV_PER_BLOCK, v16=None):
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    B = res["q8"].shape[0]
    Nk = res["k8"].shape[2]
    nk = (Nk + 63) // 64
    out = torch.zeros((B, H, N, D), dtype=out_dtype, device="cuda")
    pvt = torch.full((H,), float(pvthreshd), dtype=torch.float32, device="cuda")
    common = (dev(res["lut"]), dev(res["valid"]), pvt, dev(res["q_scale"]), dev(res["k_scale"]))
    if fp16v:
        vt = _lib.v_tiles_f16_swizzled(v16)
        pvc = _lib.block_sparse_attn_f16v(dev(res["q8"]), dev(res["k8"]), vt, out, *common, 1.0 / D ** 0.5,
                                          is_causal=is_causal, return_pv_count=True, pv_mode=pv_mode, qk_quant_gran=2)
    else:
        v8 = _lib.v8_natural_to_tiles(dev(res["v8"][:, :, :nk * 64]))
        pvc = _lib.block_sparse_attn(dev(res["q8"]), dev(res["k8"]), v8, out, *common, dev(res["v_scale"]),
                                     1.0 / D ** 0.5, is_causal=is_causal, return_pv_count=True, pv_mode=pv_mode,
                                     qk_quant_gran=2)
    torch.cuda.synchronize()
    return out, pvc.view(B, H, -1, 4)


@pytest.mark.parametrize("dtype,D,N", [(torch.bfloat16, 128, 1024), (torch.float16, 64, 1024),
                                       (torch.bfloat16, 64, 333), (torch.float16, 128, 700)])
@pytest.mark.parametrize("topk,pvthreshd", [(0.5, 50), (1.0, 50), (1.0, 1.0)])
def test_attention_kernel_with_per_warp_q_scales(dtype, D, N, topk, pvthreshd):
    """The ORACLE's per-warp tensors through the HIP kernel: output at tolerance, PV counts equal (with pvthreshd = 1
    blocks are actually skipped, decided per block from rows that carry different scales)."""
    B, H = 1, 2
    q = _grouped_q(B, H, N, D, dtype, 30)
    k = rand_T((B, H, N, D), dtype, 31, shift=0.4)
    v = rand_T((B, H, N, D), dtype, 32)
    res = oapi.spas_sage2_attn_meansim_topk(to_np(q), to_np(k), to_np(v), tag_of(dtype), topk=topk, pvthreshd=pvthreshd,
                                            qk_quant_gran=2)
    out, pvc = _run_kernel(res, dtype, H, N, D, pvthreshd)
    _check_out(out, res["out"])
    assert bool((pvc == pvc[..., :1]).all())                      # per-block decision: equal inside a Q block
    assert np.array_equal(pvc[..., 0].cpu().numpy(), res["pv_count"])
    if pvthreshd == 50:
        assert np.array_equal(res["pv_count"], res["valid"])
    # the per-block reading of the same codes (first scale of every block) is NOT what the kernel computes
    wrong = dict(res, q_scale=np.ascontiguousarray(res["q_scale"].reshape(B, H, -1, 4)[..., 0]))
    ref_wrong, _ = oat.block_sparse_attention(wrong["q8"], wrong["k8"], wrong["v8"], wrong["lut"], wrong["valid"],
                                              np.full(H, 50.0, np.float32), wrong["q_scale"], wrong["k_scale"],
                                              wrong["v_scale"], D ** -0.5, tag_of(dtype))
    if topk == 1.0 and pvthreshd == 50:
        assert oat.precision_metric(to_np(out), ref_wrong)["L1"] > 0.05


@pytest.mark.parametrize("fp16v", [False, True])
def test_per_warp_scales_with_per_warp_pv_threshold_and_token_causal(fp16v):
    dtype, D, N, B, H = torch.float16, 64, 768, 1, 2
    q = _grouped_q(B, H, N, D, dtype, 40).abs() + 0.05
    k = rand_T((B, H, N, D), dtype, 41, scale=0.05)
    k[:, :, :64] += 4.0                                     # block 0 dominates: later blocks fall below the threshold
    v = rand_T((B, H, N, D), dtype, 42)
    qn, kn, vn = to_np(q), to_np(k), to_np(v)
    tag = tag_of(dtype)
    for mode, causal in ((_lib.PV_PER_BLOCK, False), (_lib.PV_PER_WARP, False), (_lib.PV_NONE, True)):
        if fp16v:
            res = oapi.spas_sage_attn_meansim_topk(qn, kn, vn, tag, topk=1.0, qk_quant_gran=2)
            vor, vs, pv = res["v16"], None, "f16"
        else:
            res = oapi.spas_sage2_attn_meansim_topk(qn, kn, vn, tag, topk=1.0, qk_quant_gran=2)
            vor, vs, pv = res["v8"], res["v_scale"], "fp8"
        ref, _, refc = oat.block_sparse_attention(res["q8"], res["k8"], vor, res["lut"], res["valid"],
                                                  np.full(H, 3.0, np.float32), res["q_scale"], res["k_scale"], vs,
                                                  D ** -0.5, tag, is_causal=causal, return_pv_count=True, pv=pv,
                                                  pv_mode=mode, qk_quant_gran=2)
        out, pvc = _run_kernel(res, dtype, H, N, D, 3.0, fp16v=fp16v, is_causal=causal, pv_mode=mode, v16=v)
        _check_out(out, ref)
        want = refc if mode == _lib.PV_PER_WARP else np.repeat(refc[..., None], 4, axis=-1)
        assert np.array_equal(pvc.cpu().numpy(), want), mode
    assert refc.max() == 12                                  # no threshold: everything computed


@pytest.mark.parametrize("H,Hkv,D,dtype,causal", [(4, 2, 64, torch.float16, False), (6, 1, 128, torch.bfloat16, True)])
def test_operators_with_per_warp_granularity(H, Hkv, D, dtype, causal):
    """The opt-in keyword of the operators, with grouped K/V heads and qo_len != kv_len; the default stays per block."""
    B, Nq, Nk = 1, 640, 900
    tag = tag_of(dtype)
    q = _grouped_q(B, H, Nq, D, dtype, 70)
    k = rand_T((B, Hkv, Nk, D), dtype, 71, shift=0.3)
    v = rand_T((B, Hkv, Nk, D), dtype, 72)
    qn, kn, vn = to_np(q), to_np(k), to_np(v)
    res = oapi.spas_sage2_attn_meansim_topk(qn, kn, vn, tag, topk=0.6, is_causal=causal, qk_quant_gran=2)
    km = _lib.km_mean(k)
    lut, valid, q8, qs, k8, ks = utils.get_block_map_meansim_fuse_quant(q, k, km, is_causal=causal, simthreshd1=-0.1,
                                                                        cdfthreshd=None, topk=0.6, return_lut=True,
                                                                        qk_quant_gran="per_warp")
    assert np.array_equal(q8.cpu().numpy(), res["q8"]) and np.array_equal(qs.cpu().numpy(), res["q_scale"])
    assert np.array_equal(k8.cpu().numpy(), res["k8"]) and np.array_equal(ks.cpu().numpy(), res["k_scale"])
    assert np.array_equal(lut.cpu().numpy(), res["lut"]) and np.array_equal(valid.cpu().numpy(), res["valid"])
    o, sp = sa.spas_sage2_attn_meansim_topk_cuda(q, k, v, topk=0.6, is_causal=causal, return_sparsity=True,
                                                 qk_quant_gran=2)
    assert abs(sp - res["sparsity"]) < 1e-6
    _check_out(o, res["out"])
    # the default is the reference's per-block granularity, and differs
    o1 = sa.spas_sage2_attn_meansim_topk_cuda(q, k, v, topk=0.6, is_causal=causal)
    res1 = oapi.spas_sage2_attn_meansim_topk(qn, kn, vn, tag, topk=0.6, is_causal=causal)
    _check_out(o1, res1["out"])
    assert not torch.equal(o, o1)
    # CDF selection, the custom-mask operator and the INT8-QK / FP16-PV operators
    res = oapi.spas_sage2_attn_meansim_topk(qn, kn, vn, tag, simthreshd1=0.3, cdfthreshd=0.9, topk=None, qk_quant_gran=2)
    _check_out(sa.spas_sage2_attn_meansim_cuda(q, k, v, simthreshd1=0.3, cdfthreshd=0.9, qk_quant_gran="per_warp"), res["out"])
    nq, nk = (Nq + 127) // 128, (Nk + 63) // 64
    g = torch.Generator().manual_seed(5)
    mask = (torch.rand((B, H, nq, nk), generator=g) < 0.5).to(torch.int32)
    mask[..., nk - 1] = 1
    res = oapi.block_sparse_sage2_attn(qn, kn, vn, mask.numpy(), tag, pvthreshd=3.0, qk_quant_gran=2)
    _check_out(sa.block_sparse_sage2_attn_cuda(q, k, v, mask_id=mask.cuda(), pvthreshd=3.0, qk_quant_gran=2), res["out"])
    res = oapi.spas_sage_attn_meansim_topk(qn, kn, vn, tag, topk=0.5, is_causal=causal, qk_quant_gran=2)
    _check_out(sa.spas_sage_attn_meansim_topk_cuda(q, k, v, topk=0.5, is_causal=causal, qk_quant_gran=2), res["out"])
    res = oapi.spas_sage_attn_meansim_topk(qn, kn, vn, tag, simthreshd1=0.3, cdfthreshd=0.9, topk=None, qk_quant_gran=2)
    _check_out(sa.spas_sage_attn_meansim_cuda(q, k, v, simthreshd1=0.3, cdfthreshd=0.9, qk_quant_gran=2), res["out"])
    with pytest.raises(ValueError, match="per thread"):
        sa.spas_sage2_attn_meansim_topk_cuda(q, k, v, qk_quant_gran=3)
    with pytest.raises(RuntimeError, match="q_scale"):          # per-block scales handed over as per-warp ones
        o = torch.empty_like(q)
        pvt = torch.full((H,), 50.0, device="cuda")
        _, _, _, qs1 = _lib.pool_sim_quant(q, None, 128, with_pool=False)
        v8, vs = _lib.v_quant_fp8(v)
        _lib.block_sparse_attn(q8, k8, v8, o, lut, valid, pvt, qs1, ks, vs, 0.1, qk_quant_gran=2)


def test_per_warp_granularity_is_the_more_accurate_one():
    """Against fp32 attention on the original tensors (all blocks kept), on rows of mixed magnitude."""
    dtype, B, H, N, D = torch.bfloat16, 1, 2, 1024, 128
    q = _grouped_q(B, H, N, D, dtype, 80)
    k = rand_T((B, H, N, D), dtype, 81, shift=0.3)
    v = rand_T((B, H, N, D), dtype, 82)
    ref = torch.nn.functional.scaled_dot_product_attention(q.float(), k.float(), v.float())
    err = {}
    for gran in (1, 2):
        o = sa.spas_sage2_attn_meansim_topk_cuda(q, k, v, topk=1.0, qk_quant_gran=gran)
        err[gran] = float((o.float() - ref).abs().sum() / ref.abs().sum())
    assert err[2] < err[1], err
