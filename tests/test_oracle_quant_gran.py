"""Pins the per-warp INT8 granularity of the oracle (qk_quant_gran = 2: one Q scale per 32 query rows).

Reference behaviour restated: per_warp_int8 (spas_sage_attn/quant_per_block.py:102-148) runs the per-group quantiser
over 32-row groups of Q and 64-row groups of K; the kernel reads q_scale at 4 * block + warp
(csrc/qattn/qk_int_sv_f8_cuda_sm89.cuh:111-115).  Checks chosen so that a wrong group size, a scale read at the wrong
warp, or a scale applied per block instead of per warp fails one of them.
"""
import numpy as np
import pytest
import torch

from oracle import api, attention as at, maskpred as mp, vquant as vq
from oracle import rounding as R
from test_oracle_maskpred import _quant_scalar


def _rows_with_group_magnitudes(rng, b, h, n, d, tag):
    """Q whose 32-row groups differ in magnitude by up to 100x: per-block scales then waste most of the INT8 range of the
    quiet groups, per-warp scales do not."""
    mags = np.array([1.0, 10.0, 0.1, 3.0])[(np.arange(n) // 32) % 4]
    return R.round_to(rng.standard_normal((b, h, n, d)) * mags[None, None, :, None], tag)


@pytest.mark.parametrize("n", [256, 300, 128 + 40, 130])
def test_32_row_groups_against_the_scalar_quantiser(n):
    rng = np.random.default_rng(n)
    x = _rows_with_group_magnitudes(rng, 1, 2, n, 64, R.BF16)
    thr = np.full(2, 0.3, np.float32)
    got = mp.pool_sim_quant(x, None, 128, thr, R.BF16, quant_rows=32)
    nb = (n + 127) // 128
    assert got["scale"].shape == (1, 2, nb * 4) and got["q"].shape == x.shape
    for h in range(2):
        for g in range(nb * 4):
            rows = x[0, h, 32 * g:min(n, 32 * g + 32)]
            if rows.shape[0] == 0:                       # a group past the end: all masked, scale of a zero group
                assert got["scale"][0, h, g] == np.float32(1e-7)
                continue
            qb, sb = _quant_scalar(rows)
            assert got["scale"][0, h, g] == sb and np.array_equal(got["q"][0, h, 32 * g:32 * g + rows.shape[0]], qb)
    # pooling and the similarity flag are per 128-row block whatever the granularity
    per_block = mp.pool_sim_quant(x, None, 128, thr, R.BF16)
    assert np.array_equal(got["pool"], per_block["pool"]) and np.array_equal(got["sim"], per_block["sim"])
    # the block scale is the largest of its groups' scales (same maximum, same arithmetic)
    assert np.array_equal(got["scale"].reshape(1, 2, nb, 4).max(axis=-1), per_block["scale"])
    # quant-only entry
    only = mp.pool_sim_quant(x, None, 128, None, R.BF16, with_pool=False, quant_rows=32)
    assert np.array_equal(only["q"], got["q"]) and np.array_equal(only["scale"], got["scale"])


def _dequantised(res, n, q_rows):
    q = res["q8"].astype(np.float64) * np.repeat(res["q_scale"].astype(np.float64), q_rows, axis=2)[:, :, :n, None]
    k = res["k8"].astype(np.float64) * np.repeat(res["k_scale"].astype(np.float64), 64, axis=2)[:, :, :n, None]
    v = vq.dequant(res["v8"])[:, :, :n].astype(np.float64) * res["v_scale"].astype(np.float64)[:, :, None, :]
    return torch.from_numpy(q), torch.from_numpy(k), torch.from_numpy(v)


@pytest.mark.parametrize("tag,d,n", [(R.BF16, 128, 384), (R.FP16, 64, 300)])
def test_per_warp_scales_reduce_to_dense_sdpa_on_the_dequantised_tensors(tag, d, n):
    """Every block selected: the kernel restatement equals softmax attention on q8 * q_scale[row // 32], k8 * k_scale,
    v8 * v_scale - which fails if a scale is read at the wrong warp or per block (the groups differ 100x)."""
    rng = np.random.default_rng(7)
    q = _rows_with_group_magnitudes(rng, 1, 2, n, d, tag) * 0.3
    q = R.round_to(q, tag)
    k = R.round_to(rng.standard_normal((1, 2, n, d)) + 0.5, tag)
    v = R.round_to(rng.standard_normal((1, 2, n, d)), tag)
    res = api.spas_sage2_attn_meansim_topk(q, k, v, tag, topk=1.0, qk_quant_gran=2)
    assert res["q_scale"].shape == (1, 2, 4 * ((n + 127) // 128))
    qd, kd, vd = _dequantised(res, n, 32)
    ref = torch.nn.functional.scaled_dot_product_attention(qd, kd, vd).numpy()
    met = at.precision_metric(res["out"], ref)
    assert met["Cossim"] > 0.9995 and met["L1"] < 0.03, met
    # the wrong reading - per-warp codes with one scale per block - is far outside that tolerance
    wrong = dict(res, q_scale=res["q_scale"].reshape(1, 2, -1, 4)[..., 0])
    qd2, _, _ = _dequantised(wrong, n, 128)
    ref_wrong = torch.nn.functional.scaled_dot_product_attention(qd2, kd, vd).numpy()
    assert at.precision_metric(res["out"], ref_wrong)["L1"] > 0.1
    # against the un-quantised inputs per-warp scales are the more accurate of the two granularities
    ref32 = torch.nn.functional.scaled_dot_product_attention(
        torch.from_numpy(q).double(), torch.from_numpy(k).double(), torch.from_numpy(v).double()).numpy()
    res1 = api.spas_sage2_attn_meansim_topk(q, k, v, tag, topk=1.0, qk_quant_gran=1)
    assert at.precision_metric(res["out"], ref32)["L1"] < at.precision_metric(res1["out"], ref32)["L1"]
    # ... by a wide margin on the quiet rows (magnitude 0.1 beside a group of magnitude 10: a per-block scale leaves them
    # one or two INT8 levels, so their scores collapse)
    quiet = (np.arange(n) // 32) % 4 == 2
    e2 = at.precision_metric(res["out"][:, :, quiet], ref32[:, :, quiet])["L1"]
    e1 = at.precision_metric(res1["out"][:, :, quiet], ref32[:, :, quiet])["L1"]
    assert e2 < 0.9 * e1, (e1, e2)


def test_equal_scales_in_a_block_give_the_per_block_result_bit_for_bit():
    """Granularity 2 with the four scales of every block equal IS granularity 1 (same codes, same arithmetic)."""
    tag, d, n = R.FP16, 64, 512
    rng = np.random.default_rng(3)
    q, k, v = (R.round_to(rng.standard_normal((1, 2, n, d)), tag) for _ in range(3))
    res = api.spas_sage2_attn_meansim_topk(q, k, v, tag, topk=0.5, pvthreshd=2.0)
    args = (res["q8"], res["k8"], res["v8"], res["lut"], res["valid"], np.full(2, 2.0, np.float32))
    o1, w1, c1 = at.block_sparse_attention(*args, res["q_scale"], res["k_scale"], res["v_scale"], d ** -0.5, tag,
                                           return_pv_count=True)
    o2, w2, c2 = at.block_sparse_attention(*args, np.repeat(res["q_scale"], 4, axis=2), res["k_scale"], res["v_scale"],
                                           d ** -0.5, tag, return_pv_count=True, qk_quant_gran=2)
    assert np.array_equal(o1, o2) and np.array_equal(w1, w2) and np.array_equal(c1, c2)
    assert np.array_equal(o1, res["out"])


def test_mask_and_sage1_operators_take_the_granularity():
    tag, d, n = R.BF16, 64, 384
    rng = np.random.default_rng(11)
    q = R.round_to(_rows_with_group_magnitudes(rng, 1, 1, n, d, tag) * 0.3, tag)
    k, v = (R.round_to(rng.standard_normal((1, 1, n, d)), tag) for _ in range(2))
    mask = np.ones((1, 1, 3, 6), np.int32)
    r = api.block_sparse_sage2_attn(q, k, v, mask, tag, qk_quant_gran=2)
    assert r["q_scale"].shape == (1, 1, 12)
    qd, kd, vd = _dequantised(r, n, 32)
    ref = torch.nn.functional.scaled_dot_product_attention(qd, kd, vd).numpy()
    assert at.precision_metric(r["out"], ref)["L1"] < 0.03
    s = api.spas_sage_attn_meansim_topk(q, k, v, tag, topk=1.0, qk_quant_gran=2)
    qd = torch.from_numpy(s["q8"].astype(np.float64) * np.repeat(s["q_scale"].astype(np.float64), 32, axis=2)[:, :, :n, None])
    kd = torch.from_numpy(s["k8"].astype(np.float64) * np.repeat(s["k_scale"].astype(np.float64), 64, axis=2)[:, :, :n, None])
    ref = torch.nn.functional.scaled_dot_product_attention(qd, kd, torch.from_numpy(s["v16"][:, :, :n]).double()).numpy()
    assert at.precision_metric(s["out"], ref)["L1"] < 2e-3
