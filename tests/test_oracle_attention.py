"""Pins oracle/attention.py: dense special case, token-mask equivalence, PV-skip rule, end-to-end API."""
import numpy as np
import pytest
import torch

from oracle import api, attention as at, maskpred as mp, vquant as vq
from oracle import rounding as R


def _inputs(seed, b, h, n, d, tag):
    rng = np.random.default_rng(seed)
    mk = lambda s: R.round_to(rng.standard_normal((b, h, n, d)) * s, tag)
    return mk(1.0), mk(1.0) + 0.5, mk(1.0)


def _dequantised(res, n, d):
    """Float tensors the kernel effectively multiplies: q8*q_scale, k8*k_scale, v8*v_scale."""
    q = res["q8"].astype(np.float64) * np.repeat(res["q_scale"].astype(np.float64), 128, axis=2)[:, :, :n, None]
    k = res["k8"].astype(np.float64) * np.repeat(res["k_scale"].astype(np.float64), 64, axis=2)[:, :, :n, None]
    v = vq.dequant(res["v8"])[:, :, :n].astype(np.float64) * res["v_scale"].astype(np.float64)[:, :, None, :]
    return torch.from_numpy(q), torch.from_numpy(k), torch.from_numpy(v)


def _token_mask(block_map, n):
    """Token-level mask of a 128x64 block map (what block_map_to_mask builds, utils.py:424-432)."""
    m = np.repeat(np.repeat(block_map, 128, axis=2), 64, axis=3)
    return torch.from_numpy(m[:, :, :n, :n])


@pytest.mark.parametrize("tag,d,n", [(R.BF16, 128, 384), (R.FP16, 64, 300)])
def test_all_blocks_reduces_to_dense_sdpa(tag, d, n):
    q, k, v = _inputs(0, 1, 2, n, d, tag)
    res = api.spas_sage2_attn_meansim_topk(q, k, v, tag, topk=1.0)
    assert res["map"].all() and np.array_equal(res["pv_count"], res["valid"])
    qd, kd, vd = _dequantised(res, n, d)
    ref = torch.nn.functional.scaled_dot_product_attention(qd, kd, vd).numpy()
    met = at.precision_metric(res["out"], ref)
    # remaining error: e4m3 rounding of P (numerator only) and the output rounding
    assert met["Cossim"] > 0.9995 and met["L1"] < 0.03, met
    # and against the un-quantised inputs (reported accuracy of the method itself)
    ref2 = torch.nn.functional.scaled_dot_product_attention(
        torch.from_numpy(q).double(), torch.from_numpy(k).double(), torch.from_numpy(v).double()).numpy()
    assert at.precision_metric(res["out"], ref2)["Cossim"] > 0.999


def test_block_map_equals_token_masked_sdpa():
    tag, d, n = R.BF16, 64, 512
    q, k, v = _inputs(1, 1, 2, n, d, tag)
    rng = np.random.default_rng(2)
    mask = rng.random((1, 2, 4, 8)) < 0.4
    mask[:, :, np.arange(4), 2 * np.arange(4)] = True
    res = api.block_sparse_sage2_attn(q, k, v, mask.astype(np.int32), tag)
    qd, kd, vd = _dequantised(res, n, d)
    ref = torch.nn.functional.scaled_dot_product_attention(qd, kd, vd, attn_mask=_token_mask(mask, n)).numpy()
    met = at.precision_metric(res["out"], ref)
    assert met["Cossim"] > 0.9995 and met["L1"] < 0.03, met
    assert res["written"].all()


def test_kernel_causal_flag_equals_token_causal_sdpa():
    tag, d, n = R.FP16, 64, 512
    q, k, v = _inputs(3, 1, 1, n, d, tag)
    res = api.spas_sage2_attn_meansim_topk(q, k, v, tag, topk=1.0, is_causal=True, kernel_causal=True)
    qd, kd, vd = _dequantised(res, n, d)
    ref = torch.nn.functional.scaled_dot_product_attention(qd, kd, vd, is_causal=True).numpy()
    assert at.precision_metric(res["out"], ref)["Cossim"] > 0.9995
    # reference behaviour (kernel flag False): causality only at block granularity
    res_b = api.spas_sage2_attn_meansim_topk(q, k, v, tag, topk=1.0, is_causal=True, kernel_causal=False)
    cm = mp.causal_block_mask(4, 8)
    ref_b = torch.nn.functional.scaled_dot_product_attention(
        qd, kd, vd, attn_mask=_token_mask(np.broadcast_to(cm, (1, 1, 4, 8)), n)).numpy()
    assert at.precision_metric(res_b["out"], ref_b)["Cossim"] > 0.9995


def test_partial_blocks_and_empty_rows():
    tag, d, n = R.BF16, 64, 333            # partial last Q block (77 rows) and K block (13 rows)
    q, k, v = _inputs(4, 1, 1, n, d, tag)
    mask = np.ones((1, 1, 3, 6), np.int32)
    mask[0, 0, 1] = 0                       # a row block with no selected K block stays unwritten
    res = api.block_sparse_sage2_attn(q, k, v, mask, tag)
    assert list(res["written"][0, 0]) == [True, False, True]
    assert np.all(res["out"][0, 0, 128:256] == 0)
    qd, kd, vd = _dequantised(res, n, d)
    ref = torch.nn.functional.scaled_dot_product_attention(qd, kd, vd).numpy()
    sel = np.r_[0:128, 256:n]
    assert at.precision_metric(res["out"][0, 0, sel], ref[0, 0, sel])["Cossim"] > 0.9995


def test_pv_threshold_skip_rule():
    """Two-scale example: K blocks 0..1 carry large scores, blocks 2..3 tiny ones, 4..5 close the row.

    With the running maximum set by block 0, every later middle block has m_blk far below m.
    Threshold t skips a middle block iff max_rows(m_blk - m_prev) + t <= 0 (sm89.cuh:353)."""
    tag, d, n = R.FP16, 64, 384
    rng = np.random.default_rng(5)
    q = R.round_to(np.abs(rng.standard_normal((1, 1, n, d))) + 0.5, tag)
    k = R.round_to(rng.standard_normal((1, 1, n, d)) * 0.05, tag)
    k[0, 0, :64] += 6.0                                  # block 0 dominates every row
    v = R.round_to(rng.standard_normal((1, 1, n, d)), tag)
    mask = np.ones((1, 1, 3, 6), np.int32)
    hi = api.block_sparse_sage2_attn(q, k, v, mask, tag, pvthreshd=1e6)
    lo = api.block_sparse_sage2_attn(q, k, v, mask, tag, pvthreshd=5.0)
    # 6 blocks per row: 4 middle (skippable) + 2 final (never skipped); block 0 always raises the max
    assert np.all(hi["pv_count"] == 6)
    assert np.all(lo["pv_count"] == 3), lo["pv_count"]
    # skipped blocks carried < 2^-5 of the weight... the result changes only slightly
    assert at.precision_metric(lo["out"], hi["out"])["Cossim"] > 0.99
    # the first block raises m from the -5e6 sentinel, i.e. delta ~ 5e6: it survives t = -1e6 but not t = -1e7
    assert np.all(api.block_sparse_sage2_attn(q, k, v, mask, tag, pvthreshd=-1e6)["pv_count"] == 3)
    assert np.all(api.block_sparse_sage2_attn(q, k, v, mask, tag, pvthreshd=-1e7)["pv_count"] == 2)


def test_topk_api_end_to_end_small():
    tag, d, n = R.BF16, 64, 1024
    q, k, v = _inputs(6, 1, 2, n, d, tag)
    res = api.spas_sage2_attn_meansim_topk(q, k, v, tag, topk=0.5)
    assert res["lut"].shape == (1, 2, 8, 16) and np.all(res["valid"] == 8)
    assert abs(res["sparsity"] - 0.5) < 1e-12
    qd, kd, vd = _dequantised(res, n, d)
    ref = torch.nn.functional.scaled_dot_product_attention(qd, kd, vd, attn_mask=_token_mask(res["map"], n)).numpy()
    assert at.precision_metric(res["out"], ref)["Cossim"] > 0.9995
    res_c = api.spas_sage2_attn_meansim_topk(q, k, v, tag, topk=0.5, is_causal=True)
    assert list(res_c["valid"][0, 0]) == [2, 4, 6, 8, 8, 8, 8, 8]
    tot = float(res_c["valid"].sum())
    assert abs(res_c["sparsity"] - (1 - tot / (9 * 8 * 2))) < 1e-12      # causal denominator (nk+2)//2


# ---- SageAttention1 variant (INT8 QK^T, FP16 PV): pinned by the same library-routine special cases ----------------

def _dequantised_f16v(res, n):
    q = res["q8"].astype(np.float64) * np.repeat(res["q_scale"].astype(np.float64), 128, axis=2)[:, :, :n, None]
    k = res["k8"].astype(np.float64) * np.repeat(res["k_scale"].astype(np.float64), 64, axis=2)[:, :, :n, None]
    return torch.from_numpy(q), torch.from_numpy(k), torch.from_numpy(res["v16"][:, :, :n].astype(np.float64))


@pytest.mark.parametrize("tag,d,n", [(R.BF16, 128, 384), (R.FP16, 64, 300)])
def test_f16v_all_blocks_reduces_to_dense_sdpa(tag, d, n):
    q, k, v = _inputs(10, 1, 2, n, d, tag)
    res = api.spas_sage_attn_meansim_topk(q, k, v, tag, topk=1.0)
    assert res["map"].all() and np.array_equal(res["pv_count"], res["valid"])
    assert np.array_equal(res["v16"][:, :, :n], v.astype(np.float16).astype(np.float32))
    qd, kd, vd = _dequantised_f16v(res, n)
    ref = torch.nn.functional.scaled_dot_product_attention(qd, kd, vd).numpy()
    met = at.precision_metric(res["out"], ref)
    # remaining error: fp16 rounding of P (numerator and denominator alike) and the output rounding: far below the
    # e4m3 variant's
    assert met["Cossim"] > 0.99999 and met["L1"] < (6e-3 if tag == R.BF16 else 1.5e-3), met


def test_f16v_token_causal_and_block_mask():
    tag, d, n = R.FP16, 64, 512
    q, k, v = _inputs(11, 1, 2, n, d, tag)
    res = api.spas_sage_attn_meansim_topk(q, k, v, tag, topk=0.5, is_causal=True)
    qd, kd, vd = _dequantised_f16v(res, n)
    tok = _token_mask(res["map"], n) & torch.tril(torch.ones(n, n, dtype=torch.bool))
    ref = torch.nn.functional.scaled_dot_product_attention(qd, kd, vd, attn_mask=tok).numpy()
    met = at.precision_metric(res["out"], ref)
    assert met["Cossim"] > 0.99999 and met["L1"] < 1.5e-3, met
    # sparsity is reported against the causal denominator (core.py:314-317)
    assert abs(res["sparsity"] - (1 - res["valid"].sum() / ((8 + 2) // 2 * 4 * 2))) < 1e-12


def test_f16v_denominator_uses_rounded_p():
    """One dominant key (p = 1, v = 1) and 63 999 keys whose probability 1.4 * 2^-24 rounds to the fp16 subnormal 2^-24
    (v = 0): the output is 1 / (1 + 63999 * 2^-24) = 0.99620 when the denominator sums the ROUNDED P and 0.99469 when
    it sums the exact P; fp16 resolves the two."""
    d, nblk = 64, 1000
    n = 64 * nblk
    q8 = np.zeros((1, 1, 128, d), np.int8); q8[0, 0, :, 0] = 100
    k8 = np.zeros((1, 1, n, d), np.int8); k8[0, 0, 0, 0] = 100
    v16 = np.zeros((1, 1, n, d), np.float32); v16[0, 0, 0, :] = 1.0
    lut = np.ones((1, 1, 1, nblk), np.int32); lut[0, 0, 0, 0] = 0
    valid = np.full((1, 1, 1), nblk, np.int32)
    target = 1.4 * 2.0 ** -24
    c = -np.log(target) / 10000.0                         # softmax scale: exp(-10000 c) = target
    out, written, pvc = at.block_sparse_attention(
        q8, k8, v16, lut, valid, np.array([50.0], np.float32), np.full((1, 1, 1), 0.1, np.float32),
        np.full((1, 1, nblk), 0.1, np.float32), None, c / 0.01, "fp16", return_pv_count=True, pv="f16")
    assert pvc[0, 0, 0] == nblk
    rounded = 1.0 / (1.0 + (n - 1) * 2.0 ** -24)
    exact = 1.0 / (1.0 + (n - 1) * target)
    got = float(out[0, 0, 5, 3])
    assert abs(got - rounded) < 4e-4 < abs(got - exact), (got, rounded, exact)


def test_fp8_denominator_sums_unrounded_p_and_uses_the_offset():
    """The two choices of the FP8 kernel that a tolerance test on random data cannot see (sm89.cuh:353-391,
    attn_utils.cuh:28): the denominator sums the binary32 P while the numerator uses e4m3(P), and P carries the
    2^8.807 factor that decides on which e4m3 grid it is rounded.  A construction whose closed form separates the
    reference semantics from both alternatives by more than 0.04."""
    from gpu_common import fp8_denominator_case
    args, forms = fp8_denominator_case()
    out, written, pvc = at.block_sparse_attention(*args[:9], args[9], "fp16", return_pv_count=True)
    assert pvc[0, 0, 0] == 4
    got = float(out[0, 0, 7, 3])
    assert abs(got - forms["reference"]) < 1.5e-3, (got, forms)
    assert abs(got - forms["rounded_denominator"]) > 0.03 and abs(got - forms["no_offset"]) > 0.03, (got, forms)
    assert np.all(np.abs(out[0, 0] - got) < 1e-6)           # every row and channel alike


def test_gqa_equals_mha_with_repeated_kv_heads():
    """Grouped-query attention: query head h reads K/V head h // (H / Hkv) (sm89.cuh:118).  With K/V heads repeated
    the multi-head path must give the identical result (quantisation is per K/V head, so nothing else changes)."""
    tag, d, n, H, Hkv = R.BF16, 64, 384, 4, 2
    rng = np.random.default_rng(21)
    mk = lambda h: R.round_to(rng.standard_normal((1, h, n, d)), tag)
    q, k, v = mk(H), mk(Hkv) + 0.3, mk(Hkv)
    mask = (rng.random((1, H, 3, 6)) < 0.5).astype(np.int32)
    mask[:, :, np.arange(3), 2 * np.arange(3)] = 1
    res = api.block_sparse_sage2_attn(q, k, v, mask, tag, pvthreshd=4.0)
    rep = api.block_sparse_sage2_attn(q, np.repeat(k, H // Hkv, axis=1), np.repeat(v, H // Hkv, axis=1), mask, tag,
                                      pvthreshd=4.0)
    assert res["k8"].shape[1] == Hkv and rep["k8"].shape[1] == H
    assert np.array_equal(res["out"], rep["out"]) and np.array_equal(res["pv_count"], rep["pv_count"])
    assert not np.array_equal(res["out"][:, 0], res["out"][:, 2])       # heads of different groups do differ


def _skip_problem(seed, d=64, nblk=6):
    """int8 tensors in which block 0 dominates for SOME 32-row groups only, so that the warps of a Q block decide differently."""
    rng = np.random.default_rng(seed)
    n = 64 * nblk
    q8 = rng.integers(-20, 21, size=(1, 1, 128, d)).astype(np.int8)
    k8 = rng.integers(-20, 21, size=(1, 1, n, d)).astype(np.int8)
    q8[0, 0, 32:64, 0] = 120                       # rows of group 1 ...
    k8[0, 0, :64, 0] = 120                         # ... see a huge score on every key of block 0
    v8 = rng.integers(0, 120, size=(1, 1, n, d)).astype(np.uint8)
    lut = np.ones((1, 1, 1, nblk), np.int32); lut[0, 0, 0, 0] = 0
    valid = np.full((1, 1, 1), nblk, np.int32)
    one = np.ones((1, 1, 1), np.float32)
    args = dict(pvthreshd=np.array([2.0], np.float32), q_scale=one * 0.05, k_scale=np.full((1, 1, nblk), 0.05, np.float32),
                v_scale=np.ones((1, 1, d), np.float32), sm_scale=d ** -0.5, out_dtype="fp16")
    return q8, k8, v8, lut, valid, args


def _run(q8, k8, v8, lut, valid, args, **kw):
    return at.block_sparse_attention(q8, k8, v8, lut, valid, args["pvthreshd"], args["q_scale"], args["k_scale"],
                                     args["v_scale"], args["sm_scale"], args["out_dtype"], return_pv_count=True, **kw)


def test_pv_threshold_modes():
    q8, k8, v8, lut, valid, args = _skip_problem(5)
    out1, _, c1 = _run(q8, k8, v8, lut, valid, args, pv_mode=1)
    out2, _, c2 = _run(q8, k8, v8, lut, valid, args, pv_mode=2)
    out0, _, c0 = _run(q8, k8, v8, lut, valid, args, pv_mode=0)
    assert c0[0, 0, 0] == 6 and c1[0, 0, 0] == 6            # the other groups keep the block decision at "compute"
    assert c2.shape == (1, 1, 1, 4) and c2[0, 0, 0, 1] == 3 and (c2[0, 0, 0, [0, 2, 3]] == 6).all()
    # never skipping = per-block with a threshold nothing can miss
    big = dict(args, pvthreshd=np.array([1e6], np.float32))
    outb, _, _ = _run(q8, k8, v8, lut, valid, big, pv_mode=1)
    assert np.array_equal(out0, outb)
    # the per-warp decision of group g is the per-block decision of a Q block made of four copies of group g
    for g in range(4):
        qg = np.tile(q8[:, :, 32 * g:32 * g + 32], (1, 1, 4, 1))
        outg, _, cg = _run(qg, k8, v8, lut, valid, args, pv_mode=1)
        assert np.array_equal(outg[0, 0, :32], out2[0, 0, 32 * g:32 * g + 32]) and cg[0, 0, 0] == c2[0, 0, 0, g]
    # skipping changed something for group 1 only
    assert not np.array_equal(out2[0, 0, 32:64], out1[0, 0, 32:64])
    assert np.array_equal(out2[0, 0, :32], out1[0, 0, :32]) and np.array_equal(out2[0, 0, 64:], out1[0, 0, 64:])
