"""End-to-end oracle of the two operator entry points.  Test infrastructure only.

``spas_sage2_attn_meansim_topk`` follows spas_sage_attn/core.py:105-169,
``block_sparse_sage2_attn`` follows spas_sage_attn/core.py:171-233 (non-sm90
branch: BLKQ = 128, BLKK = 64) and ``spas_sage_attn_meansim_topk`` follows
spas_sage_attn/core.py:235-319, returning every intermediate tensor so that a
test can compare stage by stage.  Inputs are numpy float32 arrays in HND layout
whose values are representable in ``dtype`` (bf16 or fp16).
"""
import numpy as np

from . import maskpred as mp
from . import vquant as vq
from . import attention as at
from .rounding import FP16

F32 = np.float32


def hyperparameter(h, value):
    """Scalar or (H,) -> (H,) float32 (spas_sage_attn/utils.py:38-50)."""
    a = np.asarray(value, dtype=F32)
    if a.ndim == 0:
        return np.full((h,), a, dtype=F32)
    assert a.ndim == 1 and a.size == h
    return a


def _common_tail(res, q, v, dtype, pvthreshd, scale, kernel_causal, qk_quant_gran=1):
    b, h, n, d = q.shape
    v16 = vq.to_fp16(v)
    v8, v_scale = vq.v_quant_fp8(v16)
    res["v8"], res["v_scale"] = v8, v_scale
    sm_scale = (1.0 / d ** 0.5) if scale is None else scale
    out, written, pvc = at.block_sparse_attention(
        res["q8"], res["k8"], v8, res["lut"], res["valid"], hyperparameter(h, pvthreshd),
        res["q_scale"], res["k_scale"], v_scale, sm_scale, dtype,
        is_causal=kernel_causal, return_pv_count=True, qk_quant_gran=qk_quant_gran)
    res["out"], res["written"], res["pv_count"] = out, written, pvc
    return res


def _q_rows(qk_quant_gran):
    """Rows of Q that share an INT8 scale: the 128-row block, or the 32 rows of a warp (quant_per_block.py:102-148)."""
    assert qk_quant_gran in (1, 2)
    return mp.BLKQ if qk_quant_gran == 1 else 32


def spas_sage2_attn_meansim_topk(q, k, v, dtype, is_causal=False, scale=None, simthreshd1=-0.1,
                                 cdfthreshd=None, topk=0.5, pvthreshd=50, attention_sink=False,
                                 kernel_causal=False, stop_after_mask=False, qk_quant_gran=1):
    """core.py:105-169.  ``kernel_causal`` is the flag the reference always passes as False (core.py:154-158);
    ``qk_quant_gran`` is the kernel's granularity argument, which the reference's operator fixes at 1 (core.py:156):
    with 2, Q is quantised in 32-row groups and the kernel reads one scale per warp."""
    q = np.asarray(q, dtype=F32)
    k = np.asarray(k, dtype=F32)
    b, h, n, d = q.shape
    assert n >= 128 and d in (64, 128)
    res = {}
    km = mp.km_mean(k, dtype)
    res["km"] = km
    thr = hyperparameter(h, simthreshd1)
    rq = mp.pool_sim_quant(q, None, mp.BLKQ, thr, dtype, quant_rows=_q_rows(qk_quant_gran))
    # grouped K/V heads (not in the reference, whose pooled-score matmul needs equal head counts): K is pooled once per
    # K head with the similarity threshold of the first query head of its group
    rk = mp.pool_sim_quant(k, km, mp.BLKK, thr[::h // k.shape[1]], dtype)
    res.update(pool_q=rq["pool"], sim_q=rq["sim"], q8=rq["q"], q_scale=rq["scale"],
               pool_k=rk["pool"], sim_k=rk["sim"], k8=rk["q"], k_scale=rk["scale"])
    fmap = mp.block_map(rq["pool"], rq["sim"], rk["pool"], rk["sim"], dtype, is_causal=is_causal,
                        topk=None if topk is None else hyperparameter(h, topk),
                        cdfthreshd=None if cdfthreshd is None else hyperparameter(h, cdfthreshd),
                        attention_sink=attention_sink)
    res["map"] = fmap
    res["lut"], res["valid"] = mp.map_to_lut(fmap)
    nq, nk = fmap.shape[2], fmap.shape[3]
    tot = float(res["valid"].astype(F32).sum())
    if is_causal is False:
        res["sparsity"] = 1 - tot / (nk * nq * b * h)
    else:
        res["sparsity"] = 1 - tot / ((nk + 2) // 2 * nq * b * h)       # core.py:166
    if stop_after_mask:
        return res
    return _common_tail(res, q, v, dtype, pvthreshd, scale, kernel_causal, qk_quant_gran)


def spas_sage_attn_meansim_topk(q, k, v, dtype, is_causal=False, scale=None, simthreshd1=-0.1, cdfthreshd=None,
                                topk=0.5, pvthreshd=50, attention_sink=False, qk_quant_gran=1):
    """core.py:278-319 (and 235-276 with cdfthreshd): the mask prediction of the Sage2 operator, then the INT8-QK /
    FP16-PV kernel on fp16(v) with the token-level causal flag (core.py:308-310)."""
    res = spas_sage2_attn_meansim_topk(q, k, v, dtype, is_causal=is_causal, scale=scale, simthreshd1=simthreshd1,
                                       cdfthreshd=cdfthreshd, topk=topk, attention_sink=attention_sink,
                                       stop_after_mask=True, qk_quant_gran=qk_quant_gran)
    q = np.asarray(q, dtype=F32)
    b, h, n, d = q.shape
    hkv, nkv = np.shape(v)[1], np.shape(v)[2]              # K/V may have fewer heads and another length than Q
    nk = (nkv + 63) // 64
    v16 = np.zeros((b, hkv, nk * 64, d), dtype=F32)
    v16[:, :, :nkv] = vq.to_fp16(v)
    res["v16"] = v16
    sm_scale = (1.0 / d ** 0.5) if scale is None else scale
    out, written, pvc = at.block_sparse_attention(
        res["q8"], res["k8"], v16, res["lut"], res["valid"], hyperparameter(h, pvthreshd), res["q_scale"],
        res["k_scale"], None, sm_scale, dtype, is_causal=bool(is_causal), return_pv_count=True, pv="f16",
        qk_quant_gran=qk_quant_gran)
    res["out"], res["written"], res["pv_count"] = out, written, pvc
    return res


def block_sparse_sage2_attn(q, k, v, mask_id, dtype, scale=None, pvthreshd=50, kernel_causal=False, qk_quant_gran=1):
    """core.py:171-233 (get_vanilla_qk_quant + block_map_lut_triton + kernel)."""
    q = np.asarray(q, dtype=F32)
    k = np.asarray(k, dtype=F32)
    b, h, n, d = q.shape
    assert n >= 128 and d in (64, 128)
    res = {}
    km = mp.km_mean(k, dtype)
    res["km"] = km
    rq = mp.pool_sim_quant(q, None, mp.BLKQ, None, dtype, with_pool=False, quant_rows=_q_rows(qk_quant_gran))
    rk = mp.pool_sim_quant(k, km, mp.BLKK, None, dtype, with_pool=False)
    res.update(q8=rq["q"], q_scale=rq["scale"], k8=rk["q"], k_scale=rk["scale"])
    res["lut"], res["valid"] = mp.map_to_lut(mask_id)
    nq, nk = res["lut"].shape[2], res["lut"].shape[3]
    res["sparsity"] = 1 - float(res["valid"].astype(F32).sum()) / ((nk + 2) // 2 * nq * b * h)  # core.py:230
    return _common_tail(res, q, v, dtype, pvthreshd, scale, kernel_causal, qk_quant_gran)
