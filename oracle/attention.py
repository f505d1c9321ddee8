"""Oracle for the block-sparse INT8-QK / FP8-PV attention kernel.  Test infrastructure only.

Blockwise numpy restatement of ``qk_int_sv_f8_block_sparse_attn_kernel``
(csrc/qattn/qk_int_sv_f8_cuda_sm89.cuh:42-755, instantiated with per-block
quantisation, per-block PV threshold, fp32 PV accumulation, fused V scale:
csrc/qattn/qk_int_sv_f8_cuda_sm89.cu:365) and of its helpers ``update_mo``,
``update_mdo``, ``exponentiate_r``, ``accumulate_d``, ``RS_32_to_8``,
``normalize_d``, ``apply_causal_mask``, ``apply_out_of_bound_mask``
(csrc/qattn/attn_utils.cuh:334-625, 757-811).

One Q block = 128 rows, one K/V block = 64 rows, visited in LUT order:
all blocks but the last two take the PV-threshold branch (sm89.cuh:277-464), the
second-last and last take the masked branch (sm89.cuh:467-648).  State per row:
m = -5e6, d = 1, O = 0.  Scores are integers (exact); softmax runs in binary32
base-2 with the +8.807 offset; P is rounded to e4m3 for the numerator while the
denominator sums the un-rounded P.

The reference uses ex2.approx / rcp.approx, so the output is only defined up to
tolerance; tests compare by cosine similarity >= 0.999 and relative L1 <= 1e-2.

Pinned by tests/test_oracle_attention.py: with every block selected and
pvthreshd = 50 it reduces to dense softmax attention on the dequantised
tensors (checked against torch SDPA in float64); with a block map it equals
SDPA under the token mask ``block_map_to_mask`` builds (utils.py:424-432);
pv_count == valid_block_num at threshold 50; the skip rule against a
hand-built two-scale example.  Parity unpinned: ex2/rcp approximation bits.
"""
import numpy as np

from .rounding import f32_to_e4m3fn, e4m3fn_to_f32, round_to

F32 = np.float32
LOG2E = F32(1.44269504088896340736)
S_FP8_OFFSET = F32(8.807)           # attn_utils.cuh:28
NEG_BIG = F32(-5000000.0)           # attn_utils.cuh:350, sm89.cuh:171
CTA_Q = 128
CTA_K = 64


def _exp2(x):
    with np.errstate(under="ignore"):
        return np.exp2(x.astype(F32)).astype(F32)


def _fma(a, b, c):
    return (a.astype(np.float64) * np.float64(b) + c.astype(np.float64)).astype(F32)


def block_sparse_attention(q8, k8, v8, lut, valid, pvthreshd, q_scale, k_scale, v_scale,
                           sm_scale, out_dtype, is_causal=False, return_pv_count=False, pv="fp8", pv_mode=1,
                           qk_quant_gran=1):
    """q8,k8 int8 (B,H,N,D); v8 e4m3 codes uint8 (B,H,Npad,D); lut/valid int32.

    Returns (out float32 (B,H,N,D) holding out_dtype values, written (B,H,nq) bool[, pv_count (B,H,nq)]).
    Row blocks with valid == 0 are left untouched (zeros here; sm89.cuh:232-235).
    ``pv_mode`` is the kernel template's PVThresholdMode (attn_utils.cuh:58-62): 1 = the skip is decided for the whole
    128-row block (what every Python entry point uses), 2 = for each warp of 32 rows on its own (sm89.cuh:302-318
    without the block reduction of 320-343; pv_count is then (B,H,nq,4)), 0 = never skip.

    ``qk_quant_gran`` is the kernel entry's granularity switch (csrc/qattn/attn_cuda.h:61-76): 1 = q_scale (B,H,nq), one
    scale per 128-row block; 2 = q_scale (B,H,nq*4), one per warp of 32 query rows, read at 4*block + row//32
    (sm89.cuh:111-115).  K scales are (B,Hkv,nk) in both (a K "warp" spans the whole 64-row block, sm89.cuh:123-131).

    ``pv="f16"`` restates the SageAttention1 kernel instead (qk_int_sv_f16_cuda_sm80.cuh:42-671 instantiated with
    per-block quantisation, per-block PV threshold and the row sum on the tensor cores, sm80.cuh:690): ``v8`` then holds
    fp16 VALUES (float array, (B,H,Npad,D), zero beyond N), ``v_scale`` is ignored, P has no exponent offset and is
    rounded to fp16 (RS_32_to_16, attn_utils.cuh:563-580), the denominator sums the ROUNDED P in binary32
    (accumulate_d on the tensor-core path, attn_utils.cuh:599-626) and the output is O / d.  The PV product is
    accumulated in binary32 here; the reference accumulates the four 16-key steps of a block in fp16 before adding
    the block to its binary32 accumulator (compute_fp16_sv_permuted_inst_buf, attn_utils.cuh:683-751) - parity
    unpinned for that rounding, the comparison is by tolerance.
    """
    assert pv in ("fp8", "f16") and pv_mode in (0, 1, 2) and qk_quant_gran in (1, 2)
    q8 = np.asarray(q8)
    k8 = np.asarray(k8)
    b_, h_, n, d_ = q8.shape
    nkv = k8.shape[2]
    groups = h_ // k8.shape[1]            # grouped-query attention: K/V head = query head // groups (sm89.cuh:118)
    nq = (n + CTA_Q - 1) // CTA_Q
    vf = e4m3fn_to_f32(v8) if pv == "fp8" else np.asarray(v8, dtype=F32)
    offset = S_FP8_OFFSET if pv == "fp8" else F32(0.0)
    c = F32(F32(sm_scale) * LOG2E)
    out = np.zeros((b_, h_, n, d_), dtype=F32)
    written = np.zeros((b_, h_, nq), dtype=bool)
    pv_count = np.zeros((b_, h_, nq, 4), dtype=np.int32)
    for b in range(b_):
        for h in range(h_):
            thr = F32(pvthreshd[h])
            hk = h // groups
            for i in range(nq):
                nv = int(valid[b, h, i])
                if nv == 0:
                    continue
                written[b, h, i] = True
                r0 = i * CTA_Q
                rows = min(CTA_Q, n - r0)
                qb = np.zeros((CTA_Q, d_), dtype=np.float64)
                qb[:rows] = q8[b, h, r0:r0 + rows]
                q_idx = r0 + np.arange(CTA_Q)
                m = np.full(CTA_Q, NEG_BIG, dtype=F32)
                dsum = np.ones(CTA_Q, dtype=F32)
                o = np.zeros((CTA_Q, d_), dtype=F32)
                idxs = np.cumsum(lut[b, h, i, :nv].astype(np.int64))
                if qk_quant_gran == 1:
                    qs = np.full(CTA_Q, q_scale[b, h, i], dtype=F32)
                else:
                    qs = np.repeat(np.asarray(q_scale[b, h, 4 * i:4 * i + 4], dtype=F32), 32)
                cnt = np.zeros(4, dtype=np.int32)
                for it, j in enumerate(idxs):
                    c0 = int(j) * CTA_K
                    cols = max(0, min(CTA_K, nkv - c0))
                    kb = np.zeros((CTA_K, d_), dtype=np.float64)
                    kb[:cols] = k8[b, hk, c0:c0 + cols]
                    vb = vf[b, hk, c0:c0 + CTA_K]
                    s = (qb @ kb.T).astype(F32)                 # exact integers
                    dq = (qs * F32(k_scale[b, hk, j])).astype(F32)[:, None]      # per query row
                    if it < nv - 2:
                        a = (c * dq).astype(F32)
                        m_blk = (s.max(axis=1) * a[:, 0]).astype(F32)
                        d_row = (m_blk - m).astype(F32)
                        if pv_mode == 1:
                            act4 = np.full(4, bool(F32(np.max(d_row) + thr) > 0))
                        elif pv_mode == 2:
                            act4 = (d_row.reshape(4, 32).max(axis=1) + thr).astype(F32) > 0
                        else:
                            act4 = np.ones(4, dtype=bool)
                        m_new = np.maximum(m, m_blk)
                        o_scale = _exp2(m - m_new)
                        dsum = (dsum * o_scale).astype(F32)
                        o = (o * o_scale[:, None]).astype(F32)
                        m = m_new
                        if not act4.any():
                            continue
                        neg_m = (-m + offset).astype(F32)
                        p = _exp2(_fma(s, a, neg_m[:, None]))
                    else:
                        act4 = np.ones(4, dtype=bool)
                        sf = (s * dq).astype(F32)
                        k_idx = c0 + np.arange(CTA_K)
                        if is_causal:
                            sf = np.where(k_idx[None, :] > q_idx[:, None], NEG_BIG, sf)
                        if it == nv - 1:
                            sf = np.where(k_idx[None, :] >= nkv, NEG_BIG, sf)
                        m_blk = (sf.max(axis=1) * c).astype(F32)
                        m_new = np.maximum(m, m_blk)
                        o_scale = _exp2(m - m_new)
                        dsum = (dsum * o_scale).astype(F32)
                        o = (o * o_scale[:, None]).astype(F32)
                        m = m_new
                        neg_m = (-m + offset).astype(F32)
                        p = _exp2(_fma(sf, c, neg_m[:, None]))
                    cnt += act4
                    act = np.repeat(act4, 32)
                    if pv == "fp8":
                        dsum = np.where(act, (dsum + p.sum(axis=1, dtype=F32)).astype(F32), dsum)
                        p8 = e4m3fn_to_f32(f32_to_e4m3fn(p))
                    else:
                        p8 = round_to(p.astype(np.float64), "fp16").astype(F32)
                        dsum = np.where(act, (dsum + p8.sum(axis=1, dtype=F32)).astype(F32), dsum)
                    o = np.where(act[:, None], (o + (p8 @ vb).astype(F32)).astype(F32), o)
                pv_count[b, h, i] = cnt
                res = (o / dsum[:, None]).astype(F32)
                if pv == "fp8":
                    res = res * np.asarray(v_scale[b, hk], dtype=F32)[None, :]
                out[b, h, r0:r0 + rows] = round_to(res[:rows].astype(np.float64), out_dtype)
    if return_pv_count:
        return out, written, (pv_count if pv_mode == 2 else pv_count[..., 0])
    return out, written


def precision_metric(x, ref):
    """cosine similarity, relative L1, RMSE (spas_sage_attn/utils.py:25-36, without the rounding)."""
    x = np.asarray(x, dtype=np.float64).ravel()
    y = np.asarray(ref, dtype=np.float64).ravel()
    cos = float(np.dot(x, y) / (np.linalg.norm(x) * np.linalg.norm(y)))
    l1 = float(np.abs(x - y).sum() / np.abs(y).sum())
    rmse = float(np.sqrt(np.mean((x - y) ** 2)))
    return {"Cossim": cos, "L1": l1, "RMSE": rmse}
