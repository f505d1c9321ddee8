"""Oracle for sparse-mask prediction and INT8 Q/K quantisation.  Test infrastructure only.

Restates (numpy, CPU) the reference functions

* ``k.mean(dim=-2, keepdim=True)``                      spas_sage_attn/core.py:119-120
* ``triton_bmm_pool_sim_simmean_fuse_quant``            spas_sage_attn/utils.py:161-214
* ``qk_quantize``                                       spas_sage_attn/utils.py:89-159
* ``get_block_map_meansim_fuse_quant`` (torch glue)     spas_sage_attn/utils.py:371-421
* ``triton_fill_causal_mask``                           spas_sage_attn/utils.py:304-316
* ``triton_fill_block_map_kernel``                      spas_sage_attn/utils.py:282-302
* ``triton_block_map_to_lut_kernel``                    spas_sage_attn/utils.py:54-87

under the arithmetic contract stated in ``oracle/__init__.py``.

T-typed tensors are float32 numpy arrays holding values representable in T.

Pinning (tests/test_oracle_maskpred.py):
* ``km_mean``      - torch.mean in float64 then one rounding; closed forms.
* quantisation     - round-trip bound |x - q*s| <= s/2 (+1 ulp), max|q| = 127
                     attained, sign symmetry, brute-force scalar loop.
* pooling / sim    - identity mean(gram) = ||sum x_hat||^2 / BS^2 against an
                     explicit float64 gram matrix; constant block => sim 1;
                     partial block => False (0/0 NaN, utils.py:179-199).
* softmax          - ``cexp`` against numpy.exp (<= 2 ulp); rounded
                     probabilities against torch.softmax(float64) rounded to T.
* selection / map  - brute-force stable argsort on tiny inputs; row-count
                     invariants (utils.py:405-415).
* LUT              - ascending-index / first-difference closed form, and the
                     dense restatement the reference itself ships
                     (``block_map_lut``, utils.py:434-447) reproduced in the test.
Parity unpinned: the bit patterns of the real Triton/cuBLAS/ATen run
(approximate fp32 divide, tl.sum / tl.dot order, cuBLAS accumulation order,
torch.sort tie order).  No reference test or golden vector exists for them;
the contract above replaces them.
"""
import numpy as np

from .rounding import round_to, bits16, BF16, FP16

F32 = np.float32
F64 = np.float64

BLKQ = 128
BLKK = 64

# --------------------------------------------------------------------------
# canonical exp / softmax
# --------------------------------------------------------------------------
_LOG2E = F64(1.4426950408889634)
_LN2_HI = F64(0.6931471803691238)      # upper 33 bits of ln 2
_LN2_LO = F64(1.9082149292705877e-10)  # ln 2 - _LN2_HI
_EXP_COEF = [F64(1.0) / F64(np.prod(np.arange(1, n + 1, dtype=np.float64))) if n else F64(1.0) for n in range(14)]
_EXP_MIN = F64(-700.0)
WAVE = 64         # width of the fixed summation tree (one GPU wavefront)


def cexp(t):
    """exp(t) for t <= 0 as a FIXED sequence of binary64 mul/add (no fma).

    k = rint(t*log2e); r = (t - k*ln2_hi) - k*ln2_lo; Horner degree 13 with
    coefficients 1/n!; result scaled by 2**k.  t < -700 (and -inf) -> 0.
    """
    t = np.asarray(t, dtype=F64)
    tz = np.where(t >= _EXP_MIN, t, 0.0)
    k = np.rint(tz * _LOG2E)
    r = (tz - k * _LN2_HI) - k * _LN2_LO
    p = np.full_like(r, _EXP_COEF[13])
    for n in range(12, -1, -1):
        p = p * r
        p = p + _EXP_COEF[n]
    y = np.ldexp(p, k.astype(np.int64))
    return np.where(t >= _EXP_MIN, y, 0.0)


def _butterfly(acc, width):
    """xor-butterfly over the last axis (offsets width/2 .. 1); every lane ends with the same value."""
    idx = np.arange(width)
    off = width // 2
    while off >= 1:
        acc = acc + acc[..., idx ^ off]
        off //= 2
    return acc[..., 0]


def tree_sum(e):
    """Sum along the last axis with the fixed tree the GPU kernel uses.

    Lane l of 64 adds elements l, l+64, ... in ascending order; the 64 partial sums are combined by an
    xor-butterfly (offsets 32,16,8,4,2,1).
    """
    e = np.asarray(e, dtype=F64)
    n = e.shape[-1]
    nchunk = (n + WAVE - 1) // WAVE
    pad = nchunk * WAVE - n
    if pad:
        e = np.concatenate([e, np.zeros(e.shape[:-1] + (pad,), dtype=F64)], axis=-1)
    e = e.reshape(e.shape[:-1] + (nchunk, WAVE))
    acc = np.zeros(e.shape[:-2] + (WAVE,), dtype=F64)
    for c in range(nchunk):
        acc = acc + e[..., c, :]
    return _butterfly(acc, WAVE)


def softmax_T(score, dtype):
    """softmax over the last axis of T-typed scores (may hold -inf) -> T (utils.py:396)."""
    s = np.asarray(score, dtype=F64)
    m = np.max(s, axis=-1, keepdims=True)
    with np.errstate(invalid="ignore"):
        t = np.where(np.isneginf(s), -np.inf, s - m)
    e = cexp(t)
    tot = tree_sum(e)[..., None]
    with np.errstate(invalid="ignore", divide="ignore"):
        p = e / tot
    p = np.where(np.isfinite(p), p, 0.0)   # all--inf row: defined as 0 (map is all-ones there anyway)
    return round_to(p, dtype)


# --------------------------------------------------------------------------
# A2: K column mean
# --------------------------------------------------------------------------

def km_mean(k, dtype):
    """km[b,h,d] = (sum_n k[b,h,n,d]) / N rounded once to T (core.py:120).  Shape (B,H,D)."""
    k = np.asarray(k, dtype=F64)
    n = k.shape[-2]
    return round_to(k.sum(axis=-2) / F64(n), dtype)


# --------------------------------------------------------------------------
# A3 / A4 / A13: pool + sim + per-block INT8 quantisation
# --------------------------------------------------------------------------

def _blocked(x, bs):
    b, h, n, d = x.shape
    nb = (n + bs - 1) // bs
    pad = nb * bs - n
    if pad:
        x = np.concatenate([x, np.zeros((b, h, pad, d), dtype=x.dtype)], axis=2)
    rows_valid = np.minimum(bs, n - np.arange(nb) * bs)
    valid = (np.arange(nb * bs) < n).reshape(nb, bs)
    return x.reshape(b, h, nb, bs, d), rows_valid, valid


def smooth(x, km, dtype):
    """(x - km) rounded once to T (utils.py:184-188; bf16 - bf16 -> bf16)."""
    return round_to(np.asarray(x, F64) - np.asarray(km, F64)[:, :, None, :], dtype)


def quant_int8_block(xb):
    """Per-block INT8 quantisation of xb (..., BS, D) float32 (utils.py:140-148 / 206-210).

    s = max|x|/127 + 1e-7 ; y = x/s ; y += 0.5*sign ; truncate.  All in binary32.
    Returns (int8 array, float32 scale (...)).
    """
    xb = np.asarray(xb, dtype=F32)
    # tl.max lowers to a maxnum: NaN elements do not take part in the block maximum (an all-NaN block is not defined)
    amax = np.fmax.reduce(np.fmax.reduce(np.abs(xb), axis=-1, initial=F32(0)), axis=-1, initial=F32(0))
    scale = (amax / F32(127.0)).astype(F32)
    scale = (scale + F32(1e-7)).astype(F32)
    with np.errstate(invalid="ignore"):
        y = (xb / scale[..., None, None]).astype(F32)
        y = (y + np.where(y >= 0, F32(0.5), F32(-0.5)).astype(F32)).astype(F32)
        q = np.where(np.isnan(y), F32(0), np.trunc(y)).astype(np.int32).astype(np.int8)   # a NaN converts to 0
    return q, scale


def pool_sim_quant(x, km, bs, simthreshd1, dtype, with_pool=True, quant_rows=None):
    """One pass of the fused Triton kernel over x (B,H,N,D) T-typed float32.

    km: (B,H,D) T-typed or None.  simthreshd1: (H,) float32.
    Returns dict(pool (B,H,nb,D) T, sim (B,H,nb) bool, q (B,H,N,D) int8, scale (B,H,nb) f32).
    With ``with_pool=False`` this is ``qk_quantize`` (utils.py:89-159): q and scale only.

    ``quant_rows`` (a divisor of ``bs``; default ``bs``) is the number of rows that share one INT8 scale.  32 with
    bs = 128 is the per-warp granularity of Q: ``per_warp_int8`` (spas_sage_attn/quant_per_block.py:102-148) launches
    the same per-group arithmetic (quant_per_block.py:41-48 = utils.py:140-148) over nb * bs / 32 groups per head, a
    group past the end of the tensor included (all masked -> scale 1e-7); scale is then (B,H,nb*bs/quant_rows).
    Pooling and the similarity flag are per block of ``bs`` rows whatever the granularity.
    """
    x = np.asarray(x, dtype=F32)
    b, h, n, d = x.shape
    if km is not None:
        x = smooth(x, km, dtype)
    xb, rows_valid, valid = _blocked(x, bs)
    xb = np.where(valid[None, None, :, :, None], xb, F32(0))   # utils.py:188 (re-zero masked rows)
    nb = xb.shape[2]
    qr = bs if quant_rows is None else int(quant_rows)
    assert qr > 0 and bs % qr == 0
    q, scale = quant_int8_block(xb.reshape(b, h, nb * (bs // qr), qr, d))
    out = {"q": q.reshape(b, h, nb * bs, d)[:, :, :n, :], "scale": scale}
    if not with_pool:
        return out

    x64 = xb.astype(F64)
    pool = round_to(x64.sum(axis=3) / rows_valid[None, None, :, None].astype(F64), dtype)

    ss = (x64 * x64).sum(axis=-1)                       # exact in binary64
    norm = np.sqrt(ss.astype(F32))                      # binary32 sqrt (utils.py:194)
    with np.errstate(invalid="ignore", divide="ignore"):
        xhat = (xb / norm[..., None]).astype(F32).astype(np.float16)   # utils.py:195
    finite = np.isfinite(xhat).all(axis=(3, 4))
    xi = np.where(np.isfinite(xhat), xhat, 0).astype(F64) * 2.0 ** 24   # fp16 -> exact integer (unit 2**-24)
    xi = xi.astype(np.int64)
    s = xi.sum(axis=3)                                   # (B,H,nb,D) exact
    g = (s * s).sum(axis=-1)                             # = sum(gram) * 2**48, exact in int64
    thr = np.asarray(simthreshd1, dtype=F32).astype(F64)[None, :, None]
    rv2 = (rows_valid.astype(F64) ** 2)[None, None, :]
    sim = (g.astype(F64) > thr * rv2 * 2.0 ** 48) & finite   # NaN > t is False (utils.py:198-199)
    out["pool"] = pool
    out["sim"] = sim
    return out


# --------------------------------------------------------------------------
# A5-A7: compressed attention, selection, block map
# --------------------------------------------------------------------------

def pooled_scores(pool_q, pool_k, dtype):
    """(pooledQ @ pooledK^T) -> T, then * fp32(D**-0.5) -> T (utils.py:388).

    Fixed order of the dot product: binary64 accumulation over d = 0, 1, ..., D-1.  (Products of two T values are
    exact in binary64.)
    """
    pq = np.asarray(pool_q, dtype=F64)
    pk = np.asarray(pool_k, dtype=F64)
    d = pq.shape[-1]
    acc = np.zeros(pq.shape[:-1] + (pk.shape[-2],), dtype=F64)
    for i in range(d):
        acc = acc + pq[..., :, i, None] * pk[..., None, :, i]
    s1 = round_to(acc, dtype)
    return round_to(s1.astype(F64) * F64(F32(d ** -0.5)), dtype)


def causal_block_mask(nq, nk):
    """mask[q,k] = k < (q+1)*(BLKQ/BLKK) (utils.py:304-316)."""
    return np.arange(nk)[None, :] < (np.arange(nq)[:, None] + 1) * (BLKQ // BLKK)


def stable_desc_rank(p, dtype):
    """rank[..., j] = position of column j in a stable descending sort of p (>=0, T-typed)."""
    nk = p.shape[-1]
    assert nk <= 0xFFFF
    key = (bits16(p, dtype).astype(np.uint32) << np.uint32(16)) | (np.uint32(0xFFFF) - np.arange(nk, dtype=np.uint32))
    order = np.argsort(-key.astype(np.int64), axis=-1, kind="stable")
    rank = np.empty_like(order)
    np.put_along_axis(rank, order, np.broadcast_to(np.arange(nk), order.shape), axis=-1)
    return rank, order


def num_to_select_topk(topk, nk):
    """(topk * K).to(int64) with the product in binary32 (utils.py:405)."""
    t = np.asarray(topk, dtype=F32)
    return np.trunc((t * F32(nk)).astype(F32)).astype(np.int64)


def num_to_select_cdf(p, order, cdfthreshd, dtype):
    """cumsum of the sorted probabilities rounded to T, then searchsorted(right=True) (utils.py:398-403).

    cdf[i] is the EXACT running sum rounded once to T, compared with the binary32 threshold.  Pinned by
    tests/test_oracle_cdf_pin.py against the routines the reference calls (torch.sort -> torch.cumsum ->
    torch.searchsorted(right=True)) on CPU tensors of dtype T: torch's CPU scan accumulates in binary32 and rounds every
    prefix once, and the counts agree on random rows, long flat rows and thresholds on / beside cdf values.
    What stays open is the CUDA scan of the same call: if it combines partial sums in T (a rounding per combine step),
    a long flat bf16 row stalls below 1 and counts MORE blocks for the same threshold, so a cdfthreshd tuned with the
    CUDA reference may select fewer blocks here.

    p (B,H,nq,nk); cdfthreshd (H,) float32.  Returns int64 (B,H,nq).
    """
    ps = np.take_along_axis(np.asarray(p, F64), order, axis=-1)
    cdf = round_to(np.cumsum(ps, axis=-1), dtype).astype(F64)
    thr = np.asarray(cdfthreshd, dtype=F32).astype(F64)[None, :, None, None]
    return (cdf <= thr).sum(axis=-1).astype(np.int64)


def block_map(pool_q, sim_q, pool_k, sim_k, dtype, is_causal=False, topk=None, cdfthreshd=None,
              attention_sink=False, return_probs=False):
    """Steps 4-8: boolean block map (B,H,nq,nk) (utils.py:386-415).

    pool_k / sim_k may carry fewer heads than pool_q (grouped K/V heads, an extension the reference's matmul at
    utils.py:388 does not have): query head h then uses K head h // (H / Hkv), i.e. the K tensors repeated per group."""
    assert (topk is None) != (cdfthreshd is None), "Only one of cdfthreshd and topk can be set."
    b, h, nq, _ = pool_q.shape
    nk = pool_k.shape[2]
    if pool_k.shape[1] != h:
        assert h % pool_k.shape[1] == 0
        pool_k = np.repeat(pool_k, h // pool_k.shape[1], axis=1)
        sim_k = np.repeat(sim_k, h // sim_k.shape[1], axis=1)
    score = pooled_scores(pool_q, pool_k, dtype).astype(F32)
    score = np.where(sim_k[:, :, None, :], score, -np.inf)
    cm = causal_block_mask(nq, nk)
    if is_causal:
        score = np.where(cm[None, None], score, -np.inf)
    p = softmax_T(score, dtype)
    rank, order = stable_desc_rank(p, dtype)
    if topk is not None:
        n = np.broadcast_to(num_to_select_topk(topk, nk)[None, :, None], (b, h, nq))
    else:
        n = num_to_select_cdf(p, order, cdfthreshd, dtype)
    n = np.where(n == 0, 1, n)                              # utils.py:289
    fmap = rank < n[..., None]
    fmap = fmap | ~sim_k[:, :, None, :] | ~sim_q[:, :, :, None]
    if is_causal:
        fmap = fmap & cm[None, None]
    if attention_sink:
        fmap = fmap.copy()
        fmap[..., 0] = True
    if return_probs:
        return fmap, p
    return fmap


# --------------------------------------------------------------------------
# A8: block map -> delta LUT
# --------------------------------------------------------------------------

def map_to_lut(block_map_):
    """lut[..., c] = idx_c - idx_{c-1} over ascending set columns (idx_{-1} = 0); tail 0 (utils.py:54-87)."""
    m = np.asarray(block_map_) != 0
    nk = m.shape[-1]
    valid = m.sum(axis=-1).astype(np.int32)
    # ascending indices of set columns, packed to the front
    key = np.where(m, np.arange(nk), nk + np.arange(nk))
    idx = np.sort(key, axis=-1)
    sel = np.arange(nk) < valid[..., None]
    idx = np.where(sel, idx, 0)
    prev = np.concatenate([np.zeros(idx.shape[:-1] + (1,), idx.dtype), idx[..., :-1]], axis=-1)
    lut = np.where(sel, idx - prev, 0).astype(np.int32)
    return lut, valid


def lut_to_indices(lut_row, valid):
    """Absolute K-block indices encoded by one LUT row."""
    return np.cumsum(np.asarray(lut_row[:valid], dtype=np.int64))
