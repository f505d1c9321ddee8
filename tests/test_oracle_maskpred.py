"""Pins oracle/maskpred.py: library routines, closed forms, brute force on tiny inputs."""
import math

import numpy as np
import pytest
import torch

from oracle import maskpred as mp
from oracle import rounding as R


def _t(x, tag):
    """float64/32 array -> T-typed float32 array."""
    return R.round_to(np.asarray(x, dtype=np.float64), tag)


@pytest.mark.parametrize("tag", [R.BF16, R.FP16])
def test_km_mean_against_torch_float64(tag):
    rng = np.random.default_rng(0)
    k = _t(rng.standard_normal((2, 3, 1000, 64)) + 0.3, tag)
    got = mp.km_mean(k, tag)
    ref64 = torch.from_numpy(k).double().mean(dim=-2).numpy()
    assert np.array_equal(got, R.round_to(ref64, tag))
    # closed form: constant column -> that constant; alternating +-c -> 0
    c = _t(np.full((1, 1, 512, 64), 0.3), tag)
    assert np.array_equal(mp.km_mean(c, tag), c[:, :, 0, :])
    alt = c * np.where(np.arange(512) % 2 == 0, 1, -1)[None, None, :, None]
    assert np.all(mp.km_mean(alt, tag) == 0)


def _quant_scalar(block):
    """Element-by-element restatement in Python floats rounded to binary32 at each step."""
    f = np.float32
    amax = f(0)
    for v in block.ravel():
        amax = max(amax, abs(f(v)))
    s = f(f(amax / f(127.0)) + f(1e-7))
    out = np.zeros(block.shape, dtype=np.int8)
    for idx, v in np.ndenumerate(block):
        y = f(f(v) / s)
        y = f(y + (f(0.5) if y >= 0 else f(-0.5)))
        out[idx] = int(y)          # int() truncates toward zero
    return out, s


def test_quant_bruteforce_and_bounds():
    rng = np.random.default_rng(1)
    x = _t(rng.standard_normal((3, 16, 32)) * np.array([1e-3, 1.0, 50.0])[:, None, None], R.BF16)
    q, s = mp.quant_int8_block(x)
    for i in range(3):
        qb, sb = _quant_scalar(x[i])
        assert np.array_equal(q[i], qb) and s[i] == sb
    # the block maximum maps to +-127 unless the +1e-7 in the scale is not negligible (first block: amax ~ 3e-3)
    assert list(np.abs(q.astype(np.int32)).max(axis=(1, 2))) == [126, 127, 127]
    err = np.abs(x.astype(np.float64) - q.astype(np.float64) * s[:, None, None].astype(np.float64))
    assert np.all(err <= 0.5 * s[:, None, None] * (1 + 1e-5))             # round-to-nearest bound
    q2, s2 = mp.quant_int8_block(-x)                                       # sign symmetry
    assert np.array_equal(q2, -q) and np.array_equal(s2, s)
    qz, sz = mp.quant_int8_block(np.zeros((1, 4, 8), np.float32))          # all-zero block
    assert np.all(qz == 0) and sz[0] == np.float32(1e-7)


@pytest.mark.parametrize("tag", [R.BF16, R.FP16])
def test_pool_sim_quant_against_explicit_gram(tag):
    rng = np.random.default_rng(2)
    b, h, n, d, bs = 1, 2, 300, 64, 128            # last block is partial (44 rows)
    x = _t(rng.standard_normal((b, h, n, d)) + 0.5, tag)
    km = mp.km_mean(x, tag)
    thr = np.array([0.1, 0.35], dtype=np.float32)
    res = mp.pool_sim_quant(x, km, bs, thr, tag)
    xs = R.round_to(x.astype(np.float64) - km.astype(np.float64)[:, :, None, :], tag)
    for hh in range(h):
        for blk in range(3):
            rows = xs[0, hh, blk * bs:(blk + 1) * bs].astype(np.float64)
            nv = rows.shape[0]
            assert np.array_equal(res["pool"][0, hh, blk], R.round_to(rows.sum(0) / nv, tag))
            norm = np.sqrt((rows * rows).sum(1).astype(np.float32))
            xhat = (rows.astype(np.float32) / norm[:, None]).astype(np.float16).astype(np.float64)
            gram_mean = (xhat @ xhat.T).sum() / (nv * nv)       # exact enough in float64 to be far from thr
            if nv == bs:
                assert res["sim"][0, hh, blk] == (gram_mean > np.float64(thr[hh]))
            else:
                assert not res["sim"][0, hh, blk]               # zero rows -> 0/0 -> NaN -> False
            qb, sb = mp.quant_int8_block(rows.astype(np.float32) if nv == bs else
                                         np.concatenate([rows, np.zeros((bs - nv, d))]).astype(np.float32))
            assert np.array_equal(res["q"][0, hh, blk * bs:blk * bs + nv], qb[:nv])
            assert res["scale"][0, hh, blk] == sb
    assert res["q"].shape == (b, h, n, d)


def test_sim_closed_forms():
    d, bs = 64, 64
    base = R.round_to(np.random.default_rng(3).standard_normal(d), R.BF16)
    const = np.broadcast_to(base, (1, 1, bs, d)).copy()
    r = mp.pool_sim_quant(const, None, bs, np.array([0.99], np.float32), R.BF16)
    assert r["sim"].all() and np.array_equal(r["pool"][0, 0, 0], base)       # identical rows: mean cos = 1
    anti = const * np.where(np.arange(bs) % 2 == 0, 1, -1)[None, None, :, None]
    r = mp.pool_sim_quant(anti, None, bs, np.array([1e-6], np.float32), R.BF16)
    assert not r["sim"].any() and np.all(r["pool"] == 0)                     # sum of x_hat is exactly 0
    r = mp.pool_sim_quant(anti, None, bs, np.array([-0.1], np.float32), R.BF16)
    assert r["sim"].all()                                                     # mean(gram) >= 0 > -0.1
    r = mp.pool_sim_quant(const[:, :, :40], None, bs, np.array([-0.1], np.float32), R.BF16)
    assert not r["sim"].any()                                                 # partial block
    assert np.array_equal(r["pool"][0, 0, 0], base)                           # divides by valid rows


def test_cexp_and_tree_sum():
    t = -np.concatenate([np.linspace(0, 50, 20001), np.random.default_rng(4).random(20000) * 700])
    got = mp.cexp(t)
    ref = np.exp(t)
    assert np.all(np.abs(got - ref) <= 2 * np.spacing(ref))
    assert mp.cexp(np.array([0.0]))[0] == 1.0
    assert np.all(mp.cexp(np.array([-701.0, -1e9, -np.inf])) == 0)
    # tree_sum: explicit lane-by-lane restatement
    rng = np.random.default_rng(5)
    e = rng.random((3, 700)) * 10.0 ** rng.integers(-12, 3, (3, 700))
    for row in range(3):
        lanes = [0.0] * 64
        for j, v in enumerate(e[row]):
            lanes[j % 64] = lanes[j % 64] + float(v)
        a = lanes
        for off in (32, 16, 8, 4, 2, 1):
            a = [a[i] + a[i ^ off] for i in range(64)]
        assert len(set(a)) == 1
        assert mp.tree_sum(e)[row] == a[0]
        assert abs(a[0] - math.fsum(e[row])) <= 1e-13 * a[0]


@pytest.mark.parametrize("tag", [R.BF16, R.FP16])
def test_softmax_against_torch_float64(tag):
    rng = np.random.default_rng(6)
    s = _t(rng.standard_normal((4, 5, 300)) * 6, tag)
    s[0, 0, 10:40] = -np.inf
    got = mp.softmax_T(s, tag)
    ref = torch.softmax(torch.from_numpy(s).double(), dim=-1).numpy()
    assert np.array_equal(got, R.round_to(ref, tag))
    assert np.all(got[0, 0, 10:40] == 0)


def test_pooled_scores_against_float64_matmul():
    rng = np.random.default_rng(7)
    for tag, d in ((R.BF16, 128), (R.FP16, 64)):
        pq = _t(rng.standard_normal((1, 2, 9, d)), tag)
        pk = _t(rng.standard_normal((1, 2, 17, d)), tag)
        got = mp.pooled_scores(pq, pk, tag)
        mm = torch.from_numpy(pq).double() @ torch.from_numpy(pk).double().transpose(-1, -2)
        s1 = R.round_to(mm.numpy(), tag).astype(np.float64)
        ref = R.round_to(s1 * np.float64(np.float32(d ** -0.5)), tag)
        assert np.array_equal(got, ref)


def test_stable_rank_bruteforce_with_ties():
    rng = np.random.default_rng(8)
    p = _t(rng.integers(0, 4, (5, 40)) / 8.0, R.BF16)       # many exact ties
    rank, order = mp.stable_desc_rank(p, R.BF16)
    for r in range(5):
        brute = sorted(range(40), key=lambda j: (-float(p[r, j]), j))
        assert list(order[r]) == brute
        assert [int(rank[r, j]) for j in brute] == list(range(40))


def test_num_to_select():
    assert list(mp.num_to_select_topk(np.array([0.5, 0.3, 0.0, 1.0], np.float32), 1857)) == \
        [int(np.float32(0.5) * np.float32(1857)), 557, 0, 1857]
    assert mp.num_to_select_topk(np.array([0.5], np.float32), 512)[0] == 256
    # cdf mode: p sorted = [.5,.25,.125,.125]; cdf = [.5,.75,.875,1.0]
    p = np.array([[[[0.125, 0.5, 0.25, 0.125]]]], np.float32)
    _, order = mp.stable_desc_rank(p, R.BF16)
    for thr, n in ((0.4, 0), (0.5, 1), (0.8, 2), (0.875, 3), (1.0, 4)):
        assert mp.num_to_select_cdf(p, order, np.array([thr], np.float32), R.BF16)[0, 0, 0] == n


def _rand_pools(rng, b, h, nq, nk, d, tag):
    pq = _t(rng.standard_normal((b, h, nq, d)), tag)
    pk = _t(rng.standard_normal((b, h, nk, d)), tag)
    return pq, pk


def test_block_map_invariants_noncausal():
    rng = np.random.default_rng(9)
    b, h, nq, nk, d = 1, 3, 8, 16, 64
    pq, pk = _rand_pools(rng, b, h, nq, nk, d, R.BF16)
    sim_q = np.ones((b, h, nq), bool); sim_q[0, 1, 3] = False
    sim_k = np.ones((b, h, nk), bool); sim_k[0, 2, 5] = False
    topk = np.array([0.5, 0.25, 0.01], np.float32)
    fm, p = mp.block_map(pq, sim_q, pk, sim_k, R.BF16, topk=topk, return_probs=True)
    n = [8, 4, 1]                                          # floor(topk*16), min 1
    for hh in range(h):
        for i in range(nq):
            row = fm[0, hh, i]
            if not sim_q[0, hh, i]:
                assert row.all()
                continue
            forced = ~sim_k[0, hh]
            assert row[forced].all()
            top = sorted(range(nk), key=lambda j: (-float(p[0, hh, i, j]), j))[:n[hh]]
            expect = np.zeros(nk, bool); expect[top] = True
            assert np.array_equal(row, expect | forced)
            assert p[0, hh, i][forced].sum() == 0          # -inf columns carry no probability
    fm2 = mp.block_map(pq, sim_q, pk, sim_k, R.BF16, topk=topk, attention_sink=True)
    assert fm2[..., 0].all() and np.array_equal(fm2[..., 1:], fm[..., 1:])


def test_block_map_causal_counts():
    rng = np.random.default_rng(10)
    b, h, nq, nk, d = 1, 2, 16, 32, 64
    pq, pk = _rand_pools(rng, b, h, nq, nk, d, R.FP16)
    ones_q, ones_k = np.ones((b, h, nq), bool), np.ones((b, h, nk), bool)
    fm = mp.block_map(pq, ones_q, pk, ones_k, R.FP16, is_causal=True, topk=np.array([0.5, 0.5], np.float32))
    cm = mp.causal_block_mask(nq, nk)
    assert not (fm & ~cm[None, None]).any()
    for i in range(nq):
        assert np.all(fm[0, :, i].sum(-1) == min(2 * (i + 1), 16))
    assert cm[0].sum() == 2 and cm[-1].all()
    # CDF mode with threshold 1.0 selects everything causal-valid that has probability mass
    fm = mp.block_map(pq, ones_q, pk, ones_k, R.FP16, is_causal=True, cdfthreshd=np.array([2.0, 2.0], np.float32))
    assert np.array_equal(fm, np.broadcast_to(cm, fm.shape))


def _lut_scan(row):
    """Sequential scan, the definition of the encoding (one thread walks the row)."""
    lut, prev, cnt = [0] * len(row), 0, 0
    for i, v in enumerate(row):
        if v:
            lut[cnt] = i - prev
            cnt += 1
            prev = i
    return lut, cnt


def test_map_to_lut_bruteforce_and_closed_form():
    rng = np.random.default_rng(11)
    m = rng.random((2, 3, 5, 37)) < 0.3
    m[0, 0, 0] = False                         # empty row
    m[0, 0, 1] = True                          # full row
    m[0, 0, 2] = False; m[0, 0, 2, 36] = True  # only the last column
    lut, valid = mp.map_to_lut(m.astype(np.int32))
    for idx in np.ndindex(2, 3, 5):
        l, c = _lut_scan(m[idx])
        assert list(lut[idx]) == l and valid[idx] == c
        assert list(mp.lut_to_indices(lut[idx], valid[idx])) == list(np.flatnonzero(m[idx]))
    assert lut.dtype == np.int32 and valid.dtype == np.int32
    # any non-zero value counts as set (float / negative entries)
    lut2, valid2 = mp.map_to_lut(np.where(m, -2.5, 0.0))
    assert np.array_equal(lut2, lut) and np.array_equal(valid2, valid)


def test_grouped_kv_heads_equal_repeated_kv_heads():
    """Mask prediction with fewer K heads than Q heads (an extension over utils.py:388): identical to multi-head
    prediction on K repeated per group, for top-k and CDF selection with per-head hyper-parameters."""
    from oracle import api
    tag, d, n, H, Hkv = R.BF16, 64, 640, 4, 2
    rng = np.random.default_rng(33)
    mk = lambda h, s=1.0: R.round_to(rng.standard_normal((1, h, n, d)) * s, tag)
    q, k, v = mk(H), mk(Hkv) + 0.3, mk(Hkv)
    krep, vrep = np.repeat(k, H // Hkv, axis=1), np.repeat(v, H // Hkv, axis=1)
    for kw in (dict(topk=np.array([0.5, 0.3, 0.7, 0.2], np.float32)),
               dict(topk=None, cdfthreshd=np.array([0.9, 0.5, 0.97, 0.7], np.float32), simthreshd1=0.05, is_causal=True)):
        g = api.spas_sage2_attn_meansim_topk(q, k, v, tag, **kw)
        m = api.spas_sage2_attn_meansim_topk(q, krep, vrep, tag, **kw)
        assert g["k8"].shape[1] == Hkv and g["map"].shape[1] == H
        assert np.array_equal(g["map"], m["map"]) and np.array_equal(g["lut"], m["lut"])
        assert np.array_equal(g["out"], m["out"])
        if kw.get("topk") is not None:
            assert not np.array_equal(g["map"][:, 0], g["map"][:, 1])      # heads of one group still select differently
