"""GPU parity (bit-exact) of the mask-prediction / quantisation kernels against the oracle, through the C ABI."""
import numpy as np
import pytest
import torch

from oracle import maskpred as mp
from oracle import vquant as vq
from spargeattn_amd import _lib, utils
from gpu_common import tag_of, to_np, bits_equal_T, v8_natural, rand_T

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,H,N,D", [(1, 2, 1024, 64), (2, 3, 333, 128), (1, 1, 5000, 128)])
def test_km_mean(dtype, B, H, N, D):
    k = rand_T((B, H, N, D), dtype, 1, shift=0.3)
    km = _lib.km_mean(k)
    assert km.shape == (B, H, 1, D) and km.dtype == dtype
    assert bits_equal_T(km[:, :, 0], mp.km_mean(to_np(k), tag_of(dtype)), dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,H,N,D", [(1, 2, 1024, 64), (2, 2, 333, 128), (1, 3, 1100, 128), (1, 2, 200, 64)])
def test_pool_sim_quant(dtype, B, H, N, D):
    tag = tag_of(dtype)
    q = rand_T((B, H, N, D), dtype, 2)
    k = rand_T((B, H, N, D), dtype, 3, shift=0.5)
    # second head: strongly self-similar rows so that both sim outcomes occur with threshold 0.5
    base = rand_T((B, 1, 1, D), dtype, 4)
    k[:, 1:2] = (base.float() * 4 + k[:, 1:2].float() * 0.3).to(dtype)
    q[:, 1:2] = (base.float() * 4 + q[:, 1:2].float() * 0.3).to(dtype)
    thr = torch.tensor([0.5] * H, dtype=torch.float32, device="cuda")
    km = _lib.km_mean(k)
    for x, mean, bs in ((q, None, 128), (k, km, 64)):
        pool, sim, xq, scale = _lib.pool_sim_quant(x, mean, bs, thr)
        ref = mp.pool_sim_quant(to_np(x), None if mean is None else to_np(mean[:, :, 0]), bs, thr.cpu().numpy(), tag)
        assert np.array_equal(xq.cpu().numpy(), ref["q"])
        assert np.array_equal(scale.cpu().numpy().view(np.uint32), ref["scale"].view(np.uint32))
        assert bits_equal_T(pool, ref["pool"], dtype)
        assert np.array_equal(sim.cpu().numpy(), ref["sim"])
        if mean is None:      # (K loses the shared component when km is subtracted)
            assert ref["sim"][:, 1, 0].all() and not ref["sim"][:, 0, 0].any()   # both outcomes are exercised
        if N % bs:
            assert not ref["sim"][:, :, -1].any()                                # partial block is never "similar"
        # quant-only entry (A13) gives the same integers and scales
        _, _, xq2, scale2 = _lib.pool_sim_quant(x, mean, bs, with_pool=False)
        assert torch.equal(xq2, xq) and torch.equal(scale2, scale)


def _pools(B, H, nq, nk, D, dtype, seed):
    pq = rand_T((B, H, nq, D), dtype, seed, scale=1.5)
    pk = rand_T((B, H, nk, D), dtype, seed + 1, scale=1.5)
    g = torch.Generator().manual_seed(seed + 2)
    sq = (torch.rand((B, H, nq), generator=g) > 0.15).cuda()
    sk = (torch.rand((B, H, nk), generator=g) > 0.1).cuda()
    return pq, sq, pk, sk


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("nq,nk,D", [(8, 16, 64), (5, 9, 128), (139, 278, 64), (40, 300, 128), (3, 700, 128),
                                     (5, 1500, 64), (3, 2100, 128),    # 32 columns per lane; the workgroup-level kernel
                                     (2, 4100, 128), (2, 8192, 64)])   # one row per workgroup, the largest LDS footprint
@pytest.mark.parametrize("mode", ["topk", "topk_causal", "cdf", "cdf_causal_sink"])
def test_block_select(dtype, nq, nk, D, mode):
    tag = tag_of(dtype)
    B, H = 1, 3
    pq, sq, pk, sk = _pools(B, H, nq, nk, D, dtype, 10 + nq)
    causal = "causal" in mode and nk == 2 * nq
    sink = "sink" in mode
    topk = cdf = None
    if mode.startswith("topk"):
        topk = torch.tensor([0.5, 0.3, 0.001], dtype=torch.float32, device="cuda")
    else:
        cdf = torch.tensor([0.9, 0.5, 0.999], dtype=torch.float32, device="cuda")
    lut, valid, bmap = _lib.block_select(pq, sq, pk, sk, topk=topk, cdfthreshd=cdf, is_causal=causal,
                                         attention_sink=sink, return_map=True)
    ref_map = mp.block_map(to_np(pq), sq.cpu().numpy(), to_np(pk), sk.cpu().numpy(), tag, is_causal=causal,
                           topk=None if topk is None else topk.cpu().numpy(),
                           cdfthreshd=None if cdf is None else cdf.cpu().numpy(), attention_sink=sink)
    ref_lut, ref_valid = mp.map_to_lut(ref_map)
    got_map = bmap.cpu().numpy()
    assert np.array_equal(got_map, ref_map), f"{(got_map != ref_map).sum()} of {ref_map.size} map entries differ"
    assert np.array_equal(valid.cpu().numpy(), ref_valid)
    assert np.array_equal(lut.cpu().numpy(), ref_lut)


def test_block_select_rejects_bad_arguments():
    pq, sq, pk, sk = _pools(1, 1, 4, 8, 64, torch.float16, 5)
    t = torch.tensor([0.5], device="cuda")
    with pytest.raises(ValueError, match="Only one of cdfthreshd and topk"):
        _lib.block_select(pq, sq, pk, sk, topk=t, cdfthreshd=t)
    with pytest.raises(ValueError, match="Only one of cdfthreshd and topk"):
        _lib.block_select(pq, sq, pk, sk)


@pytest.mark.parametrize("mdtype", [torch.bool, torch.uint8, torch.int32, torch.int64, torch.float16, torch.bfloat16,
                                    torch.float32])
def test_map_to_lut(mdtype):
    g = torch.Generator().manual_seed(7)
    m = torch.rand((2, 3, 11, 301), generator=g) < 0.3
    m[0, 0, 0] = False
    m[0, 0, 1] = True
    mm = m.to(mdtype).cuda()
    if mdtype.is_floating_point:
        mm = mm * -2.5 if mdtype != torch.bool else mm
    lut, valid = _lib.map_to_lut(mm.contiguous())
    ref_lut, ref_valid = mp.map_to_lut(m.numpy())
    assert np.array_equal(lut.cpu().numpy(), ref_lut) and np.array_equal(valid.cpu().numpy(), ref_valid)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,H,N,D", [(1, 2, 1024, 64), (2, 2, 333, 128), (1, 1, 4100, 128)])
def test_v_quant_fp8(dtype, B, H, N, D):
    v = rand_T((B, H, N, D), dtype, 20)
    v[:, :, :, 1] *= 0.01
    v8, v_scale = _lib.v_quant_fp8(v)
    ref_codes, ref_scale = vq.v_quant_fp8(vq.to_fp16(to_np(v)))
    nk = (N + 63) // 64
    assert v8.shape == (B, H, nk, D, 64)
    nat = v8_natural(v8)
    assert np.array_equal(nat[:, :, :N], ref_codes[:, :, :N])
    assert np.all(nat[:, :, N:] == 0)
    assert np.array_equal(v_scale.cpu().numpy().view(np.uint32), ref_scale.view(np.uint32))
    # hardware e4m3 convert agrees with torch's float8_e4m3fn cast on the same products
    v16 = v.to(torch.float16).float()
    recp = torch.from_numpy(np.float32(2.25) / v16.abs().amax(dim=2).cpu().numpy()).cuda()
    lib = (v16 * recp[:, :, None, :]).to(torch.float8_e4m3fn).view(torch.uint8).cpu().numpy()
    assert np.array_equal(nat[:, :, :N], lib)


def test_shared_reciprocal_division_is_ieee():
    """q = a/b through RN(1/b) and one residual correction equals the correctly rounded quotient for every fp16/bf16
    numerator (2^17 patterns) against 2^18 pseudo-random divisors per seed."""
    from spargeattn_amd import _lib
    for seed in (1, 2):
        total, bad = _lib.selftest_division(1 << 18, seed)
        assert total > (1 << 18) * 100000 and bad == 0, (seed, total, bad)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_block_select_score_on_a_rounding_tie(dtype):
    """A pooled score that lies just above a rounding tie of the 16-bit format, by less than binary32 resolves, must be
    rounded from its exact value (up), not through binary32 (which lands on the tie and then rounds to even, down)."""
    tag = tag_of(dtype)
    B, H, nq, nk, D = 1, 1, 4, 8, 64
    half_ulp = 0.25 if dtype == torch.bfloat16 else 2.0 ** -5       # half a unit in the last place at 64
    q1, k1 = (0.5, 0.5) if dtype == torch.bfloat16 else (2.0 ** -3, 2.0 ** -2)
    assert q1 * k1 == half_ulp
    pq = torch.zeros((B, H, nq, D), dtype=dtype, device="cuda")
    pk = torch.zeros((B, H, nk, D), dtype=dtype, device="cuda")
    pq[..., 0], pq[..., 1], pq[..., 2] = 8.0, q1, 2.0 ** -10
    pk[..., 0] = -8.0                                               # every other column: score -64
    pk[0, 0, 2, :3] = torch.tensor([8.0, k1, 0.0], dtype=dtype)           # column 2: 64 + half_ulp exactly (tie -> 64)
    pk[0, 0, 5, :3] = torch.tensor([8.0, k1, 2.0 ** -10], dtype=dtype)    # column 5: 2^-20 above the tie -> next value up
    sq = torch.ones((B, H, nq), dtype=torch.bool, device="cuda")
    sk = torch.ones((B, H, nk), dtype=torch.bool, device="cuda")
    topk = torch.tensor([0.13], dtype=torch.float32, device="cuda")       # int(0.13 * 8) = 1 block per row
    lut, valid, bmap = _lib.block_select(pq, sq, pk, sk, topk=topk, cdfthreshd=None, is_causal=False,
                                         attention_sink=False, return_map=True)
    ref_map = mp.block_map(to_np(pq), sq.cpu().numpy(), to_np(pk), sk.cpu().numpy(), tag, is_causal=False,
                           topk=topk.cpu().numpy(), cdfthreshd=None, attention_sink=False)
    want = np.zeros((B, H, nq, nk), bool)
    want[..., 5] = True                                             # the larger score wins; a tie would go to column 2
    assert np.array_equal(ref_map, want)
    assert np.array_equal(bmap.cpu().numpy().astype(bool), want)
    assert np.array_equal(valid.cpu().numpy(), np.ones((B, H, nq), np.int32))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("thr_value", [-0.1, -1.0, 0.0, 0.3])
def test_similarity_flag_on_degenerate_rows(dtype, thr_value):
    """Negative thresholds are decided without the normalised rows; the flag must still match the oracle on all-zero
    rows, rows whose squares underflow, rows whose squares overflow binary32, infinities and NaNs."""
    B, H, N, D = 1, 2, 128 * 8, 64
    tag = tag_of(dtype)
    x = rand_T((B, H, N, D), dtype, 9)
    big = 3.0e38 if dtype == torch.bfloat16 else 60000.0
    tiny = 1.0e-30 if dtype == torch.bfloat16 else 6.0e-8
    x[0, 0, 128 * 1 + 5] = 0                      # an all-zero row          -> block 1 not similar
    x[0, 0, 128 * 2 + 7] = tiny                   # squares underflow        -> block 2: norm 0 in binary32 (bf16 only)
    x[0, 0, 128 * 3 + 9] = big                    # sum of squares overflows binary32 (bf16): x / inf = 0, still finite
    x[0, 0, 128 * 4 + 11, 3] = float("inf")       # -> not similar
    x[0, 0, 128 * 5 + 13, 60] = float("nan")      # -> not similar
    x[0, 1, 128 * 6 + 1, :32] = 0                 # half a row of zeros is harmless
    thr = torch.tensor([thr_value] * H, dtype=torch.float32, device="cuda")
    for bs in (128, 64):
        pool, sim, xq, scale = _lib.pool_sim_quant(x, None, bs, thr)
        ref = mp.pool_sim_quant(to_np(x), None, bs, thr.cpu().numpy(), tag)
        assert np.array_equal(sim.cpu().numpy(), ref["sim"]), (bs, sim.cpu().numpy(), ref["sim"])
    if thr_value < 0:
        want = np.ones((1, 2, 8), bool)
        want[0, 0, [1, 4, 5]] = False
        if dtype == torch.bfloat16:
            want[0, 0, 2] = False
        assert np.array_equal(ref_sim_128(x, thr, tag), want)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("thr_value", [-0.1, 0.2])
@pytest.mark.parametrize("N", [64 * 7 + 13, 64 * 6 + 5, 64 * 5, 64 * 4 + 64, 50])
@pytest.mark.parametrize("D", [64, 128])
def test_pool_sim_quant_two_blocks_per_workgroup(dtype, thr_value, N, D):
    """A workgroup covers 128 rows, i.e. two 64-row blocks: the second one may be partial, full, or absent, and a
    degenerate row (all zero, infinity) in one block must not change the other block's flag, scale or pooled mean."""
    B, H = 1, 2
    tag = tag_of(dtype)
    k = rand_T((B, H, N, D), dtype, 21, shift=0.25)
    if N > 70:
        k[0, 0, 3] = 0                             # block 0 of head 0: an all-zero row before centring
        k[0, 1, 64 + 2, 5] = float("inf")          # block 1 of head 1
    thr = torch.tensor([thr_value] * H, dtype=torch.float32, device="cuda")
    km = _lib.km_mean(k)
    for mean in (km, None):
        pool, sim, xq, scale = _lib.pool_sim_quant(k, mean, 64, thr)
        ref = mp.pool_sim_quant(to_np(k), None if mean is None else to_np(mean[:, :, 0]), 64, thr.cpu().numpy(), tag)
        assert np.array_equal(sim.cpu().numpy(), ref["sim"]), (sim.cpu().numpy(), ref["sim"])
        finite = np.isfinite(ref["scale"])        # an infinity in a block makes its scale and codes undefined
        assert np.array_equal(scale.cpu().numpy()[finite].view(np.uint32), ref["scale"][finite].view(np.uint32))
        nb = ref["scale"].shape[-1]
        rows_ok = np.repeat(finite, 64, axis=-1)[..., :N]
        assert np.array_equal(xq.cpu().numpy()[rows_ok], ref["q"][rows_ok])
        got_pool, want_pool = to_np(pool), ref["pool"]
        ok = np.isfinite(want_pool)
        assert np.array_equal(got_pool[ok], want_pool[ok])
        assert nb == (N + 63) // 64


def ref_sim_128(x, thr, tag):
    return mp.pool_sim_quant(to_np(x), None, 128, thr.cpu().numpy(), tag)["sim"]


def test_helper_wrappers_of_the_reference_utils():
    """get_quant / get_pool_sim_triton_simmean[_fuse_quant] return what the fused stage returns (utils.py:243-280)."""
    torch.manual_seed(11)
    x = torch.randn((1, 2, 300, 64), device="cuda").to(torch.float16)
    km = _lib.km_mean(x)
    thr = utils.hyperparameter_check(0.2, 2, x.device)
    pool, sim, xq, xs = _lib.pool_sim_quant(x, km, 64, thr)
    got = utils.get_pool_sim_triton_simmean_fuse_quant(x, km, 64, thr)
    assert all(torch.equal(a, b) for a, b in zip(got, (pool, sim, xq, xs)))
    q8, qs = utils.get_quant(x, km, 64)
    assert torch.equal(q8, xq) and torch.equal(qs, xs)
    p2, s2 = utils.get_pool_sim_triton_simmean(x, 128, thr)
    want = _lib.pool_sim_quant(x, None, 128, thr)
    assert torch.equal(p2, want[0]) and torch.equal(s2, want[1])
    with pytest.raises(ValueError):
        utils.get_quant(x, None, 32)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("D", [64, 128])
def test_a_nan_poisons_its_own_element_not_the_scale(dtype, D):
    """The reference's maxima ignore NaN (fmaxf / fminf in csrc/fused/fused.cu:120-123, tl.max = maxnum in
    spas_sage_attn/utils.py:140, 206): one NaN in V or Q leaves the channel / block scale that of the other elements and
    only its own code is affected (FP8 NaN, INT8 0); the block that holds it is never "similar"."""
    tag = tag_of(dtype)
    B, H, N = 1, 2, 700
    v = rand_T((B, H, N, D), dtype, 11)
    q = rand_T((B, H, N, D), dtype, 12)
    v[0, 1, 333, 5] = float("nan")
    q[0, 0, 200, 7] = float("nan")                      # block 1 of head 0 (rows 128..255), 32-row group 6
    v8, vs = _lib.v_quant_fp8(v)
    ref8, refs = vq.v_quant_fp8(vq.to_fp16(to_np(v)))
    assert np.array_equal(vs.cpu().numpy().view(np.uint32), refs.view(np.uint32)) and np.isfinite(refs).all()
    got8 = v8_natural(v8, N)
    nan_at = np.zeros(got8.shape, dtype=bool)
    nan_at[0, 1, 333, 5] = True
    assert np.array_equal(got8[~nan_at], ref8[:, :, :N][~nan_at])
    # the NaN element itself: an e4m3 NaN code (sign bit free: 0x7f or 0xff) on both sides, and nowhere else
    assert (got8[nan_at] & 0x7F) == 0x7F and (ref8[:, :, :N][nan_at] & 0x7F) == 0x7F, (got8[nan_at], ref8[:, :, :N][nan_at])
    assert ((got8[0, 1, :, 5] & 0x7F) == 0x7F).sum() == 1
    thr = torch.full((H,), 0.2, dtype=torch.float32, device="cuda")
    for quant_rows, with_pool in ((128, True), (32, True), (128, False)):
        pool, sim, xq, scale = _lib.pool_sim_quant(q, None, 128, thr, with_pool=with_pool, quant_rows=quant_rows)
        ref = mp.pool_sim_quant(to_np(q), None, 128, thr.cpu().numpy(), tag, with_pool=with_pool, quant_rows=quant_rows)
        assert np.array_equal(xq.cpu().numpy(), ref["q"]) and xq[0, 0, 200, 7] == 0
        assert np.array_equal(scale.cpu().numpy().view(np.uint32), ref["scale"].view(np.uint32))
        assert np.isfinite(ref["scale"]).all()
        if with_pool:
            assert np.array_equal(sim.cpu().numpy(), ref["sim"]) and not ref["sim"][0, 0, 1]
            gp = to_np(pool)
            assert np.array_equal(np.isnan(gp), np.isnan(ref["pool"])) and np.isnan(gp[0, 0, 1, 7])
            ok = ~np.isnan(gp)
            assert np.array_equal(gp[ok], ref["pool"][ok])
    # a negative similarity threshold decides the flag without the normalised rows: the NaN still clears it
    _, sim, _, _ = _lib.pool_sim_quant(q, None, 128, torch.full((H,), -0.1, dtype=torch.float32, device="cuda"))
    assert not bool(sim[0, 0, 1]) and bool(sim[0, 0, 0])
    # K path (mean subtracted): the NaN reaches the column mean of its channel, as in the reference
    km = _lib.km_mean(q)
    _, _, kq, ks = _lib.pool_sim_quant(q, km, 64, thr)
    refk = mp.pool_sim_quant(to_np(q), mp.km_mean(to_np(q), tag), 64, thr.cpu().numpy(), tag)
    assert np.array_equal(kq.cpu().numpy(), refk["q"])
    assert np.array_equal(ks.cpu().numpy().view(np.uint32), refk["scale"].view(np.uint32))
