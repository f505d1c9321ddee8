"""Seeded sweep over small random shapes and options: every stage output of the operator is compared with the oracle
(block map, LUT, INT8 tensors and scales bit-exact; attention output by tolerance)."""
import numpy as np
import pytest
import torch

import spargeattn_amd as sa
from oracle import api as oapi, attention as oat
from spargeattn_amd import _lib, utils
from gpu_common import tag_of, to_np

pytestmark = pytest.mark.gpu


def _cases():
    rng = np.random.default_rng(20240607)
    out = []
    for i in range(40):
        D = int(rng.choice([64, 128]))
        dtype = [torch.float16, torch.bfloat16][int(rng.integers(2))]
        B, H = int(rng.integers(1, 3)), int(rng.integers(1, 4))
        N = int(rng.choice([128, 129, 191, 193, 255, 257, 511, 513, 1023, 1025, int(rng.integers(128, 1300))]))
        causal = bool(rng.integers(2))
        mode = ["topk", "cdf"][int(rng.integers(2))]
        out.append((i, B, H, N, D, dtype, causal, mode, float(rng.uniform(0.2, 0.9)), bool(rng.integers(2)),
                    float(rng.choice([50.0, 3.0, 0.5])), float(rng.choice([-0.1, 0.0, 0.3, 0.8]))))
    return out


@pytest.mark.parametrize("case", _cases(), ids=lambda c: f"{c[0]}-B{c[1]}H{c[2]}N{c[3]}D{c[4]}-{'c' if c[6] else 'n'}-{c[7]}")
def test_random_case(case):
    i, B, H, N, D, dtype, causal, mode, level, sink, pvthr, sim = case
    g = torch.Generator().manual_seed(1000 + i)
    base = torch.randn((B, H, 1, D), generator=g)
    q = (torch.randn((B, H, N, D), generator=g) + 0.5 * base).to(dtype)
    k = (torch.randn((B, H, N, D), generator=g) * 1.5 + base).to(dtype)
    v = (torch.randn((B, H, N, D), generator=g) * 2.0).to(dtype)
    # a smooth stretch so that some blocks are self-similar and the similarity threshold matters
    n0 = N // 3
    q[:, :, :n0] = (q[:, :, :1] + 0.05 * q[:, :, :n0].float()).to(dtype)
    kw = dict(topk=level, cdfthreshd=None) if mode == "topk" else dict(topk=None, cdfthreshd=level)
    res = oapi.spas_sage2_attn_meansim_topk(to_np(q), to_np(k), to_np(v), tag_of(dtype), is_causal=causal,
                                            simthreshd1=sim, pvthreshd=pvthr, attention_sink=sink, **kw)
    qg, kg, vg = q.cuda(), k.cuda(), v.cuda()
    km = _lib.km_mean(kg)
    lut, valid, q8, qs, k8, ks = utils.get_block_map_meansim_fuse_quant(
        qg, kg, km, is_causal=causal, simthreshd1=sim, return_lut=True, attention_sink=sink, **kw)
    assert np.array_equal(lut.cpu().numpy(), res["lut"]) and np.array_equal(valid.cpu().numpy(), res["valid"])
    assert np.array_equal(q8.cpu().numpy(), res["q8"]) and np.array_equal(k8.cpu().numpy(), res["k8"])
    assert np.array_equal(qs.cpu().numpy(), res["q_scale"]) and np.array_equal(ks.cpu().numpy(), res["k_scale"])
    common = dict(is_causal=causal, simthreshd1=sim, pvthreshd=pvthr, attention_sink=sink, return_sparsity=True)
    if i % 3 == 1:      # every third case in the (B,N,H,D) layout, read and written in place by the kernels
        qg, kg, vg = (t.transpose(1, 2).contiguous() for t in (qg, kg, vg))
        common["tensor_layout"] = "NHD"
    if mode == "topk":
        o, sparsity = sa.spas_sage2_attn_meansim_topk_cuda(qg, kg, vg, topk=level, **common)
    else:
        o, sparsity = sa.spas_sage2_attn_meansim_cuda(qg, kg, vg, cdfthreshd=level, **common)
    if i % 3 == 1:
        assert o.is_contiguous()
        o = o.transpose(1, 2)
    assert abs(sparsity - res["sparsity"]) < 1e-6
    met = oat.precision_metric(to_np(o), res["out"])
    assert met["Cossim"] >= 0.999 and met["L1"] <= 1e-2, met


def _cases_wide():
    """Second sweep: fewer K/V heads than query heads, a key/value length of its own, input magnitudes from 0.1 to 200
    both operators (FP8 PV and FP16 PV) and both INT8 granularities of Q."""
    rng = np.random.default_rng(20250913)
    out = []
    for i in range(24):
        D = int(rng.choice([64, 128]))
        dtype = [torch.float16, torch.bfloat16][int(rng.integers(2))]
        B = int(rng.integers(1, 3))
        Hkv = int(rng.integers(1, 3))
        H = Hkv * int(rng.choice([1, 2, 3]))
        Nq = int(rng.choice([128, 200, 257, 640, int(rng.integers(128, 900))]))
        Nk = int(rng.choice([Nq, 64, 130, 333, 1000, int(rng.integers(64, 1100))]))
        mag = float(rng.choice([0.1, 1.0, 10.0, 200.0]))
        out.append((i, B, H, Hkv, Nq, Nk, D, dtype, bool(rng.integers(2)), ["topk", "cdf"][int(rng.integers(2))],
                    float(rng.uniform(0.3, 0.9)), bool(rng.integers(2)), float(rng.choice([50.0, 2.0])), mag,
                    bool(rng.integers(2))))
    return out


@pytest.mark.parametrize("case", _cases_wide(),
                         ids=lambda c: f"{c[0]}-B{c[1]}H{c[2]}/{c[3]}Nq{c[4]}Nk{c[5]}D{c[6]}-x{c[13]:g}-{'s1' if c[14] else 's2'}")
def test_random_case_grouped_heads_and_lengths(case):
    i, B, H, Hkv, Nq, Nk, D, dtype, causal, mode, level, sink, pvthr, mag, sage1 = case
    g = torch.Generator().manual_seed(5000 + i)
    q = (torch.randn((B, H, Nq, D), generator=g) * mag).to(dtype)
    k = ((torch.randn((B, Hkv, Nk, D), generator=g) + 0.4) * mag).to(dtype)
    v = torch.randn((B, Hkv, Nk, D), generator=g).to(dtype)
    kw = dict(topk=level, cdfthreshd=None) if mode == "topk" else dict(topk=None, cdfthreshd=level)
    sim = -0.1 if mode == "topk" else 0.3
    gran = 2 if i % 2 else 1                 # every other case with per-warp INT8 scales of Q
    kw["qk_quant_gran"] = gran
    if sage1:
        res = oapi.spas_sage_attn_meansim_topk(to_np(q), to_np(k), to_np(v), tag_of(dtype), is_causal=causal,
                                               simthreshd1=sim, pvthreshd=pvthr, attention_sink=sink, **kw)
        op = sa.spas_sage_attn_meansim_topk_cuda if mode == "topk" else sa.spas_sage_attn_meansim_cuda
    else:
        res = oapi.spas_sage2_attn_meansim_topk(to_np(q), to_np(k), to_np(v), tag_of(dtype), is_causal=causal,
                                                simthreshd1=sim, pvthreshd=pvthr, attention_sink=sink, **kw)
        op = sa.spas_sage2_attn_meansim_topk_cuda if mode == "topk" else sa.spas_sage2_attn_meansim_cuda
    args = dict(is_causal=causal, simthreshd1=sim, pvthreshd=pvthr, attention_sink=sink, return_sparsity=True,
                qk_quant_gran=gran)
    args["topk" if mode == "topk" else "cdfthreshd"] = level
    qg, kg, vg = q.cuda(), k.cuda(), v.cuda()
    km = _lib.km_mean(kg)
    lut, valid, q8, qs, k8, ks = utils.get_block_map_meansim_fuse_quant(
        qg, kg, km, is_causal=causal, simthreshd1=sim, return_lut=True, attention_sink=sink, **kw)
    assert lut.shape == (B, H, (Nq + 127) // 128, (Nk + 63) // 64)
    assert np.array_equal(lut.cpu().numpy(), res["lut"]) and np.array_equal(valid.cpu().numpy(), res["valid"])
    assert np.array_equal(q8.cpu().numpy(), res["q8"]) and np.array_equal(k8.cpu().numpy(), res["k8"])
    assert np.array_equal(qs.cpu().numpy(), res["q_scale"]) and np.array_equal(ks.cpu().numpy(), res["k_scale"])
    o, sparsity = op(qg, kg, vg, **args)
    assert o.shape == q.shape and abs(sparsity - res["sparsity"]) < 1e-6
    assert torch.isfinite(o.float()).all()
    met = oat.precision_metric(to_np(o), res["out"])
    assert met["Cossim"] >= 0.999 and met["L1"] <= 1e-2, met
