"""Tuner module (spas_sage_attn/autotune.py): state-dict format against the tuned-parameter file the reference ships
(tests/golden/cogvideox_tuned_params.json), bisection logic against closed forms with a synthetic kernel (CPU), and an
end-to-end tuning run on the GPU."""
import json
import os

import pytest
import torch
import torch.nn as nn

from spargeattn_amd import autotune as at

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "cogvideox_tuned_params.json")


def _golden_state_dict():
    raw = json.load(open(GOLDEN))
    return {k: torch.tensor(v["values"], dtype=getattr(torch, v["dtype"])) for k, v in raw.items()}


class _Attn(nn.Module):
    def __init__(self):
        super().__init__()
        self.inner_attention = at.SparseAttentionMeansim()
        self.proj = nn.Linear(4, 4)


class _Block(nn.Module):
    def __init__(self):
        super().__init__()
        self.attn1 = _Attn()


class _Model(nn.Module):
    def __init__(self, n):
        super().__init__()
        self.transformer_blocks = nn.ModuleList([_Block() for _ in range(n)])


def test_reference_tuned_file_round_trips():
    sd = _golden_state_dict()
    assert len(sd) == 150 and all(v.shape == (30,) for v in sd.values())
    model = at.load_sparse_attention_state_dict(_Model(30), sd)
    for i, blk in enumerate(model.transformer_blocks):
        m = blk.attn1.inner_attention
        for name in at.PARAM_NAMES:
            got = getattr(m, name)
            want = sd[f"transformer_blocks.{i}.attn1.inner_attention.{name}"]
            assert isinstance(got, nn.Parameter) and not got.requires_grad
            assert got.dtype == torch.float32                      # cast to the model's dtype, bools included
            assert torch.equal(got.data, want.to(torch.float32))
    back = at.extract_sparse_attention_state_dict(model)
    assert sorted(back) == sorted(sd)
    for k in sd:
        assert torch.equal(back[k], sd[k].to(torch.float32))
    # the values the file holds are what the operators accept per head: thresholds in range, tuned PV thresholds small
    pv = torch.stack([v for k, v in sd.items() if k.endswith("pvthreshd")])
    assert 0.0 < float(pv.min()) < 1.0 and float(pv.max()) <= 50.0
    cdf = torch.stack([v for k, v in sd.items() if k.endswith("cdfthreshd")])
    assert 0.0 <= float(cdf.min()) and float(cdf.max()) <= 1.0


def test_substring_matching_does_not_mix_blocks():
    sd = _golden_state_dict()
    model = at.load_sparse_attention_state_dict(_Model(12), {k: v for k, v in sd.items()
                                                              if int(k.split(".")[1]) < 12})
    a = model.transformer_blocks[1].attn1.inner_attention.pvthreshd
    b = model.transformer_blocks[10].attn1.inner_attention.pvthreshd
    assert torch.equal(a.data, sd["transformer_blocks.1.attn1.inner_attention.pvthreshd"])
    assert torch.equal(b.data, sd["transformer_blocks.10.attn1.inner_attention.pvthreshd"])


class _FakeKernel:
    """o = gt * (1 + err): err falls linearly with cdfthreshd and rises as pvthreshd falls; sparsity = 1 - cdfthreshd."""

    def __init__(self, c_star, p_star):
        self.c_star, self.p_star, self.calls = c_star, p_star, []

    def __call__(self, q, k, v, mask=None, is_causal=False, cdfthreshd=None, smooth_k=True, return_sparsity=False,
                 simthreshd1=None, pvthreshd=50, **kw):
        gt = torch.nn.functional.scaled_dot_product_attention(q, k, v, mask, is_causal=is_causal)
        c = float(cdfthreshd)
        err = 0.07 + 0.2 * (self.c_star - c)                     # L1 < 0.07  <=>  c > c_star
        err_pv = 0.08 + 0.001 * (self.p_star - float(pvthreshd))  # L1 < 0.08  <=>  pv > p_star
        e = max(err, 0.0) if pvthreshd == 50 else max(err_pv, 0.0)
        self.calls.append((c, float(pvthreshd)))
        return gt * (1 + e), 1.0 - c


def test_bisections_converge_to_the_acceptance_boundary():
    torch.manual_seed(0)
    q, k, v = (torch.randn(1, 1, 64, 16).abs() + 0.1 for _ in range(3))   # positive outputs: L1 of gt*(1+e) is e
    m = at.SparseAttentionMeansim()
    fake = _FakeKernel(c_star=0.3217, p_star=7.3)
    m.kernel_selection = lambda: fake
    m.init_hyperparams(1, "cpu")
    c, sparsity = m.tune_cdfthreshd(q, k, v, simthreshd1=0.0)
    # precision_metric rounds L1 to 4 digits: the boundary is resolved to that, then to the bisection's delta
    assert abs(c - 0.3217) < 0.001 + 0.0005 / 0.2
    assert 10 <= len(fake.calls) <= 12                             # log2(1 / 0.001) halvings, first probe at 0.1
    assert abs(sparsity - (1 - fake.calls[-1][0])) < 1e-12
    fake.calls.clear()
    p, _ = m.tune_pvthreshd(q, k, v, simthreshd1=0.0, cdfthreshd=0.5)
    assert abs(p - 7.3) < 0.1 + 0.05 / 0.001 * 0.001 + 0.06
    assert 9 <= len(fake.calls) <= 11                              # log2(50 / 0.1) halvings, first probe at 20
    # never reaching the target ends at full attention
    fake2 = _FakeKernel(c_star=2.0, p_star=7.3)
    m.kernel_selection = lambda: fake2
    c2, _ = m.tune_cdfthreshd(q, k, v, simthreshd1=0.0)
    assert c2 == 1


def test_grid_selection_takes_the_sparsest_bin():
    m = at.SparseAttentionMeansim(tune_pv=False)
    m.init_hyperparams(2, "cpu")
    table = {s / 16: (0.9 - 0.05 * abs(s + 4), 0.2 + 0.01 * s) for s in range(-16, 16)}   # sparsity peaks at s = -4

    def fake_tune(qi, ki, vi, mask=None, is_causal=False, smooth_k=True, simthreshd1=None):
        sp, cdf = table[simthreshd1]
        return cdf, sp
    m.tune_cdfthreshd = fake_tune
    x = torch.zeros(1, 1, 8, 4)
    orig = torch.cuda.current_device
    torch.cuda.current_device = lambda: "cpu"
    try:
        res = m.autotune(x, x, x, head_idx=1)
    finally:
        torch.cuda.current_device = orig
    # bins of width 1/8 pair (s = -4, -3): total sparsity .9 + .85 is the largest; the bin's maxima are returned
    assert res["final_simthreshd1"] == -3 / 16 and abs(res["final_cdfthreshd"] - 0.17) < 1e-12
    assert res["final_pvthreshd"] == 20 and abs(res["mean_sparsity"] - 0.875) < 1e-12
    m.fill_results(res)
    assert bool(m.is_sparse[1]) and float(m.pvthreshd[1]) == 20 and abs(float(m.simthreshd1[1]) + 3 / 16) < 1e-7
    m.fill_results({**res, "mean_sparsity": 0.05, "head_idx": 0})
    assert not bool(m.is_sparse[0]) and float(m.cdfthreshd[0]) == 1 and float(m.simthreshd1[0]) == 1


@pytest.mark.gpu
def test_tune_then_infer_on_gpu():
    import spargeattn_amd as sa
    from spargeattn_amd import workloads as W
    q, k, v = W.make_qkv(W.CONFIGS["cfg1"], device="cuda")
    q, k, v = q[:, :1].contiguous(), k[:, :1].contiguous(), v[:, :1].contiguous()
    m = at.SparseAttentionMeansim(l1=0.06, pv_l1=0.07)
    dense = m(q, k, v, tune_mode=True)
    assert torch.allclose(dense, torch.nn.functional.scaled_dot_product_attention(q, k, v))
    assert m.num_data_passed == 1 and m.cdfthreshd.shape == (1,)
    assert 0.0 <= float(m.cdfthreshd[0]) <= 1.0 and 0.0 <= float(m.pvthreshd[0]) <= 50.0
    o, sparsity = m(q, k, v, return_sparsity=True)
    want, s2 = sa.spas_sage2_attn_meansim_cuda(q, k, v, cdfthreshd=m.cdfthreshd, simthreshd1=m.simthreshd1,
                                               pvthreshd=m.pvthreshd.float(), attention_sink=True, return_sparsity=True)
    assert torch.equal(o, want) and sparsity == s2
    met = sa.utils.precision_metric(o, dense, verbose=False)
    assert met["L1"] < 0.07 + 0.02, met                                # tuned against pv_l1 = 0.07, sink only adds blocks
    # tuned parameters survive a state-dict round trip
    holder = nn.Sequential(m)
    sd = at.extract_sparse_attention_state_dict(holder)
    assert sorted(sd) == sorted(f"0.{n}" for n in at.PARAM_NAMES)
