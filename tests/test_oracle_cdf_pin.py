"""Pins oracle.maskpred.num_to_select_cdf against the library routines the reference itself calls for the CDF
selection (spas_sage_attn/utils.py:397-403): torch.sort(descending) -> torch.cumsum -> torch.searchsorted(right=True),
run here on CPU tensors of the input dtype, on random rows, on long flat rows and with thresholds placed exactly on
and just beside cdf values.

torch's CPU cumsum of a bf16 / fp16 tensor accumulates in binary32 and rounds every prefix once to the tensor dtype;
the oracle rounds the exact prefix once.  The two can only differ where binary32 accumulation error moves a prefix
across a rounding boundary of the 16-bit format, which the tests below bound (and find absent on these inputs).
The comparison with the threshold happens in binary32 (the threshold is NOT rounded to the tensor dtype), which the
last test pins separately.
"""
import numpy as np
import pytest
import torch

from oracle import maskpred as mp
from oracle import rounding as R

TORCH_DT = {R.BF16: torch.bfloat16, R.FP16: torch.float16}


def _reference_count(p_T, thr):
    """utils.py:397-403 verbatim in behaviour: p_T (rows, nk) tensor of the input dtype, thr python float or (rows,)."""
    s = torch.sort(p_T, dim=-1, descending=True)
    cdf = torch.cumsum(s.values, dim=-1)
    t = torch.as_tensor(thr, dtype=torch.float32).expand(p_T.shape[0]).reshape(-1, 1).contiguous()
    return torch.searchsorted(cdf, t, right=True).squeeze(-1).numpy(), cdf


def _oracle_count(p_T, thr, tag):
    p = p_T.float().numpy()[None, None]                                # (1,1,rows,nk)
    _, order = mp.stable_desc_rank(p, tag)
    return mp.num_to_select_cdf(p, order, np.array([thr], np.float32), tag)[0, 0]


def _softmax_rows(rng, rows, nk, spread, tag):
    x = rng.standard_normal((rows, nk)) * spread
    p = np.exp(x - x.max(axis=-1, keepdims=True))
    p /= p.sum(axis=-1, keepdims=True)
    return torch.from_numpy(R.round_to(p, tag)).to(TORCH_DT[tag])


@pytest.mark.parametrize("tag", [R.BF16, R.FP16])
@pytest.mark.parametrize("nk", [16, 278, 512, 1857])
@pytest.mark.parametrize("spread", [0.3, 2.0, 6.0])
def test_random_rows_match_torch_sort_cumsum_searchsorted(tag, nk, spread):
    rng = np.random.default_rng(nk * 7 + int(spread * 10))
    p = _softmax_rows(rng, 64, nk, spread, tag)
    for thr in (0.3, 0.5, 0.9, 0.98, 0.999, 1.0):
        want, _ = _reference_count(p, thr)
        got = _oracle_count(p, thr, tag)
        assert np.array_equal(got, want), (thr, np.nonzero(got != want))


@pytest.mark.parametrize("tag", [R.BF16, R.FP16])
@pytest.mark.parametrize("nk", [300, 1857])
def test_long_flat_rows(tag, nk):
    """Every probability equal (the worst case for a scan that rounds at every step: such a scan stalls once the running
    sum's ulp exceeds twice the addend).  torch's CPU scan does not stall and neither does the oracle."""
    val = R.round_to(np.array([1.0 / nk]), tag)[0]
    p = torch.full((3, nk), float(val)).to(TORCH_DT[tag])
    p[1, : nk // 2] *= 2                                              # two plateaus
    p[2, 0] = 0.25                                                    # one heavy block in front
    for thr in (0.1, 0.5, 0.9, 0.98, 1.0):
        want, cdf = _reference_count(p, thr)
        got = _oracle_count(p, thr, tag)
        assert np.array_equal(got, want), thr
    assert float(cdf[0, -1]) > 0.99                                   # the reference's cumulative sum reached ~1: no stall


@pytest.mark.parametrize("tag", [R.BF16, R.FP16])
def test_thresholds_on_and_beside_cdf_values(tag):
    """searchsorted(right=True) counts cdf <= threshold with the threshold kept in binary32: a threshold EQUAL to a cdf
    value includes that element, one binary32 ulp below excludes it, and a threshold that merely ROUNDS to the cdf
    value in the 16-bit format still excludes it."""
    rng = np.random.default_rng(5)
    p = _softmax_rows(rng, 8, 278, 2.0, tag)
    _, cdf = _reference_count(p, 0.5)
    cdf32 = cdf.float().numpy()
    for r in range(p.shape[0]):
        for j in (0, 3, 17, 100):
            c = np.float32(cdf32[r, j])
            for thr in (c, np.nextafter(c, np.float32(0)), np.nextafter(c, np.float32(2))):
                want, _ = _reference_count(p[r:r + 1], float(thr))
                got = _oracle_count(p[r:r + 1], float(thr), tag)
                assert np.array_equal(got, want), (r, j, thr)
    # closed form: p sorted = [.5,.25,.125,.125]; cdf = [.5,.75,.875,1.0]
    p4 = torch.tensor([[0.125, 0.5, 0.25, 0.125]]).to(TORCH_DT[tag])
    for thr, n in ((0.4, 0), (0.5, 1), (0.8, 2), (0.8749, 2), (0.875, 3), (1.0, 4)):
        assert _reference_count(p4, thr)[0][0] == n == _oracle_count(p4, thr, tag)[0]


def test_a_scan_that_rounds_every_step_would_differ():
    """What the pin separates: a cumulative sum carried in bf16 (one rounding per addition) stalls on a long flat row and
    counts MORE blocks for the same threshold than the library routine above and the oracle do."""
    nk = 1857
    val = R.round_to(np.array([1.0 / nk]), R.BF16)[0]
    p = torch.full((1, nk), float(val)).to(torch.bfloat16)
    acc, stepwise = np.float64(0), []
    for _ in range(nk):
        acc = R.round_to(np.array([acc + val]), R.BF16)[0]
        stepwise.append(acc)
    stepwise = np.array(stepwise)
    assert stepwise[-1] < 0.3                                         # stalled far below 1
    naive = int((stepwise <= np.float32(0.5)).sum())
    want, _ = _reference_count(p, 0.5)
    got = _oracle_count(p, 0.5, R.BF16)
    assert got[0] == want[0] < naive == nk
