"""The HIP path against the committed fixture tests/golden/oracle_regression.json, without running the oracle.

The fixture holds SHA-256 digests of every bit-exact intermediate of three seeded inputs and two moments of the
attention output (written by tests/golden/make_oracle_regression_fixture.py).  The GPU results are brought into the
oracle's array conventions (T-typed values as float32, V8 in natural key order) and hashed the same way.
"""
import importlib.util
import json
import os

import numpy as np
import pytest
import torch

import spargeattn_amd as sa
from spargeattn_amd import _lib, utils
from gpu_common import to_np, v8_natural

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
spec = importlib.util.spec_from_file_location("make_oracle_regression_fixture",
                                              os.path.join(HERE, "golden", "make_oracle_regression_fixture.py"))
gen = importlib.util.module_from_spec(spec)
spec.loader.exec_module(gen)
GOLDEN = json.load(open(os.path.join(HERE, "golden", "oracle_regression.json")))


@pytest.mark.parametrize("case", gen.CASES, ids=[c["name"] for c in gen.CASES])
def test_hip_path_reproduces_the_committed_digests(case):
    want = GOLDEN[case["name"]]
    tdt = torch.bfloat16 if case["dtype"] == "bf16" else torch.float16
    q, k, v = (torch.from_numpy(x).to(tdt).cuda() for x in gen.make_inputs(case))
    kw = dict(case["kw"])
    H, N = q.shape[1], q.shape[2]
    got = {}
    km = _lib.km_mean(k)
    got["km"] = to_np(km[:, :, 0])
    thr = utils.hyperparameter_check(kw.get("simthreshd1", -0.1), H, q.device)
    got["pool_q"], got["sim_q"], got["q8"], got["q_scale"] = _lib.pool_sim_quant(q, None, 128, thr)
    got["pool_k"], got["sim_k"], got["k8"], got["k_scale"] = _lib.pool_sim_quant(k, km, 64, thr)
    sel = dict(is_causal=kw.get("is_causal", False), simthreshd1=kw.get("simthreshd1", -0.1),
               cdfthreshd=kw.get("cdfthreshd"), topk=kw.get("topk"), attention_sink=kw.get("attention_sink", False))
    got["map"] = utils.get_block_map_meansim_fuse_quant(q, k, km, **sel)[0]
    got["lut"], got["valid"] = utils.get_block_map_meansim_fuse_quant(q, k, km, return_lut=True, **sel)[:2]
    if not case.get("sage1"):
        v8, got["v_scale"] = _lib.v_quant_fp8(v)
        nat = v8_natural(v8)                                   # (B,H,ceil64(N),D); the oracle pads to ceil128(N) like fused.cu
        npad = (N + 127) // 128 * 128
        got["v8"] = np.concatenate([nat, np.zeros(nat.shape[:2] + (npad - nat.shape[2], nat.shape[3]), np.uint8)], axis=2)
    for key, val in got.items():
        a = val if isinstance(val, np.ndarray) else (to_np(val) if val.dtype in (torch.float16, torch.bfloat16) else val.cpu().numpy())
        assert gen.digest(a) == want[key], key
    fn = sa.spas_sage_attn_meansim_topk_cuda if case.get("sage1") else sa.spas_sage2_attn_meansim_topk_cuda
    api_kw = {k_: v_ for k_, v_ in kw.items() if v_ is not None}
    if case.get("sage1") or "cdfthreshd" not in api_kw:
        o, sparsity = fn(q, k, v, return_sparsity=True, **api_kw)
    else:
        o, sparsity = sa.spas_sage2_attn_meansim_cuda(q, k, v, return_sparsity=True, **api_kw)
    assert repr(float(sparsity)) == want["sparsity"] or abs(float(sparsity) - float(want["sparsity"])) < 1e-6
    # rows of Q blocks with no selected K block are left unwritten by the kernel and are zero in the oracle
    written = torch.from_numpy(np.repeat(to_np_bool(want, got), 128, axis=2)[:, :, :N]).cuda()
    o = torch.where(written[..., None], o, torch.zeros_like(o)).double()
    moments = [float(o.sum()), float(o.abs().sum())]
    assert moments[1] == pytest.approx(want["out"][1], rel=2e-3)
    assert abs(moments[0] - want["out"][0]) <= 2e-3 * want["out"][1]


def to_np_bool(want, got):
    """valid_block_num > 0 per Q block, the oracle's `written` flag."""
    return (got["valid"].cpu().numpy() > 0)
