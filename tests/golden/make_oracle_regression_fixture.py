"""Writes tests/golden/oracle_regression.json: digests of what the CPU oracle returns for three small seeded inputs.

    python tests/golden/make_oracle_regression_fixture.py

The oracle (oracle/) is the checker of every GPU parity test.  It is pinned by library routines, closed forms and brute
force (tests/test_oracle_*.py); this fixture adds a tripwire on top of that: an edit that changes what the oracle
returns on these inputs - mask, LUT, INT8/FP8 codes, scales, attention output - fails
tests/test_oracle_regression.py and has to be made on purpose by regenerating the file.  The inputs come from numpy's
PCG64 generator with fixed seeds; nothing of the reference is read or run.
"""
import hashlib
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import api as oapi          # noqa: E402
from oracle import rounding as rnd      # noqa: E402

CASES = [
    dict(name="topk_causal_bf16_d64", seed=101, B=1, H=2, N=448, D=64, dtype="bf16", kw=dict(is_causal=True, topk=0.5)),
    dict(name="cdf_sink_fp16_d128", seed=102, B=1, H=2, N=300, D=128, dtype="fp16",
         kw=dict(is_causal=False, topk=None, cdfthreshd=0.9, simthreshd1=0.3, attention_sink=True, pvthreshd=2.0)),
    dict(name="sage1_topk_fp16_d64", seed=103, B=2, H=1, N=257, D=64, dtype="fp16", sage1=True,
         kw=dict(is_causal=True, topk=0.7)),
]


def make_inputs(case):
    rng = np.random.default_rng(case["seed"])
    shape = (case["B"], case["H"], case["N"], case["D"])
    base = rng.standard_normal((case["B"], case["H"], 1, case["D"]))
    q = rng.standard_normal(shape) + 0.5 * base
    k = 1.5 * rng.standard_normal(shape) + base
    v = 2.0 * rng.standard_normal(shape)
    return tuple(rnd.round_to(x, case["dtype"]) for x in (q, k, v))


def digest(a):
    a = np.ascontiguousarray(a)
    return hashlib.sha256(str(a.dtype).encode() + str(a.shape).encode() + a.tobytes()).hexdigest()[:32]


def run_case(case):
    q, k, v = make_inputs(case)
    fn = oapi.spas_sage_attn_meansim_topk if case.get("sage1") else oapi.spas_sage2_attn_meansim_topk
    res = fn(q, k, v, case["dtype"], **case["kw"])
    out = {}
    for key in sorted(res):
        val = res[key]
        if key == "out":
            # the attention output goes through numpy's exp2, whose last bit may depend on the CPU's vector units:
            # compared by two moments instead of bit for bit
            out[key] = [float(np.asarray(val, np.float64).sum()), float(np.abs(np.asarray(val, np.float64)).sum())]
        elif isinstance(val, np.ndarray):
            out[key] = digest(val)
        elif isinstance(val, (float, int, np.floating, np.integer)):
            out[key] = repr(float(val))
    return out


def main():
    data = {c["name"]: run_case(c) for c in CASES}
    dst = os.path.join(HERE, "oracle_regression.json")
    with open(dst, "w") as f:
        json.dump(data, f, indent=1, sort_keys=True)
    print(dst, {k: len(v) for k, v in data.items()})


if __name__ == "__main__":
    main()
