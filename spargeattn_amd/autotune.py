"""Per-head hyper-parameter tuner for the CDF selection mode, same interface as ``spas_sage_attn/autotune.py``.

    SparseAttentionMeansim                     spas_sage_attn/autotune.py:78-362
    extract_sparse_attention_state_dict        spas_sage_attn/autotune.py:28-38
    load_sparse_attention_state_dict           spas_sage_attn/autotune.py:41-58

The module replaces ``F.scaled_dot_product_attention`` inside a model.  In tune mode every head is tuned against
dense attention on the data that passes through (bisection of ``cdfthreshd`` for each ``simthreshd1`` on a grid of
sixteenths, then bisection of ``pvthreshd``); afterwards ``forward`` calls ``spas_sage2_attn_meansim_cuda`` with the
five per-head tensors (``is_sparse, cdfthreshd, simthreshd1, simthreshd2, pvthreshd``), which are ``nn.Parameter``s
so that they travel in the model's state dict under the same keys the reference writes
(``<module path>.<name>``, shape ``(H,)``): files tuned with either implementation load into the other.

Differences: there is one kernel family here (no compute-capability switch, autotune.py:136-144), and heads are
tuned sequentially (the reference's ``PARALLEL_TUNE`` process pool, tools/gpu_process.py, is not rebuilt; the
environment variable is ignored).
"""
import os

import torch
import torch.nn as nn
import torch.nn.functional as F

from .core import spas_sage2_attn_meansim_cuda
from .utils import precision_metric

PARAM_NAMES = ("is_sparse", "cdfthreshd", "simthreshd1", "simthreshd2", "pvthreshd")


def extract_sparse_attention_state_dict(model, verbose=False):
    """Sub-dictionary of ``model.state_dict()`` holding the tuned tensors of every SparseAttentionMeansim."""
    full = model.state_dict()
    out = {}
    for path, module in model.named_modules():
        if not isinstance(module, SparseAttentionMeansim):
            continue
        if verbose:
            print(f"{path}: SparseAttentionMeansim")
        for key, value in full.items():
            if path in key:                      # substring match, as the reference does (autotune.py:34)
                out[key] = value
    return out


def load_sparse_attention_state_dict(model, saved_state_dict, multigpu=False, verbose=False):
    """Attach saved per-head tensors to the (still empty) SparseAttentionMeansim modules of ``model``."""
    device = dtype = None
    if not multigpu:
        first = next(model.parameters())
        device, dtype = first.device, first.dtype
    for path, module in model.named_modules():
        if not isinstance(module, SparseAttentionMeansim):
            continue
        for key, value in saved_state_dict.items():
            if path not in key:
                continue
            name = key.split(path)[1][1:]
            if verbose:
                print(f"{key} -> {path}.{name}")
            if multigpu:
                value = value.to(device=module.device)
            else:
                value = value.to(device=device, dtype=dtype)      # the reference casts every tensor, bools included
            setattr(module, name, nn.Parameter(value, requires_grad=False))
    if not multigpu:
        model = model.to(device)
    return model


def _bins_by_simthreshd1(points, width, lo=-1.0):
    bins = {}
    for pt in points:
        bins.setdefault(int((pt["simthreshd1"] - lo) // width), []).append(pt)
    return bins


class SparseAttentionMeansim(nn.Module):
    GRID = 16                 # simthreshd1 candidates are k/16, k = -16..15 (autotune.py:218-220)

    def __init__(self, sim_rule="l1", l1=0.07, pv_l1=0.08, cos_sim=0.98, rmse=0.07, rearrange_kwargs={}, tune_pv=True):
        super().__init__()
        assert l1 >= 0 and cos_sim <= 1 and rmse >= 0, "l1, cos_sim, rmse should be legal"
        assert pv_l1 > l1, 'pv l1 must greater than l1'
        self.sim_rule, self.l1, self.pv_l1, self.cos_sim, self.rmse = sim_rule, l1, pv_l1, cos_sim, rmse
        self.rearrange_kwargs = rearrange_kwargs
        self.tune_pv = tune_pv
        self.head_num = None
        self.is_sparse = None
        self.cdfthreshd = None
        self.simthreshd1 = None
        self.simthreshd2 = None
        self.pvthreshd = None
        self.tuning_sparsity = None
        self.num_data_passed = 0
        self.hyperparams_cache = {}

    # ---- acceptance rule (autotune.py:100-108) -------------------------------------------------------------
    def is_sim(self, o_gt, o_sparse):
        m = precision_metric(o_sparse, o_gt, verbose=False)
        if self.sim_rule == "cosine":
            return m["Cossim"] > self.cos_sim
        if self.sim_rule == "rmse":
            return m["RMSE"] < self.rmse
        if self.sim_rule == "l1":
            return m["L1"] < self.l1
        raise ValueError("sim_rule should be one of ['cosine', 'rmse', 'l1']")

    def init_hyperparams(self, head_num, device):
        def param(t):
            return nn.Parameter(t, requires_grad=False)
        self.head_num = head_num
        self.is_sparse = param(torch.ones(head_num, dtype=torch.bool, device=device))
        self.cdfthreshd = param(torch.full((head_num,), 0.1, device=device))
        self.simthreshd1 = param(torch.full((head_num,), -1.0, device=device))
        self.simthreshd2 = param(torch.zeros(head_num, device=device))
        self.pvthreshd = param(torch.full((head_num,), 20.0, device=device))
        self.tuning_sparsity = torch.zeros(head_num, device=device)
        self.num_data_passed = 0
        self.hyperparams_cache = {}

    def kernel_selection(self):
        return spas_sage2_attn_meansim_cuda

    # ---- bisections (autotune.py:146-209) ------------------------------------------------------------------
    def _run(self, qi, ki, vi, mask, is_causal, smooth_k, simthreshd1, cdfthreshd, **extra):
        return self.kernel_selection()(
            qi, ki, vi, mask, is_causal=is_causal, cdfthreshd=cdfthreshd, smooth_k=smooth_k, return_sparsity=True,
            simthreshd1=simthreshd1 if simthreshd1 is not None else self.simthreshd1, **extra)

    @torch.no_grad()
    def tune_pvthreshd(self, qi, ki, vi, mask=None, is_causal=False, smooth_k=True, simthreshd1=None, cdfthreshd=None):
        gt = F.scaled_dot_product_attention(qi, ki, vi, mask, is_causal=is_causal)
        lo, hi, cur = 0.0, 50.0, 20.0
        sparsity = None
        while hi - lo > 0.1:
            o, sparsity = self._run(qi, ki, vi, mask, is_causal, smooth_k, simthreshd1, cdfthreshd, pvthreshd=cur)
            if precision_metric(o, gt, verbose=False)["L1"] < self.pv_l1:
                hi, cur = cur, (cur + lo) / 2
            else:
                lo, cur = cur, (cur + hi) / 2
        return cur, sparsity

    @torch.no_grad()
    def tune_cdfthreshd(self, qi, ki, vi, mask=None, is_causal=False, smooth_k=True, simthreshd1=None):
        gt = F.scaled_dot_product_attention(qi, ki, vi, mask, is_causal=is_causal)
        lo, hi, cur = 0.0, 1.0, 0.1
        delta = 0.001
        sparsity = None
        while hi - lo > delta:
            o, sparsity = self._run(qi, ki, vi, mask, is_causal, smooth_k, simthreshd1, cur)
            if self.is_sim(gt, o):
                hi, cur = cur, (cur + lo) / 2
            else:
                lo, cur = cur, (cur + hi) / 2
        if cur > 1 - delta:          # the precision target was never met: fall back to full attention
            cur = 1
        return cur, sparsity

    @torch.no_grad()
    def autotune(self, qi, ki, vi, head_idx, mask=None, is_causal=False, smooth_k=True):
        dev = torch.cuda.current_device()
        qi, ki, vi = qi.to(dev), ki.to(dev), vi.to(dev)
        found = []
        for step in range(-self.GRID, self.GRID):
            s1 = step / self.GRID
            cdf, sparsity = self.tune_cdfthreshd(qi, ki, vi, mask, is_causal=is_causal, smooth_k=smooth_k, simthreshd1=s1)
            pv = 20
            if self.tune_pv:
                pv, _ = self.tune_pvthreshd(qi, ki, vi, mask, is_causal=is_causal, smooth_k=smooth_k, simthreshd1=s1,
                                            cdfthreshd=cdf)
            found.append({"simthreshd1": s1, "cdfthreshd": cdf, "pvthreshd": pv, "sparsity": sparsity,
                          "data_idx": self.num_data_passed})
            if sparsity < 0.1:
                break                # a higher similarity threshold only lowers the sparsity further
        found = found + self.hyperparams_cache.get(head_idx, [])
        self.hyperparams_cache[head_idx] = found

        # bins of width 2/16 in simthreshd1; the bin with the largest total sparsity wins, and inside it the
        # largest (most conservative) value of each parameter is taken (autotune.py:258-265)
        groups = sorted(_bins_by_simthreshd1(found, 2 / self.GRID).values(),
                        key=lambda g: sum(p["sparsity"] for p in g), reverse=True)
        best = groups[0]
        return {"final_simthreshd1": float(max(p["simthreshd1"] for p in best)),
                "final_cdfthreshd": float(max(p["cdfthreshd"] for p in best)),
                "final_pvthreshd": float(max(p["pvthreshd"] for p in best)),
                "mean_sparsity": float(sum(p["sparsity"] for p in best) / len(best)),
                "head_idx": head_idx}

    def fill_results(self, rtdict):
        h = rtdict["head_idx"]
        self.simthreshd1[h] = rtdict["final_simthreshd1"]
        self.cdfthreshd[h] = rtdict["final_cdfthreshd"]
        self.pvthreshd[h] = rtdict["final_pvthreshd"]
        self.is_sparse[h] = rtdict["mean_sparsity"] > 0.1 and self.is_sparse[h]
        self.tuning_sparsity[h] = rtdict["mean_sparsity"]
        if not self.is_sparse[h]:
            self.cdfthreshd[h] = 1
            self.simthreshd1[h] = 1

    @torch.no_grad()
    def forward(self, q, k, v, mask=None, is_causal=False, scale=None, tensor_layout="HND", tune_mode=False,
                smooth_k=True, return_sparsity=False):
        assert len(q.shape) == 4, "q should be 4-d tensor with B, H, L, D"
        if os.environ.get("TUNE_MODE", "") != "" or tune_mode:
            if tensor_layout == "NHD":
                q, k, v = (t.transpose(-2, -3) for t in (q, k, v))
            if self.is_sparse is None:
                self.init_hyperparams(q.shape[1], q.device)
            for h in range(self.head_num):
                if not self.is_sparse[h].item():
                    continue
                res = self.autotune(q[:, h:h + 1], k[:, h:h + 1], v[:, h:h + 1], head_idx=h, mask=mask,
                                    is_causal=is_causal, smooth_k=smooth_k)
                self.fill_results(res)
            self.num_data_passed += 1
            o = F.scaled_dot_product_attention(q, k, v, mask, is_causal=is_causal)   # tuning passes stay dense
            if tensor_layout == "NHD":
                o = o.transpose(-2, -3)
            if return_sparsity:
                # the reference unpacks the dense output as if it were (o, sparsity) here (autotune.py:358-360),
                # which raises ValueError for every batch size but 2
                raise ValueError("return_sparsity is not available in tune mode")
            return o
        assert self.cdfthreshd is not None, "attention hyperparameters should be tuned first"
        return self.kernel_selection()(
            q, k, v, mask, is_causal=is_causal, smooth_k=smooth_k, scale=scale, tensor_layout=tensor_layout,
            cdfthreshd=self.cdfthreshd, simthreshd1=self.simthreshd1, pvthreshd=self.pvthreshd.float(),
            return_sparsity=return_sparsity, attention_sink=True)
