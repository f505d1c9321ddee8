#!/usr/bin/env python3
"""Headline benchmark: spas_sage2_attn_meansim_topk_cuda on one MI355X.

One step = one call of the operator (K mean, mask prediction + INT8 quantisation, V FP8 quantisation,
block-sparse attention) on the headline configuration cfg4 (B=1, H=32, N=32768, D=128, bf16, causal,
topk=0.5, pvthreshd=50) with synthetic inputs already resident in HBM.

Prints ONE JSON line.  value = dense-equivalent TOPS of the whole step (4*B*H*N^2*D/2 per step time).
Extra keys: the attention kernel alone, the mask-prediction/quantisation stages (us and GB/s), the dense FP16
comparator built in the same library, the MFMA roofline of the attention kernel and a CPU baseline (the numpy
oracle on a bounded sample).
"""
import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_MFMA_8BIT = 5.0e15   # MI355X dense INT8 = FP8 MFMA peak, op/s
PEAK_MFMA_F16 = 2.5e15    # MI355X dense FP16 MFMA peak, flop/s
PEAK_HBM = 8.0e12
# HBM-side bytes per launch of the attention kernel, measured with two rocprofv3 --pmc runs (FETCH_SIZE, WRITE_SIZE,
# each scaled by what the same counter reads for a 1 GiB device copy: x2.0 and x1.0).  Only known for the workload it
# was measured on AND for the kernel source it was measured with: the entry carries the SHA-256 of csrc/attn.hip at
# the time of the measurement, and the bench line reports the figure only while the source still has that digest.
MEASURED_ATTN_TRAFFIC = {
    "cfg4": {"bytes": int((1.894 + 0.250) * 2 ** 30), "attn_hip_sha256": "9d3835bafde519dec8ed5b1f64fe12aa40221642b738c159112c255c267f55b1",
             "profile": "profiles/cfg4_attn_kernel_pmc.md"},
}


def measured_traffic(cfg_name):
    """(bytes or None, note) for the roofline's traffic field."""
    import hashlib
    ent = MEASURED_ATTN_TRAFFIC.get(cfg_name)
    if ent is None:
        return None, "not measured for this workload"
    src = os.path.join(ROOT, "spargeattn_amd", "csrc", "attn.hip")
    digest = hashlib.sha256(open(src, "rb").read()).hexdigest()
    if digest != ent["attn_hip_sha256"]:
        return None, (f"{ent['profile']} was measured with another version of csrc/attn.hip (sha256 "
                      f"{ent['attn_hip_sha256'][:12]}, now {digest[:12]}): re-measure")
    return ent["bytes"], (f"constant: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this kernel on this workload, scaled by a "
                          f"1 GiB copy ({ent['profile']}, csrc/attn.hip sha256 {digest[:12]}); not measured by this run")


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--config", default="cfg4", help="workload (cfg1..cfg5); the headline is cfg4")
    ap.add_argument("--api", default="sage2", choices=["sage2", "sage1"],
                    help="sage2: INT8 QK^T + FP8 PV (headline); sage1: INT8 QK^T + FP16 PV (spas_sage_attn_meansim_topk_cuda)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-dense", action="store_true")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="run only a 1 GiB device-to-device copy (known traffic) - the reference point for scaling the "
                         "FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run")
    ap.add_argument("--attn-only", action="store_true",
                    help="time only the attention kernel launches (for rocprofv3 runs of the dominant kernel)")
    return ap.parse_args()


def cpu_baseline(cfg):
    """numpy oracle on a bounded sample of the headline workload: one of its heads at full sequence length."""
    import numpy as np
    from oracle import api as oapi
    from spargeattn_amd import workloads as W
    n = cfg.N if cfg.N <= 32768 else 32768
    q, k, v = W.make_qkv(cfg, device="cpu", shrink=dict(B=1, H=1, N=n))
    qn, kn, vn = (t.float().numpy() for t in (q, k, v))
    tag = "bf16" if cfg.dtype == torch.bfloat16 else "fp16"
    threads = os.cpu_count() or 1
    t0 = time.perf_counter()
    oapi.spas_sage2_attn_meansim_topk(qn, kn, vn, tag, is_causal=cfg.is_causal, topk=cfg.topk, pvthreshd=cfg.pvthreshd)
    dt = time.perf_counter() - t0
    flop = 4.0 * n * n * cfg.D * (0.5 if cfg.is_causal else 1.0)
    return {"value": flop / dt / 1e12, "unit": "dense-equiv TOPS", "cores": threads, "kind": "port",
            "sample": f"numpy oracle (BLAS threads = host cores), full operator on B=1,H=1,N={n},D={cfg.D} of the "
                      f"{cfg.name} generator, {dt:.1f} s"}


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    import spargeattn_amd as sa
    from spargeattn_amd import core, _lib, workloads as W

    if args.copy_calibration:
        torch.cuda.set_device(0)
        n = 1 << 30
        a = torch.empty(n, dtype=torch.uint8, device="cuda")
        b = torch.zeros(n, dtype=torch.uint8, device="cuda")
        for _ in range(3):
            a.copy_(b)
        torch.cuda.synchronize()
        print(json.dumps({"copy_bytes_read": n, "copy_bytes_written": n}))
        return

    cfg = W.CONFIGS[args.config]
    if cfg.api != "topk":
        print("bench.py times the top-k operator; pick cfg1, cfg3, cfg4 or cfg5", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    _lib.load()
    q, k, v = W.make_qkv(cfg, device=dev)
    B, H, N, D = q.shape
    nq, nk = (N + 127) // 128, (N + 63) // 64
    dense_flop = 4.0 * B * H * N * N * D * (0.5 if cfg.is_causal else 1.0)

    sage1 = args.api == "sage1"
    op = sa.spas_sage_attn_meansim_topk_cuda if sage1 else sa.spas_sage2_attn_meansim_topk_cuda
    # executed ops split evenly between the two products: the blended MFMA peak is the harmonic mean of their peaks
    peak_mfma = 2.0 / (1.0 / PEAK_MFMA_8BIT + 1.0 / PEAK_MFMA_F16) if sage1 else PEAK_MFMA_8BIT

    def step():
        return op(q, k, v, is_causal=cfg.is_causal, topk=cfg.topk, pvthreshd=cfg.pvthreshd)

    # ---- stage events (recorded on the stream the kernels are launched on) -------------------------------
    names = ["km", "maskpred", "vquant", "attn", "end"]      # stage boundaries of a single-stream call
    marks = []

    def hook(name):
        e = torch.cuda.Event(enable_timing=True)
        e.record()
        marks.append((name, e))

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()

    if args.attn_only:
        # the dominant kernel alone, on the tensors the operator would hand it
        km = _lib.km_mean(k)
        from spargeattn_amd import utils
        lut, valid, q8, qs, k8, ks = utils.get_block_map_meansim_fuse_quant(
            q, k, km, is_causal=cfg.is_causal, simthreshd1=-0.1, cdfthreshd=None, topk=cfg.topk, return_lut=True)
        o = torch.empty_like(q)
        pvt = torch.full((H,), float(cfg.pvthreshd), device=dev)
        if sage1:
            vt = _lib.v_tiles_f16_swizzled(v)
            run = lambda: _lib.block_sparse_attn_f16v(q8, k8, vt, o, lut, valid, pvt, qs, ks, 1.0 / D ** 0.5,
                                                      is_causal=cfg.is_causal)
        else:
            v8, vs = _lib.v_quant_fp8(v.to(torch.float16))
            run = lambda: _lib.block_sparse_attn(q8, k8, v8, o, lut, valid, pvt, qs, ks, vs, 1.0 / D ** 0.5)
        for _ in range(args.warmup):
            run()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            run()
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / args.steps
        print(json.dumps({"attn_only_ms": dt * 1e3, "dense_equiv_tops": dense_flop / dt / 1e12}))
        return

    def stats(xs):
        xs = sorted(xs)
        n = len(xs)
        med = xs[n // 2] if n % 2 else 0.5 * (xs[n // 2 - 1] + xs[n // 2])
        return {"median": med, "min": xs[0], "max": xs[-1], "mean": sum(xs) / n}

    # ---- the timed region: exactly `steps` calls of the operator; every call records an event on the stream the
    #      kernels run on at each stage boundary (K mean | pooling, quantisation, selection | V quantisation | attention)
    core._stage_hook = hook
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    step_s = (t1 - t0) / args.steps
    timed_marks = len(marks)
    # stage medians want at least 20 samples: further calls outside the timed region when `steps` is smaller
    for _ in range(max(0, 20 - args.steps)):
        step()
    torch.cuda.synchronize()
    core._stage_hook = None
    per_stage = {n: [] for n in names[:-1]}
    per_step_total = []
    for i in range(0, len(marks), len(names)):
        grp = marks[i:i + len(names)]
        for (n0, e0), (_, e1) in zip(grp[:-1], grp[1:]):
            per_stage[n0].append(e0.elapsed_time(e1))
        per_step_total.append(grp[0][1].elapsed_time(grp[-1][1]))
    n_timed = timed_marks // len(names)
    assert n_timed == args.steps
    step_stats = stats(per_step_total[:n_timed])
    attn_stats = stats(per_stage["attn"][:n_timed])
    attn_s = attn_stats["mean"] * 1e-3          # average launch duration over the timed region (roofline denominator)
    stage_ms = {n0: stats(v)["median"] for n0, v in per_stage.items()}
    mp_serial = stats([a + b for a, b in zip(per_stage["km"], per_stage["maskpred"])])
    serial_runs = len(per_stage["km"])
    marks.clear()

    # ---- executed work of the attention kernel ----------------------------------------------------------------
    from spargeattn_amd import utils
    km = _lib.km_mean(k)
    lut, valid, *_ = utils.get_block_map_meansim_fuse_quant(q, k, km, is_causal=cfg.is_causal, simthreshd1=-0.1,
                                                            cdfthreshd=None, topk=cfg.topk, return_lut=True)
    sel_blocks = int(valid.sum().item())
    executed_ops = sel_blocks * 2.0 * (128 * 64 * D) * 2.0
    del lut, valid, km

    # ---- algorithmic bytes of mask prediction + quantisation (read Q once, K twice, V twice; write Q8,K8,V8) ---
    elt = B * H * N * D
    mp_bytes = 2 * elt * (1 + 2) + 2 * elt + (nq + nk) * B * H * D * 2 + 4 * B * H * nq * nk
    vq_bytes = 2 * elt * 2 + elt
    mp_ms = mp_serial["median"]

    out = {
        "metric": "dense-equiv TOPS + MFMA util % at N=32K,D=128 causal topk=0.5; mask-pred us",
        "value": dense_flop / step_s / 1e12,
        "unit": "dense-equiv TOPS (4*B*H*N^2*D/2 per step time)",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": step_s * 1e3,
        "ms_per_step_events": step_stats,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": ("int8 QK^T + fp16 PV" if sage1 else "int8 QK^T + fp8-e4m3 PV") + " (fp32 softmax/accumulate), bf16 in/out",
        "data": "synthetic (seeded generator, see spargeattn_amd/workloads.py)",
        "config": {"workload": f"{cfg.name}: {op.__name__} B={B} H={H} N={N} D={D} "
                               f"{'causal' if cfg.is_causal else 'non-causal'} topk={cfg.topk} pvthreshd={cfg.pvthreshd}",
                   "selected_blocks": sel_blocks, "block_density": sel_blocks / (B * H * nq * nk)},
        "attn_kernel": {"ms": attn_stats, "dense_equiv_tops": dense_flop / attn_s / 1e12,
                        "executed_tops": executed_ops / attn_s / 1e12,
                        "mfma_util_pct": 100.0 * executed_ops / attn_s / peak_mfma},
        # mask prediction = K mean + pooling/similarity/INT8 of Q and K + block selection (stages A2-A8): median of the
        # HIP-event times of `runs` calls (the timed steps, topped up to 20)
        "mask_pred": {"us": mp_ms * 1e3, "us_min": mp_serial["min"] * 1e3, "us_max": mp_serial["max"] * 1e3,
                      "runs": serial_runs, "km_us": stage_ms["km"] * 1e3,
                      "pool_quant_select_us": stage_ms["maskpred"] * 1e3,
                      "algorithmic_GB": mp_bytes / 1e9, "GBps": mp_bytes / (mp_ms * 1e-3) / 1e9,
                      "hbm_frac": mp_bytes / (mp_ms * 1e-3) / PEAK_HBM},
        "v_quant": {"us": stage_ms["vquant"] * 1e3, "GBps": vq_bytes / (stage_ms["vquant"] * 1e-3) / 1e9},
        "roofline": {"kernel": f"block_sparse_attn_kernel<{D},{'bf16' if q.dtype == torch.bfloat16 else 'fp16'},{'fp16 PV' if sage1 else 'fp8 PV'}>",
                     "bound": "mfma",
                     "achieved": executed_ops / attn_s / 1e12, "peak": peak_mfma / 1e12, "unit": "TFLOP/s",
                     "frac": executed_ops / attn_s / peak_mfma,
                     "traffic": None if sage1 else measured_traffic(cfg.name)[0],
                     "traffic_source": "fp16-PV variant: not measured" if sage1 else measured_traffic(cfg.name)[1],
                     "note": "achieved = executed MFMA ops of both products (selected blocks * 2*128*64*D*2) / mean HIP-event "
                             "time of the kernel over the timed steps; peak = MI355X dense 8-bit MFMA"
                             + (" for QK^T and dense fp16 MFMA for PV, blended" if sage1 else "")},
    }

    # ---- accuracy of the operator output on sampled Q blocks: against dense fp32 attention on the original tensors
    #      (includes the effect of dropping blocks) and against fp32 attention restricted to the selected blocks -------
    o = step()
    o_pw = op(q, k, v, is_causal=cfg.is_causal, topk=cfg.topk, pvthreshd=cfg.pvthreshd, qk_quant_gran=2)
    # per-warp granularity of Q (one INT8 scale per 32 query rows): same kernels, same time - measured here on a few steps
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(max(3, args.steps // 2)):
        op(q, k, v, is_causal=cfg.is_causal, topk=cfg.topk, pvthreshd=cfg.pvthreshd, qk_quant_gran=2)
    torch.cuda.synchronize()
    pw_ms = (time.perf_counter() - t0) / max(3, args.steps // 2) * 1e3
    km = _lib.km_mean(k)
    lut, valid, *_ = utils.get_block_map_meansim_fuse_quant(q, k, km, is_causal=cfg.is_causal, simthreshd1=-0.1,
                                                            cdfthreshd=None, topk=cfg.topk, return_lut=True)
    num = {"dense": [0.0, 0.0, 0.0, 0.0, 0.0], "masked": [0.0, 0.0, 0.0, 0.0, 0.0], "masked_pw": [0.0, 0.0, 0.0, 0.0, 0.0]}
    samples = [(0, nq // 2), (H // 2, nq - 1), (H - 1, nq // 5)]
    for (h, qb) in samples:
        r0, r1 = qb * 128, min(N, qb * 128 + 128)
        sc = (q[0, h, r0:r1].float() @ k[0, h].float().T) * D ** -0.5
        if cfg.is_causal:
            rows = torch.arange(r0, r1, device=dev)[:, None]
            sc = sc.masked_fill(torch.arange(N, device=dev)[None, :] > rows, float("-inf"))
        idx = torch.cumsum(lut[0, h, qb, :int(valid[0, h, qb])].long(), 0)
        bm = torch.zeros(nk, dtype=torch.bool, device=dev)
        bm[idx] = True
        tok = bm.repeat_interleave(64)[:N]
        sc_m = sc.masked_fill(~tok[None, :], float("-inf"))
        for name, scores, got in (("dense", sc, o[0, h, r0:r1].float()), ("masked", sc_m, o[0, h, r0:r1].float()),
                                  ("masked_pw", sc_m, o_pw[0, h, r0:r1].float())):
            ref = torch.softmax(scores, dim=-1) @ v[0, h].float()
            a = num[name]
            a[0] += float((got * ref).sum()); a[1] += float((got * got).sum()); a[2] += float((ref * ref).sum())
            a[3] += float((got - ref).abs().sum()); a[4] += float(ref.abs().sum())
    out["accuracy"] = {
        "note": "parity is judged against the oracle, which quantises identically (tests: cos >= 0.999, rel-L1 <= 1e-2); "
                "the figures here are the METHOD's error on this synthetic workload: INT8/FP8 quantisation on the selected "
                "blocks, and - against dense attention - the mass that top-k 0.5 drops, because the generator's scores are "
                "close to uniform (rank-16 signal plus equal-variance noise), i.e. not sparse",
        "sample": f"Q blocks {samples} (head, block) of batch 0",
        "vs_fp32_attention_on_selected_blocks": {"cos": num["masked"][0] / (num["masked"][1] * num["masked"][2]) ** 0.5,
                                                 "rel_l1": num["masked"][3] / num["masked"][4]},
        "vs_dense_fp32_sdpa": {"cos": num["dense"][0] / (num["dense"][1] * num["dense"][2]) ** 0.5,
                               "rel_l1": num["dense"][3] / num["dense"][4]},
        "per_warp_q_scales": {"note": "qk_quant_gran=2 (opt-in keyword; the default above is the reference's per-block granularity): "
                                      "same block map, Q quantised with one scale per 32 rows",
                              "ms_per_step": pw_ms,
                              "vs_fp32_attention_on_selected_blocks": {
                                  "cos": num["masked_pw"][0] / (num["masked_pw"][1] * num["masked_pw"][2]) ** 0.5,
                                  "rel_l1": num["masked_pw"][3] / num["masked_pw"][4]}}}
    del o, o_pw, lut, valid, km

    if not args.no_dense:
        qh, kh, vh = q.to(torch.float16), k.to(torch.float16), v.to(torch.float16)
        vt = _lib.v_tiles_f16_swizzled(vh)
        oh = torch.empty_like(qh)
        sc = 1.0 / D ** 0.5
        for _ in range(max(1, args.warmup)):
            _lib.dense_attn_f16(qh, kh, vt, sc, is_causal=cfg.is_causal, out=oh)
        torch.cuda.synchronize()
        evs = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps + 1)]
        t0 = time.perf_counter()
        for i in range(args.steps):
            evs[i].record()
            _lib.dense_attn_f16(qh, kh, vt, sc, is_causal=cfg.is_causal, out=oh)
        evs[args.steps].record()
        torch.cuda.synchronize()
        dn = (time.perf_counter() - t0) / args.steps
        dense_stats = stats([evs[i].elapsed_time(evs[i + 1]) for i in range(args.steps)])
        out["dense_fp16"] = {"ms": dn * 1e3, "ms_events": dense_stats, "tops": dense_flop / dn / 1e12,
                             "mfma_frac": dense_flop / dn / PEAK_MFMA_F16,
                             "speedup_step": dn / step_s, "speedup_attn_kernel": dn / attn_s,
                             "speedup_step_median": dense_stats["median"] / step_stats["median"]}
        # an independent dense FP16 kernel for scale: PyTorch's own flash-attention backend on the same tensors (not
        # part of this library; skipped when the backend refuses the shape or is missing)
        try:
            from torch.nn.attention import sdpa_kernel, SDPBackend
            with sdpa_kernel([SDPBackend.FLASH_ATTENTION]):
                sd = lambda: torch.nn.functional.scaled_dot_product_attention(qh, kh, vh, is_causal=cfg.is_causal)
                for _ in range(2):
                    sd()
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for _ in range(max(3, args.steps // 2)):
                    sd()
                torch.cuda.synchronize()
                ts = (time.perf_counter() - t0) / max(3, args.steps // 2)
            out["dense_fp16"]["torch_sdpa_flash"] = {"ms": ts * 1e3, "tops": dense_flop / ts / 1e12,
                                                     "speedup_step": ts / step_s,
                                                     "note": "torch.nn.functional.scaled_dot_product_attention, "
                                                             "FLASH_ATTENTION backend, fp16, same shape"}
        except Exception as e:      # noqa: BLE001 - a missing backend must not break the bench line
            out["dense_fp16"]["torch_sdpa_flash"] = {"ms": None, "note": f"not available: {type(e).__name__}"}
        del qh, kh, vh, vt, oh

    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(cfg)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
