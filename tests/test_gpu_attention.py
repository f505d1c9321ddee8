"""GPU parity of the block-sparse attention kernel and of the operator API against the oracle.

Tolerances (floating point, approximate exp2/rcp on both sides): cosine similarity >= 0.999 and
relative L1 <= 1e-2 against the oracle; the quantised tensors, scales, block maps and LUTs are bit-exact.
"""
import numpy as np
import pytest
import torch

import spargeattn_amd as sa
from oracle import api as oapi, attention as oat, maskpred as mp
from spargeattn_amd import _lib, utils, workloads as W
from gpu_common import tag_of, to_np, bits_equal_T, v8_natural, rand_T

pytestmark = pytest.mark.gpu

COS_MIN, L1_MAX = 0.999, 1e-2


def _check_out(o_gpu, ref_out, written=None):
    got = to_np(o_gpu)
    if written is not None:
        rows = np.repeat(written, 128, axis=2)[:, :, :got.shape[2]]
        got, ref_out = got[rows], ref_out[rows]
    if not np.any(ref_out):                      # degenerate case (everything skipped): exact zeros on both sides
        assert not np.any(got)
        return None
    met = oat.precision_metric(got, ref_out)
    assert met["Cossim"] >= COS_MIN and met["L1"] <= L1_MAX, met
    return met


def _stage_inputs(B, H, N, D, dtype, seed):
    q = rand_T((B, H, N, D), dtype, seed)
    k = rand_T((B, H, N, D), dtype, seed + 1, shift=0.4)
    v = rand_T((B, H, N, D), dtype, seed + 2)
    return q, k, v


def _run_kernel_on_oracle_tensors(res, out_dtype, H, N, D, pvthreshd, is_causal=False):
    """Feeds the ORACLE's quantised tensors to the HIP attention kernel (isolates the kernel)."""
    dev = "cuda"
    q8 = torch.from_numpy(res["q8"]).to(dev)
    k8 = torch.from_numpy(res["k8"]).to(dev)
    B = q8.shape[0]
    nk = (N + 63) // 64
    v8_nat = torch.from_numpy(res["v8"][:, :, :nk * 64]).to(dev)            # (B,H,nk*64,D)
    v8 = _lib.v8_natural_to_tiles(v8_nat)                                   # tile layout
    out = torch.zeros((B, H, N, D), dtype=out_dtype, device=dev)
    pvt = torch.full((H,), float(pvthreshd), dtype=torch.float32, device=dev)
    pvc = _lib.block_sparse_attn(q8, k8, v8, out, torch.from_numpy(res["lut"]).to(dev),
                                 torch.from_numpy(res["valid"]).to(dev), pvt,
                                 torch.from_numpy(res["q_scale"]).to(dev), torch.from_numpy(res["k_scale"]).to(dev),
                                 torch.from_numpy(res["v_scale"]).to(dev), 1.0 / D ** 0.5, is_causal=is_causal,
                                 return_pv_count=True)
    torch.cuda.synchronize()
    per_wave = pvc.view(B, H, -1, 4)                       # one count per 32 query rows, equal inside a Q block
    assert bool((per_wave == per_wave[..., :1]).all())
    return out, per_wave[..., 0]


@pytest.mark.parametrize("dtype,D,N", [(torch.bfloat16, 128, 1024), (torch.float16, 64, 1024),
                                       (torch.bfloat16, 64, 333), (torch.float16, 128, 700)])
@pytest.mark.parametrize("topk", [0.5, 1.0])
def test_attention_kernel_on_oracle_tensors(dtype, D, N, topk):
    B, H = 1, 2
    q, k, v = _stage_inputs(B, H, N, D, dtype, 30)
    res = oapi.spas_sage2_attn_meansim_topk(to_np(q), to_np(k), to_np(v), tag_of(dtype), topk=topk)
    out, pvc = _run_kernel_on_oracle_tensors(res, dtype, H, N, D, 50)
    _check_out(out, res["out"])
    assert np.array_equal(pvc.cpu().numpy(), res["pv_count"])
    assert np.array_equal(res["pv_count"], res["valid"])


@pytest.mark.parametrize("kernel_causal", [False, True])
def test_attention_kernel_causal(kernel_causal):
    dtype, D, N, B, H = torch.bfloat16, 128, 1024, 1, 2
    q, k, v = _stage_inputs(B, H, N, D, dtype, 40)
    res = oapi.spas_sage2_attn_meansim_topk(to_np(q), to_np(k), to_np(v), tag_of(dtype), topk=0.6, is_causal=True,
                                            kernel_causal=kernel_causal)
    out, _ = _run_kernel_on_oracle_tensors(res, dtype, H, N, D, 50, is_causal=kernel_causal)
    _check_out(out, res["out"])


def test_attention_kernel_pv_threshold_and_empty_rows():
    dtype, D, N, B, H = torch.float16, 64, 768, 1, 2
    q = (rand_T((B, H, N, D), dtype, 50).float().abs() + 0.5).to(dtype)
    k = rand_T((B, H, N, D), dtype, 51, scale=0.05)
    k[:, :, :64] += 6.0                                     # block 0 dominates: later blocks fall below the threshold
    v = rand_T((B, H, N, D), dtype, 52)
    mask = np.ones((B, H, 6, 12), np.int32)
    mask[0, 1, 2] = 0                                       # a row block without any K block
    for thr in (1e6, 5.0, -1e6, -1e7):
        res = oapi.block_sparse_sage2_attn(to_np(q), to_np(k), to_np(v), mask, tag_of(dtype), pvthreshd=thr)
        out, pvc = _run_kernel_on_oracle_tensors(res, dtype, H, N, D, thr)
        assert np.array_equal(pvc.cpu().numpy(), res["pv_count"]), thr
        _check_out(out, res["out"], written=res["written"])
        assert torch.all(out[0, 1, 256:384] == 0)           # untouched (buffer was zero-initialised by the test)
    assert res["pv_count"].max() == 2 and res["pv_count"][0, 1, 2] == 0


@pytest.mark.parametrize("name,shrink", [("cfg1", None), ("cfg3", dict(H=2, grid=(4, 12, 15), text_tokens=50)),
                                         ("cfg4", dict(H=2, N=2048)), ("cfg5", dict(H=2, grid=(3, 10, 22)))])
def test_topk_api_end_to_end(name, shrink):
    cfg = W.CONFIGS[name]
    q, k, v = W.make_qkv(cfg, device="cpu", shrink=shrink)
    tag = tag_of(cfg.dtype)
    res = oapi.spas_sage2_attn_meansim_topk(to_np(q), to_np(k), to_np(v), tag, is_causal=cfg.is_causal,
                                            topk=cfg.topk, pvthreshd=cfg.pvthreshd)
    qg, kg, vg = q.cuda(), k.cuda(), v.cuda()
    # stage by stage through the host API (bit-exact)
    km = _lib.km_mean(kg)
    assert bits_equal_T(km[:, :, 0], res["km"], cfg.dtype)
    bmap, q8, qs, k8, ks = utils.get_block_map_meansim_fuse_quant(qg, kg, km, is_causal=cfg.is_causal,
                                                                  simthreshd1=-0.1, cdfthreshd=None, topk=cfg.topk)
    assert np.array_equal(q8.cpu().numpy(), res["q8"]) and np.array_equal(k8.cpu().numpy(), res["k8"])
    assert np.array_equal(qs.cpu().numpy(), res["q_scale"]) and np.array_equal(ks.cpu().numpy(), res["k_scale"])
    assert np.array_equal(bmap.cpu().numpy(), res["map"])
    lut, valid, *_ = utils.get_block_map_meansim_fuse_quant(qg, kg, km, is_causal=cfg.is_causal, simthreshd1=-0.1,
                                                            cdfthreshd=None, topk=cfg.topk, return_lut=True)
    assert np.array_equal(lut.cpu().numpy(), res["lut"]) and np.array_equal(valid.cpu().numpy(), res["valid"])
    v8, vs = _lib.v_quant_fp8(vg.to(torch.float16))
    N = q.shape[2]
    assert np.array_equal(v8_natural(v8, N), res["v8"][:, :, :N]) and np.array_equal(vs.cpu().numpy(), res["v_scale"])
    # the operator itself
    o, sparsity = sa.spas_sage2_attn_meansim_topk_cuda(qg, kg, vg, is_causal=cfg.is_causal, topk=cfg.topk,
                                                       pvthreshd=cfg.pvthreshd, return_sparsity=True)
    assert o.dtype == cfg.dtype and o.shape == q.shape
    assert abs(sparsity - res["sparsity"]) < 1e-6
    _check_out(o, res["out"])
    # NHD layout gives the same numbers
    o2 = sa.spas_sage2_attn_meansim_topk_cuda(qg.transpose(1, 2).contiguous(), kg.transpose(1, 2).contiguous(),
                                              vg.transpose(1, 2).contiguous(), is_causal=cfg.is_causal, topk=cfg.topk,
                                              pvthreshd=cfg.pvthreshd, tensor_layout="NHD")
    assert torch.equal(o2.transpose(1, 2), o)
    assert o2.is_contiguous()                     # written in the caller's layout by the kernel, no copy afterwards


def test_strided_inputs_and_output_are_read_and_written_in_place():
    """NHD tensors, head slices of a wider tensor and a strided output buffer give the bits of the contiguous case."""
    torch.manual_seed(3)
    B, H, N, D = 2, 3, 448, 64
    big = torch.randn((3, B, N, H + 2, D), device="cuda").to(torch.bfloat16)      # q, k, v interleaved with 2 spare heads
    views = [big[i, :, :, 1:1 + H].transpose(1, 2) for i in range(3)]             # (B,H,N,D) views, row stride (H+2)*D
    assert not any(t.is_contiguous() for t in views)
    q, k, v = (t.contiguous() for t in views)
    km = _lib.km_mean(k)
    assert torch.equal(_lib.km_mean(views[1]), km)
    thr = torch.full((H,), 0.3, device="cuda")
    for x, xv, kmean, block in ((q, views[0], None, 128), (k, views[1], km, 64)):
        want = _lib.pool_sim_quant(x, kmean, block, thr)
        got = _lib.pool_sim_quant(xv, kmean, block, thr)
        assert all(torch.equal(a, b) for a, b in zip(want, got))
    assert all(torch.equal(a, b) for a, b in zip(_lib.v_quant_fp8(v), _lib.v_quant_fp8(views[2])))
    assert torch.equal(_lib.v_tiles_f16_swizzled(v), _lib.v_tiles_f16_swizzled(views[2]))
    o = sa.spas_sage2_attn_meansim_topk_cuda(q, k, v, topk=0.6)
    o_nhd = sa.spas_sage2_attn_meansim_topk_cuda(*(big[i, :, :, 1:1 + H] for i in range(3)), topk=0.6, tensor_layout="NHD")
    assert torch.equal(o_nhd.transpose(1, 2), o)
    o1 = sa.spas_sage_attn_meansim_topk_cuda(q, k, v, topk=0.6, is_causal=True)
    o1_nhd = sa.spas_sage_attn_meansim_topk_cuda(*(big[i, :, :, 1:1 + H] for i in range(3)), topk=0.6, is_causal=True,
                                                 tensor_layout="NHD")
    assert torch.equal(o1_nhd.transpose(1, 2), o1)
    # rows that are not 16-byte aligned are refused by the binding and copied by the operator
    odd = torch.randn((B, H, N, D + 4), device="cuda").to(torch.bfloat16)[..., 2:2 + D]
    with pytest.raises(RuntimeError, match="16-byte aligned|contiguous"):
        _lib.km_mean(odd)
    assert torch.equal(sa.spas_sage2_attn_meansim_topk_cuda(odd, odd, odd, topk=0.6),
                       sa.spas_sage2_attn_meansim_topk_cuda(odd.contiguous(), odd.contiguous(), odd.contiguous(), topk=0.6))


def test_mask_api_end_to_end_cfg2_shape():
    cfg = W.CONFIGS["cfg2"]
    B, H, N = 1, 3, 1024
    q, k, v = W.make_qkv(cfg, device="cpu", shrink=dict(B=B, H=H, N=N))
    mask = W.make_mask_id(cfg, B, H, N)
    res = oapi.block_sparse_sage2_attn(to_np(q), to_np(k), to_np(v), mask.numpy(), tag_of(cfg.dtype))
    o, sparsity = sa.block_sparse_sage2_attn_cuda(q.cuda(), k.cuda(), v.cuda(), mask_id=mask.cuda(),
                                                  return_sparsity=True)
    assert abs(sparsity - res["sparsity"]) < 1e-6
    _check_out(o, res["out"])
    # masked fp32 reference (what config 2 is specified against): error of the method, reported
    tm = utils.block_map_to_mask(mask.bool())[:, :, :N, :N].cuda()
    ref = torch.nn.functional.scaled_dot_product_attention(q.cuda().float(), k.cuda().float(), v.cuda().float(),
                                                           attn_mask=tm)
    met = oat.precision_metric(to_np(o), to_np(ref))
    assert met["Cossim"] > 0.995, met


def test_cdf_api_end_to_end():
    dtype, D, N, B, H = torch.bfloat16, 64, 1024, 1, 2
    q, k, v = W.make_qkv(W.CONFIGS["cfg1"], device="cpu")
    q, k, v = q.to(dtype), k.to(dtype), v.to(dtype)
    res = oapi.spas_sage2_attn_meansim_topk(to_np(q), to_np(k), to_np(v), tag_of(dtype), simthreshd1=0.6,
                                            cdfthreshd=0.98, topk=None, attention_sink=True)
    o, sp = sa.spas_sage2_attn_meansim_cuda(q.cuda(), k.cuda(), v.cuda(), attention_sink=True, return_sparsity=True)
    assert abs(sp - res["sparsity"]) < 1e-6
    _check_out(o, res["out"])


def test_fp32_input_and_error_paths():
    q = torch.randn(1, 2, 256, 64, device="cuda")
    o = sa.spas_sage2_attn_meansim_topk_cuda(q, q, q)
    assert o.dtype == torch.float16
    with pytest.raises(NameError):
        sa.spas_sage2_attn_meansim_topk_cuda(q, q, q, smooth_k=False)
    with pytest.raises(AssertionError, match="headdim"):
        q96 = torch.randn(1, 2, 256, 96, device="cuda", dtype=torch.float16)
        sa.spas_sage2_attn_meansim_topk_cuda(q96, q96, q96)
    with pytest.raises(AssertionError, match="Only one of cdfthreshd and topk"):
        sa.spas_sage2_attn_meansim_topk_cuda(q, q, q, cdfthreshd=0.9, topk=0.5)
    with pytest.raises(ValueError):
        sa.spas_sage2_attn_meansim_topk_cuda(q, q, q, topk="half")
    o = sa.spas_sage2_attn_meansim_topk_cuda(q, q, q, topk=torch.tensor([0.5, 0.25], device="cuda"))
    assert torch.isfinite(o.float()).all()


@pytest.mark.parametrize("D,N,causal", [(128, 1024, False), (128, 1024, True), (64, 700, False), (64, 512, True)])
def test_dense_f16_comparator(D, N, causal):
    B, H = 1, 2
    q, k, v = (rand_T((B, H, N, D), torch.float16, 60 + i) for i in range(3))
    o = _lib.dense_attn_f16(q, k, _lib.v_tiles_f16_swizzled(v), 1.0 / D ** 0.5, is_causal=causal)
    ref = torch.nn.functional.scaled_dot_product_attention(q.float(), k.float(), v.float(), is_causal=causal)
    met = oat.precision_metric(to_np(o), to_np(ref))
    assert met["Cossim"] > 0.9999 and met["L1"] < 5e-3, met


def test_operator_under_hip_graph_capture():
    """The C ABI neither allocates nor synchronises, so the operator can be captured; every replay (with eager work
    and synchronisations in between) must reproduce the eager output bit for bit."""
    cfg = W.CONFIGS["cfg1"]
    q, k, v = W.make_qkv(cfg, device="cuda")
    eager = sa.spas_sage2_attn_meansim_topk_cuda(q, k, v, topk=cfg.topk)
    qs, ks, vs = q.clone(), k.clone(), v.clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                       # warm-up on the capture stream
        sa.spas_sage2_attn_meansim_topk_cuda(qs, ks, vs, topk=cfg.topk)
    torch.cuda.current_stream().wait_stream(side)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        out = sa.spas_sage2_attn_meansim_topk_cuda(qs, ks, vs, topk=cfg.topk)
    for rep in range(3):
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), rep
        other = sa.spas_sage2_attn_meansim_topk_cuda(q.flip(2).contiguous(), k, v, topk=cfg.topk)   # eager work between replays
        torch.cuda.synchronize()
        assert other.shape == eager.shape
    # new inputs through the static buffers
    qs.copy_(q.flip(2))
    g.replay()
    torch.cuda.synchronize()
    assert torch.equal(out, sa.spas_sage2_attn_meansim_topk_cuda(q.flip(2).contiguous(), k, v, topk=cfg.topk))


@pytest.mark.parametrize("H,Hkv,D,dtype", [(4, 2, 64, torch.float16), (6, 1, 128, torch.bfloat16)])
def test_custom_mask_operator_with_grouped_kv_heads(H, Hkv, D, dtype):
    B, N = 2, 640
    q = rand_T((B, H, N, D), dtype, 70)
    k = rand_T((B, Hkv, N, D), dtype, 71, shift=0.3)
    v = rand_T((B, Hkv, N, D), dtype, 72)
    g = torch.Generator().manual_seed(5)
    mask = (torch.rand((B, H, 5, 10), generator=g) < 0.5).to(torch.int32)
    mask[:, :, torch.arange(5), 2 * torch.arange(5)] = 1
    res = oapi.block_sparse_sage2_attn(to_np(q), to_np(k), to_np(v), mask.numpy(), tag_of(dtype), pvthreshd=3.0)
    o, sparsity = sa.block_sparse_sage2_attn_cuda(q, k, v, mask_id=mask.cuda(), pvthreshd=3.0, return_sparsity=True)
    assert o.shape == q.shape and abs(sparsity - res["sparsity"]) < 1e-6
    _check_out(o, res["out"])
    with pytest.raises(ValueError, match="must be divisible by num_kv_heads"):
        bad = 4 if H == 6 else 3                        # a K/V head count that does not divide H
        sa.spas_sage2_attn_meansim_topk_cuda(q, k[:, :1].expand(B, bad, N, D), v[:, :1].expand(B, bad, N, D))


@pytest.mark.parametrize("H,Hkv,D,dtype,causal", [(4, 2, 64, torch.float16, False), (6, 1, 128, torch.bfloat16, True),
                                                   (8, 4, 128, torch.bfloat16, False)])
def test_mask_prediction_with_grouped_kv_heads(H, Hkv, D, dtype, causal):
    """Fewer K/V heads than query heads through the WHOLE operator (the reference's mask prediction needs equal head
    counts, utils.py:388): K is pooled and quantised per K head, every query head of a group is scored against it with
    its own top-k.  Block map, LUT and quantised tensors bit for bit against the oracle, output at tolerance."""
    B, N = 1, 768
    q = rand_T((B, H, N, D), dtype, 170)
    k = rand_T((B, Hkv, N, D), dtype, 171, shift=0.3)
    v = rand_T((B, Hkv, N, D), dtype, 172)
    topk = torch.linspace(0.3, 0.8, H)
    res = oapi.spas_sage2_attn_meansim_topk(to_np(q), to_np(k), to_np(v), tag_of(dtype), is_causal=causal, topk=topk.numpy())
    km = _lib.km_mean(k)
    bmap, q8, qs, k8, ks = utils.get_block_map_meansim_fuse_quant(q, k, km, is_causal=causal, simthreshd1=-0.1,
                                                                  cdfthreshd=None, topk=topk.cuda())
    assert k8.shape[1] == Hkv and np.array_equal(k8.cpu().numpy(), res["k8"]) and np.array_equal(q8.cpu().numpy(), res["q8"])
    assert np.array_equal(bmap.cpu().numpy(), res["map"])
    o, sp = sa.spas_sage2_attn_meansim_topk_cuda(q, k, v, is_causal=causal, topk=topk.cuda(), return_sparsity=True)
    assert abs(sp - res["sparsity"]) < 1e-6
    _check_out(o, res["out"])
    # CDF selection and the INT8-QK / FP16-PV operator on the same shapes
    res = oapi.spas_sage2_attn_meansim_topk(to_np(q), to_np(k), to_np(v), tag_of(dtype), simthreshd1=0.3, cdfthreshd=0.9,
                                            topk=None)
    o = sa.spas_sage2_attn_meansim_cuda(q, k, v, simthreshd1=0.3, cdfthreshd=0.9)
    _check_out(o, res["out"])
    res = oapi.spas_sage_attn_meansim_topk(to_np(q), to_np(k), to_np(v), tag_of(dtype), topk=0.5, is_causal=causal)
    o = sa.spas_sage_attn_meansim_topk_cuda(q, k, v, topk=0.5, is_causal=causal)
    _check_out(o, res["out"])


@pytest.mark.parametrize("fp16v", [False, True])
def test_pv_threshold_modes_match_the_oracle(fp16v):
    """Per-block (the API's), per-32-rows and no PV threshold: outputs and the per-wavefront PV counts."""
    d, nblk = 64, 6
    n = 64 * nblk
    rng = np.random.default_rng(5)
    nqb = n // 128                                           # queries and keys share one sequence length at this boundary
    q8 = rng.integers(-20, 21, size=(1, 1, n, d)).astype(np.int8)
    k8 = rng.integers(-20, 21, size=(1, 1, n, d)).astype(np.int8)
    q8[0, 0, 32:64, 0] = 120
    k8[0, 0, :64, 0] = 120                                   # block 0 dominates for rows 32..63 only
    lut = np.ones((1, 1, nqb, nblk), np.int32); lut[..., 0] = 0
    valid = np.full((1, 1, nqb), nblk, np.int32)
    # scales small enough that no row is dominated by a few keys (the e4m3 rounding of P then averages out), while block 0
    # still beats every other block by about one unit of log2 for rows 32..63
    qs = np.full((1, 1, nqb), 0.02, np.float32); ks = np.full((1, 1, nblk), 0.02, np.float32)
    thr = np.array([0.25], np.float32)
    if fp16v:
        v = rng.standard_normal((1, 1, n, d)).astype(np.float16)
        vdev = _lib.v_tiles_f16_swizzled(torch.from_numpy(v).cuda())
        vor, vs = v.astype(np.float32), None
    else:
        vor = rng.integers(0, 120, size=(1, 1, n, d)).astype(np.uint8)
        vs = np.ones((1, 1, d), np.float32)
        vdev = _lib.v8_natural_to_tiles(torch.from_numpy(vor).cuda())
    dev = lambda a: torch.from_numpy(a).cuda()
    counts = {}
    for mode in (_lib.PV_PER_BLOCK, _lib.PV_PER_WARP, _lib.PV_NONE):
        ref, _, refc = oat.block_sparse_attention(q8, k8, vor, lut, valid, thr, qs, ks, vs, d ** -0.5, "fp16",
                                                  return_pv_count=True, pv="f16" if fp16v else "fp8", pv_mode=mode)
        out = torch.zeros((1, 1, n, d), dtype=torch.float16, device="cuda")
        if fp16v:
            pvc = _lib.block_sparse_attn_f16v(dev(q8), dev(k8), vdev, out, dev(lut), dev(valid), dev(thr), dev(qs), dev(ks),
                                              d ** -0.5, return_pv_count=True, pv_mode=mode)
        else:
            pvc = _lib.block_sparse_attn(dev(q8), dev(k8), vdev, out, dev(lut), dev(valid), dev(thr), dev(qs), dev(ks), dev(vs),
                                         d ** -0.5, return_pv_count=True, pv_mode=mode)
        _check_out(out, ref)
        want = (refc if mode == _lib.PV_PER_WARP else np.repeat(refc[..., None], 4, axis=-1)).reshape(1, 1, 4 * nqb)
        assert np.array_equal(pvc.cpu().numpy(), want), (mode, pvc, want)
        counts[mode] = pvc.cpu().numpy().ravel().tolist()
    assert counts[_lib.PV_PER_BLOCK] == [nblk] * 4 * nqb == counts[_lib.PV_NONE]
    assert counts[_lib.PV_PER_WARP][1] < nblk and counts[_lib.PV_PER_WARP][:1] + counts[_lib.PV_PER_WARP][2:] == [nblk] * (4 * nqb - 1)


def _int_case(n, nk_blocks, d, rng, r, a_blocks, hq=1):
    """Hand-built quantised operands: small integer codes (diffuse rows) with per-block scales that put the exponent
    multiplier a = sm_scale*log2(e)*q_scale*k_scale of each K block where the test wants it."""
    nqb = (n + 127) // 128
    q8 = rng.integers(-r, r + 1, size=(1, hq, n, d)).astype(np.int8)
    k8 = rng.integers(-r, r + 1, size=(1, 1, n, d)).astype(np.int8)
    lut = np.ones((1, hq, nqb, nk_blocks), np.int32); lut[..., 0] = 0
    valid = np.full((1, hq, nqb), nk_blocks, np.int32)
    c = np.float32(d ** -0.5) * np.float32(1.44269504)
    qs = np.full((1, hq, nqb), 0.5, np.float32)
    ks = (np.asarray(a_blocks, np.float32) / (c * np.float32(0.5))).reshape(1, 1, nk_blocks).astype(np.float32)
    return q8, k8, lut, valid, qs, ks


@pytest.mark.parametrize("fp16v", [False, True])
@pytest.mark.parametrize("d,a_max", [(64, 2e-3), (128, 2e-2), (64, 0.1), (128, 0.5), (64, 2.25), (128, 9.0)])
def test_large_exponent_multiplier_blocks(d, a_max, fp16v):
    """Scores whose exponent multiplier a is far above what N(0,1) inputs give (large |q||k| or a large softmax scale):
    the bias of the integer accumulators must leave the exponent without a rounding error that grows with a, and the
    row maximum's probability must stay inside e4m3.  Blocks with small and large a alternate inside every row."""
    nblk = 8
    n = 64 * nblk
    rng = np.random.default_rng(int(a_max * 1000) + d)
    # codes in [-r, r]: std of a score ~ r^2/1.5 * sqrt(d); keep a*std around 2 so that rows stay diffuse
    r = max(1, int(round((3.0 / (a_max * d ** 0.5)) ** 0.5)))
    a_blocks = a_max * np.array([1.0, 1e-3, 0.5, 0.03, 1.0, 0.25, 1e-4, 0.7])
    q8, k8, lut, valid, qs, ks = _int_case(n, nblk, d, rng, r, a_blocks)
    thr = np.array([50.0], np.float32)
    dev = lambda a: torch.from_numpy(a).cuda()
    out = torch.zeros((1, 1, n, d), dtype=torch.float16, device="cuda")
    if fp16v:
        v = rng.standard_normal((1, 1, n, d)).astype(np.float16)
        ref, _ = oat.block_sparse_attention(q8, k8, v.astype(np.float32), lut, valid, thr, qs, ks, None, d ** -0.5, "fp16", pv="f16")
        _lib.block_sparse_attn_f16v(dev(q8), dev(k8), _lib.v_tiles_f16_swizzled(dev(v)), out, dev(lut), dev(valid), dev(thr),
                                    dev(qs), dev(ks), d ** -0.5)
    else:
        vor = rng.integers(0, 120, size=(1, 1, n, d)).astype(np.uint8)
        vs = np.ones((1, 1, d), np.float32)
        ref, _ = oat.block_sparse_attention(q8, k8, vor, lut, valid, thr, qs, ks, vs, d ** -0.5, "fp16")
        _lib.block_sparse_attn(dev(q8), dev(k8), _lib.v8_natural_to_tiles(dev(vor)), out, dev(lut), dev(valid), dev(thr),
                               dev(qs), dev(ks), dev(vs), d ** -0.5)
    assert torch.isfinite(out.float()).all()
    met = _check_out(out, ref)
    # the kernel follows the oracle far more closely than the operator tolerance: an exponent error of 0.75 a (what one
    # rounding of the bias term costs at large a) would show here
    assert met["L1"] <= 2e-3, met


@pytest.mark.parametrize("mag,scale", [(30.0, None), (100.0, None), (300.0, None), (1.0, 8.0)])
@pytest.mark.parametrize("D,dtype", [(64, torch.float16), (128, torch.bfloat16)])
@pytest.mark.parametrize("sage1", [False, True])
def test_operator_with_large_magnitude_inputs(mag, scale, D, dtype, sage1):
    """Q and K scaled far beyond N(0,1), or a large explicit softmax scale: finite output within tolerance of the oracle."""
    B, H, N = 1, 2, 512
    q = rand_T((B, H, N, D), dtype, 80, scale=mag)
    k = rand_T((B, H, N, D), dtype, 81, scale=mag, shift=0.4 * mag)
    v = rand_T((B, H, N, D), dtype, 82)
    if sage1:
        res = oapi.spas_sage_attn_meansim_topk(to_np(q), to_np(k), to_np(v), tag_of(dtype), topk=0.75, scale=scale)
        o = sa.spas_sage_attn_meansim_topk_cuda(q, k, v, topk=0.75, scale=scale)
    else:
        res = oapi.spas_sage2_attn_meansim_topk(to_np(q), to_np(k), to_np(v), tag_of(dtype), topk=0.75, scale=scale)
        o = sa.spas_sage2_attn_meansim_topk_cuda(q, k, v, topk=0.75, scale=scale)
    assert torch.isfinite(o.float()).all()
    _check_out(o, res["out"])


def test_fp8_pack_saturates_like_the_reference():
    """The e4m3 pack of the attention kernel: round to nearest even below 448, +-448 beyond (cvt.rn.satfinite,
    csrc/numeric_conversion.cuh:48-63), NaN stays NaN."""
    from oracle import rounding as R
    g = torch.Generator().manual_seed(9)
    x = torch.cat([torch.tensor([0.0, 448.0, 449.0, 455.9, 463.9, 464.0, 464.1, 480.0, 1e3, 1e6, 3e38, -3e38,
                                 -449.0, -1e6, -464.1, 2.0 ** -9, 2.0 ** -10, 3 * 2.0 ** -11]),
                   torch.rand(4096, generator=g) * 1000.0, torch.exp2(torch.rand(4096, generator=g) * 30 - 12),
                   -torch.exp2(torch.rand(1022, generator=g) * 30 - 12)]).float()
    assert x.numel() % 4 == 0
    got = _lib.selftest_fp8_pack(x.cuda()).cpu().numpy()
    want = R.f32_to_e4m3fn(x.numpy())
    assert np.array_equal(got, want), [(float(a), hex(b), hex(c)) for a, b, c in zip(x, got, want) if b != c][:10]
    # NaN stays NaN; so does an infinite input (the reference's satfinite maps +-inf to +-448), which the kernel cannot
    # produce: P = 2^x with x <= 8.807 + rounding
    nan = _lib.selftest_fp8_pack(torch.tensor([float("nan"), float("inf"), -float("inf"), 1.0], device="cuda")).cpu().numpy()
    assert np.all((nan[:3] & 0x7f) == 0x7f) and nan[3] == 0x38
    # without the mode bit the bare instruction returns NaN above 464 (what the kernel must never rely on)
    bare = _lib.selftest_fp8_pack(torch.tensor([448.0, 464.0, 464.1, 1e6], device="cuda"), saturate=False).cpu().numpy()
    assert list(bare) == [0x7e, 0x7e, 0x7f, 0x7f]


def test_query_and_key_lengths_differ():
    """qo_len != kv_len (csrc/qattn/qk_int_sv_f8_cuda_sm89.cu:256-300): a LUT of ceil(Nq/128) x ceil(Nk/64) blocks,
    the last K block partial."""
    B, H, D, dtype = 1, 2, 64, torch.float16
    for Nq, Nk in ((384, 1000), (640, 200)):
        q = rand_T((B, H, Nq, D), dtype, 90)
        k = rand_T((B, H, Nk, D), dtype, 91, shift=0.3)
        v = rand_T((B, H, Nk, D), dtype, 92)
        res = oapi.spas_sage2_attn_meansim_topk(to_np(q), to_np(k), to_np(v), tag_of(dtype), topk=0.6)
        o, sp = sa.spas_sage2_attn_meansim_topk_cuda(q, k, v, topk=0.6, return_sparsity=True)
        assert o.shape == q.shape and abs(sp - res["sparsity"]) < 1e-6
        _check_out(o, res["out"])
        nq, nk = (Nq + 127) // 128, (Nk + 63) // 64
        g = torch.Generator().manual_seed(6)
        mask = (torch.rand((B, H, nq, nk), generator=g) < 0.6).to(torch.int32)
        mask[..., nk - 1] = 1
        res = oapi.block_sparse_sage2_attn(to_np(q), to_np(k), to_np(v), mask.numpy(), tag_of(dtype))
        o = sa.block_sparse_sage2_attn_cuda(q, k, v, mask_id=mask.cuda())
        _check_out(o, res["out"])
    with pytest.raises(RuntimeError, match="inconsistent shapes"):
        sa.spas_sage2_attn_meansim_topk_cuda(q, k, v[:, :, :128])


def test_fp8_denominator_and_offset_construction():
    """The kernel on the closed-form construction that separates "fp32 P in the denominator, e4m3(P) in the numerator,
    offset 8.807" from "rounded P in the denominator" and from "no offset" (see tests/gpu_common.py)."""
    from gpu_common import fp8_denominator_case
    (q8, k8, v8, lut, valid, thr, qs, ks, vs, sm_scale), forms = fp8_denominator_case()
    dev = lambda a: torch.from_numpy(a).cuda()
    out = torch.zeros((1, 1, 128, 64), dtype=torch.float16, device="cuda")
    _lib.block_sparse_attn(dev(q8), dev(k8), _lib.v8_natural_to_tiles(dev(v8)), out, dev(lut), dev(valid), dev(thr),
                           dev(qs), dev(ks), dev(vs), sm_scale)
    got = out.float().cpu().numpy()[0, 0]
    assert np.all(np.abs(got - forms["reference"]) < 1.5e-3), (got[0, :4], forms)
