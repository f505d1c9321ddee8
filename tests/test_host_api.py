"""Host logic that needs no GPU: hyper-parameter handling, error behaviour, workload generators."""
import pytest
import torch

from spargeattn_amd import utils, workloads as W
import spargeattn_amd as sa


def test_hyperparameter_check():
    t = utils.hyperparameter_check(0.5, 4, "cpu")
    assert t.shape == (4,) and t.dtype == torch.float32 and torch.all(t == 0.5)
    assert torch.all(utils.hyperparameter_check(3, 2, "cpu") == 3.0)
    assert torch.all(utils.hyperparameter_check(torch.tensor(0.25), 3, "cpu") == 0.25)
    v = torch.tensor([0.1, 0.2, 0.3])
    assert torch.equal(utils.hyperparameter_check(v, 3, "cpu"), v)
    with pytest.raises(AssertionError):
        utils.hyperparameter_check(v, 4, "cpu")
    with pytest.raises(AssertionError):
        utils.hyperparameter_check(torch.zeros(2, 2), 4, "cpu")
    with pytest.raises(ValueError):
        utils.hyperparameter_check("0.5", 4, "cpu")


def test_api_preconditions_raise_like_the_reference():
    q = torch.zeros(1, 2, 64, 64, dtype=torch.float16)
    with pytest.raises(AssertionError, match="seq_len"):
        sa.spas_sage2_attn_meansim_topk_cuda(q, q, q)
    with pytest.raises(AssertionError):
        sa.spas_sage2_attn_meansim_topk_cuda(q, q, q, tensor_layout="BHND")
    q = torch.zeros(1, 2, 128, 64, dtype=torch.float16)
    with pytest.raises(RuntimeError, match="GPU"):          # no silent CPU fallback
        sa.spas_sage2_attn_meansim_topk_cuda(q, q, q)
    with pytest.raises(RuntimeError, match="GPU"):
        sa.block_sparse_sage2_attn_cuda(q, q, q, mask_id=torch.ones(1, 2, 1, 2))


def test_block_map_to_mask():
    m = torch.tensor([[[[1, 0], [0, 1]]]])
    t = utils.block_map_to_mask(m)
    assert t.shape == (1, 1, 256, 128)
    assert t[0, 0, :128, :64].all() and not t[0, 0, :128, 64:].any() and t[0, 0, 128:, 64:].all()


def test_workload_generators_shapes_and_determinism():
    for name, shrink in (("cfg1", None), ("cfg2", dict(B=1, H=2, N=512)), ("cfg3", dict(H=2, grid=(3, 6, 9), text_tokens=30)),
                         ("cfg4", dict(H=2, N=1024)), ("cfg5", dict(H=1, grid=(2, 8, 11)))):
        cfg = W.CONFIGS[name]
        q, k, v = W.make_qkv(cfg, shrink=shrink)
        q2, _, _ = W.make_qkv(cfg, shrink=shrink)
        assert torch.equal(q, q2) and q.dtype == cfg.dtype and q.shape == k.shape == v.shape
        assert q.shape[-1] == cfg.D and torch.isfinite(q.float()).all()
        assert 0.3 < q.float().std() < 3.0
    m = W.make_mask_id(W.CONFIGS["cfg2"], 1, 2, 1024)
    assert m.shape == (1, 2, 8, 16)
    i = torch.arange(8)
    assert m[:, :, i, 2 * i].all() and m[:, :, i, 2 * i + 1].all()
    assert 0.25 < m.float().mean() < 0.5


def test_attention_wrapper_rejects_inconsistent_shapes_before_any_launch():
    """The kernels index K, V, the LUT and the scales with ceil(kv_len/64): shapes that disagree must raise on the host."""
    from spargeattn_amd import _lib
    B, H, N, Nk, D = 1, 2, 256, 320, 64
    nq, nk = 2, 5
    q8 = torch.zeros((B, H, N, D), dtype=torch.int8)
    k8 = torch.zeros((B, H, Nk, D), dtype=torch.int8)
    v8 = torch.zeros((B, H, nk, D, 64), dtype=torch.uint8)
    lut = torch.zeros((B, H, nq, nk), dtype=torch.int32)
    valid = torch.zeros((B, H, nq), dtype=torch.int32)
    qs, ks, vs = torch.ones((B, H, nq)), torch.ones((B, H, nk)), torch.ones((B, H, D))
    assert _lib._check_attn_shapes(q8, k8, v8, lut, valid, qs, ks, vs) == (B, H, H, N, Nk, D)
    with pytest.raises(RuntimeError, match="V tiles"):         # V quantised from a tensor as long as q, not as k
        _lib._check_attn_shapes(q8, k8, torch.zeros((B, H, 4, D, 64), dtype=torch.uint8), lut, valid, qs, ks, vs)
    with pytest.raises(RuntimeError, match="lut"):
        _lib._check_attn_shapes(q8, k8, v8, torch.zeros((B, H, nq, 4), dtype=torch.int32), valid, qs, ks, vs)
    with pytest.raises(RuntimeError, match="k_scale"):
        _lib._check_attn_shapes(q8, k8, v8, lut, valid, qs, torch.ones((B, H, 4)), vs)
    with pytest.raises(RuntimeError, match="does not match"):
        _lib._check_attn_shapes(q8, torch.zeros((B, H, Nk, 128), dtype=torch.int8), v8, lut, valid, qs, ks, vs)
    # the operator: k and v of different lengths
    q = torch.zeros(1, 2, 256, 64, dtype=torch.float16)
    with pytest.raises(RuntimeError, match="inconsistent shapes"):
        sa.spas_sage2_attn_meansim_topk_cuda(q, q, q[:, :, :128])


def test_broadcast_views_are_copied_not_passed_through():
    """A stride of 0 (expand over heads) is not a layout the strided kernels read; the operator copies, as the
    reference does with .contiguous() (core.py:113-117)."""
    from spargeattn_amd import core
    k = torch.zeros(1, 1, 256, 64, dtype=torch.float16).expand(1, 4, 256, 64)
    assert k.stride(1) == 0
    kc = core._rows_ok(k)
    assert kc.is_contiguous() and kc.shape == k.shape
    nhd = torch.zeros(1, 256, 4, 64, dtype=torch.bfloat16).transpose(1, 2)
    assert core._rows_ok(nhd) is nhd                      # a plain NHD view is read in place


def test_build_refuses_kernels_that_spill():
    from spargeattn_amd import build
    log = """attn.hip:1:1: remark: Function Name: kern_a [-Rpass-analysis=kernel-resource-usage]
attn.hip:1:1: remark:     ScratchSize [bytes/lane]: 0 [-Rpass-analysis=kernel-resource-usage]
attn.hip:1:1: remark:     VGPRs Spill: 0 [-Rpass-analysis=kernel-resource-usage]
attn.hip:2:1: remark: Function Name: kern_b [-Rpass-analysis=kernel-resource-usage]
attn.hip:2:1: remark:     ScratchSize [bytes/lane]: 24 [-Rpass-analysis=kernel-resource-usage]
attn.hip:2:1: remark:     SGPRs Spill: 0 [-Rpass-analysis=kernel-resource-usage]
attn.hip:2:1: remark:     VGPRs Spill: 6 [-Rpass-analysis=kernel-resource-usage]
"""
    bad = build._spill_report(log)
    assert len(bad) == 2 and all(b.startswith("kern_b") for b in bad)


def test_build_names_the_compiler_it_was_validated_with(monkeypatch):
    """attn.hip / dense.hip wait for some inline-asm LDS reads in a later statement; the build refuses (or, with the
    override, warns about) a compiler whose generated code has not been inspected for those windows."""
    from spargeattn_amd import build as b
    ok, version = b.check_compiler()
    assert ok and "roc-7.2.0" in version                      # the toolchain of this image
    monkeypatch.setattr(b, "_compiler_version", lambda: "AMD clang version 99.0.0 (roc-99.0.0)")
    assert b.check_compiler() == (False, "AMD clang version 99.0.0 (roc-99.0.0)")
    monkeypatch.delenv("SPARGEATTN_AMD_ALLOW_UNVALIDATED_COMPILER", raising=False)
    with pytest.raises(RuntimeError, match="not a validated version"):
        b.build(verbose=False)
