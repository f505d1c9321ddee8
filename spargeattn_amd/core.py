"""Operator API: drop-in for ``spas_sage_attn.core`` of thu-ml/SpargeAttn on MI355X.

    spas_sage2_attn_meansim_topk_cuda   spas_sage_attn/core.py:105-169
    spas_sage2_attn_meansim_cuda        spas_sage_attn/core.py:39-103   (CDF selection)
    block_sparse_sage2_attn_cuda        spas_sage_attn/core.py:171-233
    spas_sage_attn_meansim_cuda         spas_sage_attn/core.py:235-276  (INT8 QK^T, FP16 PV, CDF selection)
    spas_sage_attn_meansim_topk_cuda    spas_sage_attn/core.py:278-319  (INT8 QK^T, FP16 PV, top-k selection)

Same names, argument order, defaults and return values.  The ``_cuda`` suffix is kept so that
callers need no change; everything runs as HIP kernels for gfx950.  As in the reference,
``attn_mask``, ``dropout_p`` and ``output_dtype`` are accepted and ignored, the output dtype is
fp16 for fp32/fp16 inputs and bf16 for bf16 inputs, and causality is enforced at 128x64-block
granularity through the LUT (the reference passes ``is_causal=False`` to its kernel, core.py:154-158).
``kernel_causal=True`` is an extension that additionally masks at token level.
``qk_quant_gran`` (keyword, default 1 = the reference's operators) selects the INT8 granularity of the kernel entry
(csrc/qattn/attn_cuda.h:61-76): 1 / "per_block", or 2 / "per_warp" - one Q scale per 32 query rows
(spas_sage_attn/quant_per_block.py:102-148), which lowers the quantisation error at no cost in time.
"""
import torch

from . import _lib
from .utils import (hyperparameter_check, get_block_map_meansim_fuse_quant, get_vanilla_qk_quant,
                    block_map_lut_triton)


# Optional callable(name) invoked at stage boundaries ("km", "maskpred", "vquant", "attn", "end");
# bench.py installs one that records HIP events on the current stream.  None in normal use.
_stage_hook = None


def _mark(name):
    if _stage_hook is not None:
        _stage_hook(name)


def _prologue(q, k, v, tensor_layout):
    assert tensor_layout in ['HND', 'NHD']
    if tensor_layout == 'NHD':
        q, k, v = (t.transpose(-2, -3) for t in (q, k, v))
    assert q.size(-2) >= 128, "seq_len should be not less than 128."
    assert q.size(-1) in [64, 128], "headdim should be in [64, 128]. For other headdim, you can use padding and specify the softmax scale."
    # q may be shorter or longer than k/v (qo_len / kv_len of csrc/qattn/qk_int_sv_f8_cuda_sm89.cu:256-300); k and v
    # must agree with each other and with q in batch and head_dim, which the reference's kernel entry checks
    # (CHECK_SHAPE, sm89.cu:339-363 -> RuntimeError)
    if (q.dim() != 4 or k.dim() != 4 or v.dim() != 4 or k.shape[:3] != v.shape[:3] or k.size(0) != q.size(0)
            or k.size(-1) != q.size(-1) or v.size(-1) != q.size(-1)):
        raise RuntimeError(f"inconsistent shapes: q {tuple(q.shape)}, k {tuple(k.shape)}, v {tuple(v.shape)} "
                           "(as (B,H,N,D): k and v must have the same batch, heads and length, and q's batch and head_dim)")
    if not v.is_cuda:
        raise RuntimeError("spargeattn_amd needs GPU tensors (there is no CPU path)")
    torch.cuda.set_device(v.device)
    qk_dtype = torch.bfloat16 if q.dtype == torch.bfloat16 else torch.float16
    # The reference makes contiguous HND copies here (core.py:113-117).  The kernels that read q, k, v take strides, so
    # an NHD tensor (or any view whose rows are contiguous and 16-byte aligned) is read where it lies; only other
    # layouts and dtypes are copied.
    q = _rows_ok(q).to(qk_dtype)
    k = _rows_ok(k).to(qk_dtype)
    # V is always quantised from fp16 (core.py:117).  A bf16 V is handed over as it is: the quantisation kernel
    # rounds each element to fp16 in registers, which gives the same values without a pass over HBM.
    v = _rows_ok(v)
    if v.dtype not in (torch.float16, torch.bfloat16):
        v = v.to(torch.float16)
    return q, k, v


def _rows_ok(t):
    """t itself if the strided kernels can read it (last dimension contiguous, 16-byte aligned rows), else a copy."""
    esz = t.element_size()
    # a stride of 0 (an expanded / broadcast view) or a negative one is not something the kernels take: copy, as the
    # reference does for every input (core.py:113-117)
    ok = (t.stride(-1) == 1 and t.data_ptr() % 16 == 0 and t.dtype in (torch.float16, torch.bfloat16)
          and all(st > 0 and (st * esz) % 16 == 0 for st in t.stride()[:-1]))
    return t if ok else t.contiguous()


def _empty_out(q):
    """Output buffer with q's shape whose MEMORY layout follows q's (an NHD view gets an NHD buffer, so that the
    transpose back at the end is a view of contiguous memory)."""
    if q.is_contiguous():
        return torch.empty_like(q)
    if q.transpose(-2, -3).is_contiguous():
        return torch.empty_like(q.transpose(-2, -3)).transpose(-2, -3)
    return torch.empty(q.shape, dtype=q.dtype, device=q.device)


def _attention(q, k, v, q_int8, q_scale, k_int8, k_scale, lut, valid_block_num, scale, pvthreshd, kernel_causal,
               return_pv_count=False, qk_quant_gran=1):
    headdim = q.size(-1)
    if scale is None:
        scale = 1.0 / (headdim ** 0.5)
    assert headdim in [64, 128], "headdim should be in [64, 128]. For other headdim, you can use padding and specify the softmax scale."
    pvthreshd = hyperparameter_check(pvthreshd, q.size(-3), q.device)
    o = _empty_out(q)
    _mark("vquant")
    v_fp8, v_scale = _lib.v_quant_fp8(v)
    _mark("attn")
    pvc = _lib.block_sparse_attn(q_int8, k_int8, v_fp8, o, lut, valid_block_num, pvthreshd, q_scale, k_scale, v_scale,
                                 scale, is_causal=kernel_causal, return_pv_count=return_pv_count,
                                 qk_quant_gran=qk_quant_gran)
    _mark("end")
    return o, pvc


def _finish(o, tensor_layout, return_sparsity, valid_block_num, lut, causal_denominator):
    if tensor_layout == 'NHD':
        o = o.transpose(-2, -3)
    if return_sparsity:
        nq, nk = lut.size(2), lut.size(3)
        cols = (nk + 2) // 2 if causal_denominator else nk
        qk_sparsity = 1 - (valid_block_num.float().sum()) / (cols * nq * lut.size(0) * lut.size(1))
        return o, qk_sparsity.item()
    return o


def _meansim(q, k, v, is_causal, scale, smooth_k, simthreshd1, cdfthreshd, topk, pvthreshd, attention_sink,
             tensor_layout, return_sparsity, kernel_causal, qk_quant_gran=1):
    qk_quant_gran = _lib.quant_gran(qk_quant_gran)
    q, k, v = _prologue(q, k, v, tensor_layout)
    if not smooth_k:
        # the reference leaves `km` undefined in this case (core.py:119-126)
        raise NameError("name 'km' is not defined")
    _mark("km")
    km = _lib.km_mean(k)
    _mark("maskpred")
    lut, valid_block_num, q_int8, q_scale, k_int8, k_scale = get_block_map_meansim_fuse_quant(
        q, k, km, is_causal=is_causal, simthreshd1=simthreshd1, cdfthreshd=cdfthreshd, topk=topk, return_lut=True,
        attention_sink=attention_sink, BLKQ=128, BLKK=64, qk_quant_gran=qk_quant_gran)
    o, _ = _attention(q, k, v, q_int8, q_scale, k_int8, k_scale, lut, valid_block_num, scale, pvthreshd, kernel_causal,
                      qk_quant_gran=qk_quant_gran)
    return _finish(o, tensor_layout, return_sparsity, valid_block_num, lut, causal_denominator=is_causal is not False)


def _meansim_sage1(q, k, v, is_causal, scale, smooth_k, simthreshd1, cdfthreshd, topk, pvthreshd, attention_sink,
                   tensor_layout, return_sparsity, qk_quant_gran=1):
    """INT8 QK^T / FP16 PV path (spas_sage_attn/core.py:235-319): fp16 V, token-level causal masking in the kernel,
    sparsity reported against the full grid unless is_causal."""
    qk_quant_gran = _lib.quant_gran(qk_quant_gran)
    q, k, v = _prologue(q, k, v, tensor_layout)
    if not smooth_k:
        raise NameError("name 'km' is not defined")           # as the reference (core.py:249-252)
    _mark("km")
    km = _lib.km_mean(k)
    _mark("maskpred")
    lut, valid_block_num, q_int8, q_scale, k_int8, k_scale = get_block_map_meansim_fuse_quant(
        q, k, km, is_causal=is_causal, simthreshd1=simthreshd1, cdfthreshd=cdfthreshd, topk=topk, return_lut=True,
        attention_sink=attention_sink, qk_quant_gran=qk_quant_gran)
    headdim = q.size(-1)
    if scale is None:
        scale = 1.0 / (headdim ** 0.5)
    assert headdim in [64, 128], "headdim should be in [64, 128]. For other headdim, you can use padding and specify the softmax scale."
    pvthreshd = hyperparameter_check(pvthreshd, q.size(-3), q.device)
    o = _empty_out(q)
    _mark("vquant")
    vt = _lib.v_tiles_f16_swizzled(v)
    _mark("attn")
    _lib.block_sparse_attn_f16v(q_int8, k_int8, vt, o, lut, valid_block_num, pvthreshd, q_scale, k_scale, scale,
                                is_causal=bool(is_causal), qk_quant_gran=qk_quant_gran)
    _mark("end")
    return _finish(o, tensor_layout, return_sparsity, valid_block_num, lut, causal_denominator=is_causal is not False)


@torch.compiler.disable
def spas_sage_attn_meansim_cuda(q, k, v, attn_mask=None, dropout_p=0.0, is_causal=False, scale=None, smooth_k=True,
                                simthreshd1=0.6, cdfthreshd=0.98, pvthreshd=50, attention_sink=False,
                                tensor_layout="HND", output_dtype=torch.float16, return_sparsity=False, *,
                                qk_quant_gran=1):
    return _meansim_sage1(q, k, v, is_causal, scale, smooth_k, simthreshd1, cdfthreshd, None, pvthreshd,
                          attention_sink, tensor_layout, return_sparsity, qk_quant_gran)


@torch.compiler.disable
def spas_sage_attn_meansim_topk_cuda(q, k, v, attn_mask=None, dropout_p=0.0, is_causal=False, scale=None,
                                     smooth_k=True, simthreshd1=-0.1, cdfthreshd=None, topk=0.5, pvthreshd=50,
                                     attention_sink=False, tensor_layout="HND", output_dtype=torch.float16,
                                     return_sparsity=False, *, qk_quant_gran=1):
    return _meansim_sage1(q, k, v, is_causal, scale, smooth_k, simthreshd1, cdfthreshd, topk, pvthreshd,
                          attention_sink, tensor_layout, return_sparsity, qk_quant_gran)


@torch.compiler.disable
def spas_sage2_attn_meansim_cuda(q, k, v, attn_mask=None, dropout_p=0.0, is_causal=False, scale=None, smooth_k=True,
                                 simthreshd1=0.6, cdfthreshd=0.98, pvthreshd=50, attention_sink=False,
                                 tensor_layout="HND", output_dtype=torch.float16, return_sparsity=False,
                                 kernel_causal=False, *, qk_quant_gran=1):
    return _meansim(q, k, v, is_causal, scale, smooth_k, simthreshd1, cdfthreshd, None, pvthreshd, attention_sink,
                    tensor_layout, return_sparsity, kernel_causal, qk_quant_gran)


@torch.compiler.disable
def spas_sage2_attn_meansim_topk_cuda(q, k, v, attn_mask=None, dropout_p=0.0, is_causal=False, scale=None,
                                      smooth_k=True, simthreshd1=-0.1, cdfthreshd=None, topk=0.5, pvthreshd=50,
                                      attention_sink=False, tensor_layout="HND", output_dtype=torch.float16,
                                      return_sparsity=False, kernel_causal=False, *, qk_quant_gran=1):
    return _meansim(q, k, v, is_causal, scale, smooth_k, simthreshd1, cdfthreshd, topk, pvthreshd, attention_sink,
                    tensor_layout, return_sparsity, kernel_causal, qk_quant_gran)


@torch.compiler.disable
def block_sparse_sage2_attn_cuda(q, k, v, mask_id=None, dropout_p=0.0, scale=None, smooth_k=True, pvthreshd=50,
                                 attention_sink=False, tensor_layout="HND", output_dtype=torch.float16,
                                 return_sparsity=False, kernel_causal=False, *, qk_quant_gran=1):
    qk_quant_gran = _lib.quant_gran(qk_quant_gran)
    q, k, v = _prologue(q, k, v, tensor_layout)
    if not smooth_k:
        raise NameError("name 'km' is not defined")
    _mark("km")
    km = _lib.km_mean(k)
    _mark("maskpred")
    q_int8, q_scale, k_int8, k_scale = get_vanilla_qk_quant(q, k, km, 128, 64, qk_quant_gran=qk_quant_gran)
    lut, valid_block_num = block_map_lut_triton(block_map=mask_id)
    o, _ = _attention(q, k, v, q_int8, q_scale, k_int8, k_scale, lut, valid_block_num, scale, pvthreshd, kernel_causal,
                      qk_quant_gran=qk_quant_gran)
    # the reference always reports against the causal denominator here (core.py:230)
    return _finish(o, tensor_layout, return_sparsity, valid_block_num, lut, causal_denominator=True)
