"""Host-side helpers of the operator API: hyper-parameter normalisation, the mask-prediction
pipeline on top of the C ABI, precision metrics.

Mirrors the interface of spas_sage_attn/utils.py (thu-ml/SpargeAttn): ``hyperparameter_check``
(utils.py:38-50), ``get_block_map_meansim_fuse_quant`` (utils.py:371-421),
``get_vanilla_qk_quant`` (utils.py:265-268), ``block_map_lut_triton`` (utils.py:76-87),
``block_map_to_mask`` (utils.py:424-432) and ``precision_metric`` (utils.py:25-36); the work itself
is done by HIP kernels behind libspargeattn_amd.so.
"""
import torch
from torch import Tensor

from . import _lib

BLKQ = 128
BLKK = 64


def hyperparameter_check(hyper, H, device):
    """Scalar, 0-d tensor or (H,) tensor -> (H,) float32 tensor on ``device``."""
    if type(hyper) is float or type(hyper) is int:
        return torch.full((H,), float(hyper), device=device, dtype=torch.float32)
    if isinstance(hyper, Tensor):
        assert hyper.dim() <= 1, "Hyperparameter tensor must be 1D"
        if hyper.dim() == 0:
            return torch.full((H,), hyper.item(), device=device, dtype=torch.float32)
        assert hyper.numel() == H, f"Hyperparameter tensor must have {H} elements, but has {hyper.numel()}"
        return hyper.to(device=device, dtype=torch.float32).contiguous()
    print(hyper)
    raise ValueError("Hyperparameter must be a float or a tensor")


def _check_blocks(BLKQ_, BLKK_):
    if (BLKQ_, BLKK_) != (BLKQ, BLKK):
        raise ValueError("the gfx950 kernels use 128-row Q blocks and 64-row K blocks")


def _q_quant_rows(qk_quant_gran):
    """Rows of Q that share one INT8 scale: the block, or the 32 rows of a warp / wavefront (per_warp_int8 with
    WARPQ = 32, spas_sage_attn/quant_per_block.py:102-148).  K scales are per 64-row block in both granularities."""
    return BLKQ if _lib.quant_gran(qk_quant_gran) == _lib.QUANT_PER_BLOCK else 32


def get_vanilla_qk_quant(q, k, km=None, BLKQ=128, BLKK=64, qk_quant_gran=1):
    """INT8 quantisation of q and (k - km) without pooling: per block, or with qk_quant_gran = 2 ("per_warp") one scale
    per 32 query rows, q_scale (B,H,nq*4)."""
    _check_blocks(BLKQ, BLKK)
    _, _, q_int8, q_scale = _lib.pool_sim_quant(q, None, BLKQ, with_pool=False, quant_rows=_q_quant_rows(qk_quant_gran))
    _, _, k_int8, k_scale = _lib.pool_sim_quant(k, km, BLKK, with_pool=False)
    return q_int8, q_scale, k_int8, k_scale


def _check_block_size(block_size):
    if block_size not in (BLKQ, BLKK):
        raise ValueError("the gfx950 kernels pool and quantise 128-row or 64-row blocks")


def get_quant(x, x_mean, block_size):
    """Per-block INT8 quantisation of x, or of (x - x_mean) when the (B,H,1,D) column mean is given
    (spas_sage_attn/utils.py:255-263): returns (x_int8, x_scale)."""
    _check_block_size(block_size)
    _, _, x_int8, x_scale = _lib.pool_sim_quant(x, x_mean, block_size, with_pool=False)
    return x_int8, x_scale


def get_pool_sim_triton_simmean_fuse_quant(x, x_mean, block_size, simthreshd1):
    """Block means, self-similarity flags and the INT8 quantisation in one pass over x
    (spas_sage_attn/utils.py:270-280): returns (pool, sim_blocks, x_int8, x_scale).  simthreshd1 is the (H,) float32
    tensor hyperparameter_check returns.  The name is kept for drop-in compatibility; no Triton is involved."""
    _check_block_size(block_size)
    return _lib.pool_sim_quant(x, x_mean, block_size, simthreshd1)


def get_pool_sim_triton_simmean(x, block_size, simthreshd1):
    """Block means and self-similarity flags only (spas_sage_attn/utils.py:243-252): returns (pool, sim_blocks).
    The fused kernel computes the quantisation as well; its int8 output is dropped."""
    pool, sim, _, _ = get_pool_sim_triton_simmean_fuse_quant(x, None, block_size, simthreshd1)
    return pool, sim


def block_map_lut_triton(block_map):
    """Block map (B,H,nq,nk), non-zero = keep -> (delta LUT int32, valid_block_num int32).

    The name is kept for drop-in compatibility; no Triton is involved."""
    assert block_map.dim() == 4
    assert block_map.is_contiguous()
    return _lib.map_to_lut(block_map)


block_map_lut = block_map_lut_triton


def get_block_map_meansim_fuse_quant(q, k, km=None, is_causal=False, BLKQ=128, BLKK=64, simthreshd1=0.1,
                                     cdfthreshd=0.9, topk=None, is_sparse=True, return_lut=False,
                                     attention_sink=False, qk_quant_gran=1):
    """Mask prediction fused with Q/K quantisation.  ``qk_quant_gran`` = 2 ("per_warp") quantises Q in 32-row groups
    (q_scale (B,H,nq*4)); pooling, flags and the block map do not depend on it.

    Returns (lut, valid_block_num, q_int8, q_scale, k_int8, k_scale) when ``return_lut`` else
    (block_map bool, q_int8, q_scale, k_int8, k_scale)."""
    assert (cdfthreshd is None and topk is not None) \
        or (cdfthreshd is not None and topk is None), "Only one of cdfthreshd and topk can be set."
    _check_blocks(BLKQ, BLKK)
    H, Hkv = q.size(1), k.size(1)
    if Hkv <= 0 or H % Hkv != 0:
        # the message of the reference's kernel entry (qk_int_sv_f8_cuda_sm89.cu:310-314)
        raise ValueError(f"num_qo_heads ({H}) must be divisible by num_kv_heads ({Hkv})")
    per_head_sim = isinstance(simthreshd1, Tensor) and simthreshd1.dim() == 1
    simthreshd1 = hyperparameter_check(simthreshd1, H, q.device)
    if cdfthreshd is not None:
        cdfthreshd = hyperparameter_check(cdfthreshd, H, q.device)
    if topk is not None:
        topk = hyperparameter_check(topk, H, q.device)
    pool_q, sim_q, q_int8, q_scale = _lib.pool_sim_quant(q, None, BLKQ, simthreshd1, quant_rows=_q_quant_rows(qk_quant_gran))
    # Grouped K/V heads (an extension: the reference's pooled-score matmul needs Hkv == H, utils.py:388).  K is pooled and
    # quantised once per K head, so its similarity flags can follow ONE threshold per group: the query heads of a group
    # must agree on simthreshd1 (a per-head tensor that differs inside a group is refused rather than silently reduced
    # to its first entry); every query head of the group is scored against those pooled blocks with its own topk /
    # cdfthreshd.
    if Hkv != H and per_head_sim:
        grouped = simthreshd1.view(Hkv, H // Hkv)
        if not bool((grouped == grouped[:, :1]).all()):
            raise ValueError("simthreshd1 must be equal for the query heads that share a K/V head "
                             f"({H} query heads, {Hkv} K/V heads): K is pooled once per K/V head")
    simthreshd1_k = simthreshd1 if Hkv == H else simthreshd1[::H // Hkv].contiguous()
    pool_k, sim_k, k_int8, k_scale = _lib.pool_sim_quant(k, km, BLKK, simthreshd1_k)
    lut, valid, bmap = _lib.block_select(pool_q, sim_q, pool_k, sim_k, topk=topk, cdfthreshd=cdfthreshd,
                                         is_causal=is_causal, attention_sink=attention_sink,
                                         return_map=not return_lut)
    if return_lut:
        return lut, valid, q_int8, q_scale, k_int8, k_scale
    return bmap, q_int8, q_scale, k_int8, k_scale


def get_block_map_meansim(q, k, is_causal=False, BLKQ=128, BLKK=64, simthreshd1=0.1, cdfthreshd=0.9, topk=None,
                          is_sparse=True, return_lut=False, attention_sink=False):
    """Mask prediction only (spas_sage_attn/utils.py:318-369); Q/K are not smoothed here."""
    out = get_block_map_meansim_fuse_quant(q, k, None, is_causal, BLKQ, BLKK, simthreshd1, cdfthreshd, topk,
                                           is_sparse, return_lut, attention_sink)
    return out[:2] if return_lut else out[0]


def block_map_to_mask(block_map, BLKQ=128, BLKK=64):
    """Expand a block map to a token-level boolean mask (B,H,nq*BLKQ,nk*BLKK)."""
    return block_map.bool().repeat_interleave(BLKQ, dim=-2).repeat_interleave(BLKK, dim=-1)


def precision_metric(quant_o, fa2_o, verbose=True, round_num=4):
    if quant_o.shape[-2] > 200000:
        quant_o, fa2_o = quant_o.cpu(), fa2_o.cpu()
    x, y = quant_o.float(), fa2_o.float()
    sim = torch.nn.functional.cosine_similarity(x.reshape(1, -1), y.reshape(1, -1)).item()
    l1 = ((x - y).abs().sum() / y.abs().sum()).item()
    rmse = torch.sqrt(torch.mean((x - y) ** 2)).item()
    sim, l1, rmse = round(sim, round_num), round(l1, round_num), round(rmse, round_num)
    if verbose:
        print(f"Cossim: {sim:.6f}, L1: {l1:.6f}, RMSE:{rmse:.6f}")
    return {"Cossim": sim, "L1": l1, "RMSE": rmse}
