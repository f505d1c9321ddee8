"""Oracle for the V path: fp16 cast, per-channel FP8-e4m3 quantisation.  Test infrastructure only.

Restates ``v.to(torch.float16)`` (spas_sage_attn/core.py:113-117) and
``MeanScaleKernel<pad=128, sub_mean=false>`` (csrc/fused/fused.cu:80-191) as
called with ``scale_max = 2.25`` (core.py:151).  The reference's transpose +
16-token permutation (fused.cu:26-77) is an artefact of the NVIDIA mma fragment
and is not restated: the oracle returns V8 in natural (B,H,Npad,D) order.

Arithmetic (binary32, IEEE divide): amax = max_n |v16| ; v_scale = amax/2.25 ;
recp = 2.25/amax ; V8 = e4m3_rne_satfinite(v16 * recp) ; rows N..Npad-1 are 0.
An all-zero channel gives 0*inf = NaN codes, as in the reference (unguarded).
NaN elements do not take part in the channel maximum (fmaxf / fminf, fused.cu:120-123) and get the NaN code.

Pinned by tests/test_oracle_vquant.py: ``torch.float8_e4m3fn`` cast of the same
product (library RNE cast), max|V8| == 2.25 per non-zero channel, dequantisation
error bound.  Parity unpinned: nvcc ``--use_fast_math`` divide bits (setup.py:61).
"""
import numpy as np

from .rounding import f32_to_e4m3fn, e4m3fn_to_f32

F32 = np.float32
SCALE_MAX = F32(2.25)


def to_fp16(v):
    """T -> fp16 (RNE), returned as float32 (core.py:117: bf16 V is cast to fp16)."""
    with np.errstate(over="ignore"):
        return np.asarray(v, dtype=F32).astype(np.float16).astype(F32)


def v_quant_fp8(v16, pad=128):
    """v16 (B,H,N,D) float32 holding fp16 values -> (codes uint8 (B,H,Npad,D), v_scale f32 (B,H,D))."""
    v16 = np.asarray(v16, dtype=F32)
    b, h, n, d = v16.shape
    npad = (n + pad - 1) // pad * pad
    # fmaxf / fminf of the reference (fused.cu:120-123) ignore NaN: a NaN element poisons its own code only
    amax = np.fmax.reduce(np.abs(v16), axis=2, initial=F32(0))
    with np.errstate(divide="ignore", invalid="ignore"):
        v_scale = (amax / SCALE_MAX).astype(F32)
        recp = (SCALE_MAX / amax).astype(F32)
        y = (v16 * recp[:, :, None, :]).astype(F32)
    codes = np.zeros((b, h, npad, d), dtype=np.uint8)
    codes[:, :, :n, :] = f32_to_e4m3fn(y)
    return codes, v_scale


def dequant(codes):
    return e4m3fn_to_f32(codes)
