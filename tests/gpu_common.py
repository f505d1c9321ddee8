"""Shared helpers of the GPU parity tests."""
import numpy as np
import torch

from oracle import rounding as R


def tag_of(dtype):
    return R.BF16 if dtype == torch.bfloat16 else R.FP16


def to_np(t):
    """T-typed torch tensor -> float32 numpy (exact)."""
    return t.detach().float().cpu().numpy()


def bits_equal_T(t_gpu, ref_np, dtype):
    """Bit-exact comparison of a T-typed GPU tensor with oracle values held in float32."""
    got = t_gpu.detach().cpu().view(torch.int16).numpy().view(np.uint16)
    want = R.bits16(ref_np, tag_of(dtype))
    return np.array_equal(got, want.reshape(got.shape))


def v8_natural(v8_tiles, n_rows=None):
    """(B,H,nk,D,64) tile layout -> (B,H,nk*64,D) natural order (numpy uint8)."""
    from spargeattn_amd import _lib
    nat = _lib.v8_tiles_to_natural(v8_tiles).cpu().numpy()
    return nat if n_rows is None else nat[:, :, :n_rows]


def rand_T(shape, dtype, seed, scale=1.0, shift=0.0, device="cuda"):
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale + shift).to(dtype).to(device)
