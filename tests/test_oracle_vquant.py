"""Pins oracle/vquant.py against torch's float8_e4m3fn cast and closed forms."""
import numpy as np
import torch

from oracle import vquant as vq
from oracle import rounding as R


def test_v_quant_against_torch_cast():
    rng = np.random.default_rng(0)
    b, h, n, d = 2, 2, 200, 64
    v = R.round_to(rng.standard_normal((b, h, n, d)) * np.array([0.01, 3.0])[None, :, None, None], R.BF16)
    v16 = vq.to_fp16(v)
    assert np.array_equal(v16, torch.from_numpy(v).to(torch.float16).float().numpy())
    codes, v_scale = vq.v_quant_fp8(v16)
    assert codes.shape == (b, h, 256, d) and np.all(codes[:, :, n:] == 0)          # zero padding to 128
    t = torch.from_numpy(v16)
    amax = t.abs().amax(dim=2)
    assert np.array_equal(v_scale, (amax / 2.25).numpy())
    # IEEE binary32 divide (numpy); torch's scalar/tensor goes through a reciprocal and is 1 ulp off at times
    recp = torch.from_numpy(np.float32(2.25) / amax.numpy())
    ref = (t * recp[:, :, None, :]).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(codes[:, :, :n], ref)
    deq = vq.dequant(codes[:, :, :n])
    assert np.all(np.abs(deq).max(axis=2) == 2.25)                                  # channel max hits 2.25 exactly
    err = np.abs(deq * v_scale[:, :, None, :] - v16)
    assert np.all(err <= np.abs(v16) * 2.0 ** -4 + v_scale[:, :, None, :] * 2.0 ** -10)


def test_v_quant_zero_channel_is_nan_like_reference():
    v = np.ones((1, 1, 128, 64), np.float32)
    v[..., 3] = 0
    codes, v_scale = vq.v_quant_fp8(v)
    assert v_scale[0, 0, 3] == 0 and np.all(codes[0, 0, :, 3] & 0x7F == 0x7F)
    assert np.all(vq.dequant(codes[0, 0, :, 0]) == 2.25)
