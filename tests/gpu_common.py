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


def fp8_denominator_case(d=64, nblk=4):
    """One dominant key (score 10000, v = 0) and M = 64*nblk - 1 keys with score 0 and v = 1, scaled so that the
    dominated keys' probability is 2^(8.807 - delta) = 16.9 on the kernel's e4m3 grid, which rounds DOWN to 16:

        reference semantics (e4m3(P) in the numerator, fp32 P in the denominator, offset 8.807)
                                      out = M*16 / (2^8.807 + M*16.9)                    = 0.8576
        denominator summing e4m3(P)   out = M*16 / (448 + M*16)                          = 0.9011
        no exponent offset            out = M*e4m3(0.03773) / (1 + M*0.03773), e4m3 -> 0.0390625 (rounds UP)  = 0.9379

    Returns the operands of block_sparse_attention and the three closed forms."""
    import numpy as np
    n = 64 * nblk
    m_keys = n - 1
    q8 = np.zeros((1, 1, 128, d), np.int8); q8[0, 0, :, 0] = 100
    k8 = np.zeros((1, 1, n, d), np.int8); k8[0, 0, 0, 0] = 100
    v8 = np.full((1, 1, n, d), 0x38, np.uint8); v8[0, 0, 0, :] = 0          # e4m3 code of 1.0; the dominant key carries 0
    lut = np.ones((1, 1, 1, nblk), np.int32); lut[0, 0, 0, 0] = 0
    valid = np.full((1, 1, 1), nblk, np.int32)
    delta = 8.807 - np.log2(16.9)
    a = delta / 10000.0                                   # exponent multiplier: a * (10000 - 0) = delta
    sm_scale = a / (1.44269504088896340736 * 0.01)        # q_scale = k_scale = 0.1
    qs = np.full((1, 1, 1), 0.1, np.float32)
    ks = np.full((1, 1, nblk), 0.1, np.float32)
    vs = np.ones((1, 1, d), np.float32)
    p_max, p_o = 2.0 ** 8.807, 16.9
    forms = {
        "reference": m_keys * 16.0 / (p_max + m_keys * p_o),
        "rounded_denominator": m_keys * 16.0 / (448.0 + m_keys * 16.0),
        "no_offset": m_keys * 0.0390625 / (1.0 + m_keys * p_o / p_max),
    }
    return (q8, k8, v8, lut, valid, np.array([50.0], np.float32), qs, ks, vs, sm_scale), forms
