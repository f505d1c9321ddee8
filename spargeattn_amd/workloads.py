"""Seeded synthetic inputs for the five benchmark / parity configurations.

Every generator is a pure function of (shape, seed, device): the same call on
the CPU and on the GPU box yields the same distribution (not the same bits -
tests always hand ONE generated tensor to both implementations under test).

cfg1  B1 H2  N1024   D64  fp16  0.7*rank-8 smooth field + 0.3*N(0,1), non-causal, topk .5
cfg2  B2 H24 N16384  D128 bf16  N(0,1); mask_id Bernoulli(.3) with diagonal blocks forced on
cfg3  B1 H30 N17776  D64  bf16  13x30x45 Gaussian-filtered field (+.2 noise) + 226 text tokens
cfg4  B1 H32 N32768  D128 bf16  RoPE-rotated rank-16 signal + N(0,1), causal, topk .5 (headline)
cfg5  B1 H24 N118800 D128 bf16  18x60x110 smooth field, topk .3
"""
import math
from dataclasses import dataclass, field

import torch


@dataclass
class Config:
    name: str
    B: int
    H: int
    N: int
    D: int
    dtype: torch.dtype
    is_causal: bool = False
    topk: float = 0.5
    pvthreshd: float = 50.0
    api: str = "topk"          # "topk" or "mask"
    grid: tuple = ()           # (T, Hh, Ww) latent grid for video configs
    text_tokens: int = 0
    seed: int = 1234
    extra: dict = field(default_factory=dict)


CONFIGS = {
    "cfg1": Config("cfg1", 1, 2, 1024, 64, torch.float16, seed=1235),
    "cfg2": Config("cfg2", 2, 24, 16384, 128, torch.bfloat16, api="mask", seed=1236),
    "cfg3": Config("cfg3", 1, 30, 17776, 64, torch.bfloat16, grid=(13, 30, 45), text_tokens=226, seed=1237),
    "cfg4": Config("cfg4", 1, 32, 32768, 128, torch.bfloat16, is_causal=True, seed=1238),
    "cfg5": Config("cfg5", 1, 24, 118800, 128, torch.bfloat16, topk=0.3, grid=(18, 60, 110), seed=1239),
}


def _gen(seed, device):
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    return g


def _randn(shape, g, device):
    return torch.randn(shape, generator=g, device=device, dtype=torch.float32)


def lowrank_smooth(B, H, N, D, rank, g, device):
    """U V^T with U smooth along the sequence (random sinusoids), unit variance."""
    n = torch.arange(N, device=device, dtype=torch.float32)[None, None, :, None] / N
    freq = 1.0 + 7.0 * torch.rand((B, H, 1, rank), generator=g, device=device)
    phase = 2 * math.pi * torch.rand((B, H, 1, rank), generator=g, device=device)
    u = torch.sin(2 * math.pi * freq * n + phase) * math.sqrt(2.0)
    v = _randn((B, H, rank, D), g, device) / math.sqrt(rank)
    return u @ v


def _gauss_kernel(sigma, device):
    r = int(math.ceil(3 * sigma))
    x = torch.arange(-r, r + 1, device=device, dtype=torch.float32)
    k = torch.exp(-0.5 * (x / sigma) ** 2)
    return k / k.sum()


def smooth_field_3d(B, H, grid, D, sigma, g, device):
    """N(0,1) noise on a (T,Hh,Ww) grid, separable Gaussian filter of width sigma, renormalised."""
    T, Hh, Ww = grid
    x = _randn((B * H * D, T, Hh, Ww), g, device)
    k = _gauss_kernel(sigma, device).tolist()
    r = len(k) // 2
    for axis in (1, 2, 3):
        size = x.shape[axis]
        idx = torch.arange(-r, size + r, device=device).clamp(0, size - 1)   # replicate padding
        xp = x.index_select(axis, idx)
        acc = torch.zeros_like(x)
        for o, w in enumerate(k):
            acc.add_(xp.narrow(axis, o, size), alpha=w)
        x = acc
    x = x / x.std()
    return x.view(B, H, D, T * Hh * Ww).transpose(-1, -2).contiguous()


def rope(x):
    """Rotate pairs (d, d + D/2) by position-dependent angles (base 10000)."""
    B, H, N, D = x.shape
    half = D // 2
    inv = 10000.0 ** (-torch.arange(half, device=x.device, dtype=torch.float32) / half)
    ang = torch.arange(N, device=x.device, dtype=torch.float32)[:, None] * inv[None, :]
    c, s = torch.cos(ang), torch.sin(ang)
    a, b = x[..., :half], x[..., half:]
    return torch.cat([a * c - b * s, a * s + b * c], dim=-1)


def make_qkv(cfg: Config, device="cpu", shrink=None):
    """Returns q, k, v (B,H,N,D) in cfg.dtype.  ``shrink`` = dict(B,H,N / grid) overrides for small test copies."""
    B, H, N, D = cfg.B, cfg.H, cfg.N, cfg.D
    grid, text = cfg.grid, cfg.text_tokens
    if shrink:
        B, H = shrink.get("B", B), shrink.get("H", H)
        grid = shrink.get("grid", grid)
        text = shrink.get("text_tokens", text)
        N = shrink.get("N", (grid[0] * grid[1] * grid[2] + text) if grid else N)
    g = _gen(cfg.seed, device)
    if cfg.name == "cfg1":
        q, k, v = (0.7 * lowrank_smooth(B, H, N, D, 8, g, device) + 0.3 * _randn((B, H, N, D), g, device)
                   for _ in range(3))
    elif cfg.name == "cfg2":
        q, k, v = (_randn((B, H, N, D), g, device) for _ in range(3))
    elif cfg.name in ("cfg3", "cfg5"):
        ngrid = grid[0] * grid[1] * grid[2]
        assert ngrid + text == N
        outs = []
        for _ in range(2):
            f = smooth_field_3d(B, H, grid, D, 2.0, g, device) + 0.2 * _randn((B, H, ngrid, D), g, device)
            if text:
                f = torch.cat([f, _randn((B, H, text, D), g, device)], dim=2)
            outs.append(f)
        q, k = outs
        v = _randn((B, H, N, D), g, device)
    elif cfg.name == "cfg4":
        outs = []
        for _ in range(2):
            a = _randn((B, H, N, 16), g, device)
            w = _randn((B, H, 16, D), g, device) / 4.0
            outs.append(rope(a @ w) + _randn((B, H, N, D), g, device))
        q, k = outs
        v = _randn((B, H, N, D), g, device)
    else:
        raise KeyError(cfg.name)
    return q.to(cfg.dtype).contiguous(), k.to(cfg.dtype).contiguous(), v.to(cfg.dtype).contiguous()


def make_mask_id(cfg: Config, B, H, N, device="cpu", p=0.3):
    """Bernoulli(p) 128x64-block mask per head with blocks (i,2i),(i,2i+1) forced to 1 (cfg2)."""
    nq, nk = (N + 127) // 128, (N + 63) // 64
    g = _gen(cfg.seed + 77, device)
    m = (torch.rand((B, H, nq, nk), generator=g, device=device) < p)
    i = torch.arange(nq, device=device)
    for off in (0, 1):
        j = (2 * i + off).clamp(max=nk - 1)
        m[:, :, i, j] = True
    return m.to(torch.int32)
