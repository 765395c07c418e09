"""Seeded synthetic inputs of the benchmark configurations (test infrastructure).

Everything is drawn on the CPU from ``torch.Generator().manual_seed(seed)`` in fp32 and then
cast, so the CPU checker and the GPU kernels see identical bits (the reference's tests use the
same recipe, tests/test_interface.py:38-42).
"""
import torch


def _gen(seed):
    return torch.Generator().manual_seed(seed)


def randn_bf16(shape, seed, dtype=torch.bfloat16):
    return torch.randn(shape, generator=_gen(seed), dtype=torch.float32).to(dtype)


def qkv(B, H, Sq, Skv, D, seed=0, dtype=torch.bfloat16, rms_norm_qk=False):
    """q [B,H,Sq,D], k,v [B,H,Skv,D] iid N(0,1); optionally q,k RMS-normalised over D per
    (head, token) in fp32 (x / sqrt(mean(x^2) + 1e-6)), as HunyuanVideo's qk-norm does."""
    g = _gen(seed)
    q = torch.randn((B, H, Sq, D), generator=g, dtype=torch.float32)
    k = torch.randn((B, H, Skv, D), generator=g, dtype=torch.float32)
    v = torch.randn((B, H, Skv, D), generator=g, dtype=torch.float32)
    if rms_norm_qk:
        q = q * torch.rsqrt(q.pow(2).mean(-1, keepdim=True) + 1e-6)
        k = k * torch.rsqrt(k.pow(2).mean(-1, keepdim=True) + 1e-6)
    return q.to(dtype), k.to(dtype), v.to(dtype)


def fbcache_pair(shape, seed=1234, noise=0.05, dtype=torch.bfloat16):
    """prev ~ N(0,1); cur = prev + noise * N(0,1), both rounded to ``dtype``."""
    g = _gen(seed)
    prev = torch.randn(shape, generator=g, dtype=torch.float32)
    cur = prev + noise * torch.randn(shape, generator=g, dtype=torch.float32)
    return prev.to(dtype), cur.to(dtype)


def block_mask(H, nQ, nK, seed=0, window=4, sinks=2, density=0.30):
    """bool [H,nQ,nK]: |i - j| <= window, or j < sinks, or a random fill chosen so the total
    density is about ``density``.  Returns (mask, realised density)."""
    i = torch.arange(nQ)[:, None]
    j = torch.arange(nK)[None, :]
    base = ((i - j).abs() <= window) | (j < sinks)
    base_density = base.float().mean().item()
    p_fill = max(0.0, (density - base_density) / max(1e-9, 1.0 - base_density))
    fill = torch.rand((H, nQ, nK), generator=_gen(seed)) < p_fill
    mask = base[None] | fill
    return mask, mask.float().mean().item()
