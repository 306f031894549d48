"""Shared input generators and error metrics for the tests (synthetic, seeded)."""
import numpy as np
import torch

TILE = 64


def make_qkv(B, H, N, D, dtype, seed, n=3):
    """q,k,v(,dO) ~ N(0,1) generated on the CPU from a seed, rounded to `dtype`."""
    g = torch.Generator().manual_seed(seed)
    return [torch.randn(B, H, N, D, generator=g, dtype=torch.float32).to(dtype) for _ in range(n)]


def uniform_block_mask(Bm, Hm, nb, keep, seed):
    """Bernoulli(keep) tiles with the diagonal forced kept."""
    g = torch.Generator().manual_seed(seed)
    m = torch.rand(Bm, Hm, nb, nb, generator=g) < keep
    return m | torch.eye(nb, dtype=torch.bool)


def causal_block_mask(Bm, Hm, nb, keep, seed):
    """Block-causal lower triangle intersected with Bernoulli(keep), diagonal forced kept."""
    g = torch.Generator().manual_seed(seed)
    m = (torch.rand(Bm, Hm, nb, nb, generator=g) < keep) & torch.tril(torch.ones(nb, nb, dtype=torch.bool))
    return m | torch.eye(nb, dtype=torch.bool)


def errors(x, ref):
    """(max-abs, rel-L2) of x against ref, both brought to float64 numpy."""
    x = np.asarray(x.detach().float().cpu().numpy() if isinstance(x, torch.Tensor) else x, dtype=np.float64)
    ref = np.asarray(ref.detach().float().cpu().numpy() if isinstance(ref, torch.Tensor) else ref, dtype=np.float64)
    d = x - ref
    return float(np.abs(d).max()), float(np.linalg.norm(d) / max(np.linalg.norm(ref), 1e-30))


def f32(x):
    return x.detach().float().cpu().numpy()


def same_up_to_rounding(a, b, rel=2.0 ** -9, abs_=3e-4):
    """Two runs of the forward may split a row's tiles differently over wavefronts (tiles are handed
    out dynamically), which changes the summation order and the reference exponents the fp16
    probabilities are rounded against: equal up to two rounding steps of the 16-bit output."""
    a = a.detach().float().cpu().numpy() if isinstance(a, torch.Tensor) else np.asarray(a, dtype=np.float32)
    b = b.detach().float().cpu().numpy() if isinstance(b, torch.Tensor) else np.asarray(b, dtype=np.float32)
    return bool(np.all(np.abs(a - b) <= rel * np.abs(b) + abs_))
