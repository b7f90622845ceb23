"""Shared test helpers: error metrics and seeded input builders."""
import torch
import torch.nn.functional as F


def rel_l2(ref: torch.Tensor, out: torch.Tensor) -> float:
    """||ref - out||_2 / ||ref||_2 (the reference's RMS ratio, tests/ops/utils.py:5-14)."""
    ref = ref.detach().double().cpu().flatten()
    out = out.detach().double().cpu().flatten()
    base = ref.norm().item()
    return (ref - out).norm().item() / (base if base > 0 else 1.0)


def assert_close(name, ref, out, tol):
    assert out is not None, f"{name}: got None"
    assert tuple(ref.shape) == tuple(out.shape), f"{name}: shape {tuple(out.shape)} != {tuple(ref.shape)}"
    assert torch.isfinite(out.float()).all(), f"{name}: non-finite values"
    err = rel_l2(ref, out)
    print(f"{name}: rel-L2 {err:.3e} (tol {tol})", flush=True)
    assert err < tol, f"{name}: rel-L2 {err:.3e} >= {tol}"


def random_offsets(T: int, N: int, gen: torch.Generator, min_len: int = 1):
    """N sequence lengths >= min_len that sum to T, as cumulative offsets."""
    cuts = torch.randperm(T - N * min_len + N - 1, generator=gen)[:N - 1].sort().values
    lens = torch.diff(torch.cat([torch.tensor([-1]), cuts, torch.tensor([T - N * min_len + N - 1])])) - 1 + min_len
    offs = torch.cat([torch.zeros(1, dtype=torch.long), lens.cumsum(0)])
    assert offs[-1].item() == T
    return offs


def gla_inputs(B, T, H, K, V, seed=0, dtype=torch.bfloat16, normalizer=16.0, h0=True, N=None, h0_std=0.1):
    gen = torch.Generator().manual_seed(seed)
    q = torch.randn(B, T, H, K, generator=gen).to(dtype)
    k = torch.randn(B, T, H, K, generator=gen).to(dtype)
    v = torch.randn(B, T, H, V, generator=gen).to(dtype)
    g = F.logsigmoid(torch.randn(B, T, H, K, generator=gen)) / normalizer
    N = B if N is None else N
    s0 = (torch.randn(N, H, K, V, generator=gen) * h0_std) if h0 else None
    return q, k, v, g, s0


def gdr_inputs(B, T, H, K, V, seed=0, dtype=torch.bfloat16, h0=True, N=None, h0_std=0.1, normalizer=1.0):
    gen = torch.Generator().manual_seed(seed)
    q = torch.randn(B, T, H, K, generator=gen).to(dtype)
    k = F.normalize(torch.randn(B, T, H, K, generator=gen), p=2, dim=-1).to(dtype)
    v = torch.randn(B, T, H, V, generator=gen).to(dtype)
    g = F.logsigmoid(torch.randn(B, T, H, generator=gen)) / normalizer
    beta = torch.randn(B, T, H, generator=gen).sigmoid()
    N = B if N is None else N
    s0 = (torch.randn(N, H, K, V, generator=gen) * h0_std) if h0 else None
    return q, k, v, g, beta, s0
