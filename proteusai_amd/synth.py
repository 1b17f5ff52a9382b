"""Deterministic synthetic inputs: C-alpha random-walk chains, the wavelength
schedule of README.md:24, log-spaced attention spreads, padded lengths.

Everything is generated on the CPU from a seeded torch.Generator so that the
GPU kernels and the CPU checkers see identical bits.
"""
import math

import torch


def random_walk_chain(n: int, gen: torch.Generator, bond: float = 3.8) -> torch.Tensor:
    """[n,3] float32 chain: unit steps in uniformly random directions, fixed bond length."""
    u = torch.randn(n, 3, generator=gen, dtype=torch.float64)
    u = u / u.norm(dim=1, keepdim=True)
    steps = bond * u
    steps[0] = 0.0
    return torch.cumsum(steps, dim=0).to(torch.float32)


def radius_of_gyration(x: torch.Tensor) -> float:
    x = x.double()
    return float(((x - x.mean(0)) ** 2).sum(1).mean().sqrt())


def compact_chain(x: torch.Tensor, gen: torch.Generator) -> torch.Tensor:
    """Centre, rotate by a Haar-random rotation and scale to Rg = 2.2 * n^0.38 angstrom."""
    n = x.shape[0]
    xd = x.double()
    xd = xd - xd.mean(0)
    a = torch.randn(3, 3, generator=gen, dtype=torch.float64)
    q, r = torch.linalg.qr(a)
    q = q * torch.sign(torch.diagonal(r))[None, :]
    if torch.det(q) < 0:
        q[:, 0] = -q[:, 0]
    xd = xd @ q.T
    target = 2.2 * n ** 0.38
    xd = xd * (target / radius_of_gyration(xd))
    return xd.to(torch.float32)


def wavelength_schedule(d_model: int = 512, lmin: float = 3.7, lmax: float = 20.0, base: float = 20.0) -> torch.Tensor:
    """lambda_i = lmin + (lmax-lmin)(b^(2i/d_model) - 1)/(b - 1), i = 0..d_model/2-1 (README.md:24)."""
    i = torch.arange(d_model // 2, dtype=torch.float64)
    return lmin + (lmax - lmin) * (base ** (2 * i / d_model) - 1) / (base - 1)


def wavenumbers(d_model: int = 512, lmin: float = 3.7, lmax: float = 20.0, base: float = 20.0) -> torch.Tensor:
    return (2 * math.pi / wavelength_schedule(d_model, lmin, lmax, base)).to(torch.float32)


def log_spaced_sigma(heads: int = 8, lo: float = 3.0, hi: float = 25.0) -> torch.Tensor:
    h = torch.arange(heads, dtype=torch.float64)
    if heads == 1:
        return torch.tensor([lo], dtype=torch.float32)
    return (lo * (hi / lo) ** (h / (heads - 1))).to(torch.float32)


def we_inputs(n: int, seed: int, batch: int = 1, d_model: int = 512, compact: bool = False):
    """(coords [Z,n,3], wavenumbers [K]) for the WE configurations."""
    gen = torch.Generator().manual_seed(seed)
    chains = []
    for _ in range(batch):
        x = random_walk_chain(n, gen)
        if compact:
            x = compact_chain(x, gen)
        chains.append(x)
    return torch.stack(chains), wavenumbers(d_model)


def attn_inputs(batch: int, heads: int, n: int, d_head: int, seed: int, min_len: int = None,
                compact: bool = False, coords: torch.Tensor = None):
    """(Q, K, V bf16 [Z,H,n,d], coords [Z,n,3], sigma [H], key_padding_mask [Z,n] or None)."""
    gen = torch.Generator().manual_seed(seed)
    scale = 1.0 / math.sqrt(d_head)
    Q = (torch.randn(batch, heads, n, d_head, generator=gen) * scale).to(torch.bfloat16)
    K = (torch.randn(batch, heads, n, d_head, generator=gen) * scale).to(torch.bfloat16)
    V = (torch.randn(batch, heads, n, d_head, generator=gen) * scale).to(torch.bfloat16)
    if coords is None:
        chains = []
        for _ in range(batch):
            x = random_walk_chain(n, gen)
            if compact:
                x = compact_chain(x, gen)
            chains.append(x)
        coords = torch.stack(chains)
    mask = None
    if min_len is not None:
        lens = torch.randint(min_len, n + 1, (batch,), generator=gen)
        mask = torch.arange(n)[None, :] >= lens[:, None]
    return Q, K, V, coords, log_spaced_sigma(heads), mask
