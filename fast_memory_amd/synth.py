"""Seeded synthetic workloads of the five benchmark configurations.

Everything is plain torch and runs on whichever device is asked for: the tests
generate small cases on the CPU, the benchmark generates the large ones on the
GPU (device memory and random numbers are the only things torch is used for).

Keys are a mixture of von Mises-Fisher clusters on the unit sphere (Wood's
1994 rejection sampler) scaled by log-normal norms; queries are vMF samples
around the same centres scaled to norm sqrt(d); values are N(0,1).
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Optional

import torch


@dataclass(frozen=True)
class Config:
    name: str
    dtype: torch.dtype
    H: int            # KV heads
    G: int            # query heads per KV head
    d: int
    N: int            # memory keys per KV head
    C: int            # buckets
    Z: int            # keys per bucket
    S: int            # query tokens per query head
    n_clusters: int   # mixture components (0 = plain N(0,1) keys)
    kappa: float
    kmeans_iters: int
    local: int        # local keys merged in with dense attention (0 = none)
    seed: int

    @property
    def Sq(self) -> int:
        return self.G * self.S


CONFIGS = {
    "c1": Config("c1-toy-fp32", torch.float32, 1, 1, 64, 4096, 64, 256, 512, 0, 0.0, 1, 0, 1001),
    "c2": Config("c2-prefill-bf16", torch.bfloat16, 8, 4, 128, 32768, 256, 1024, 2048, 256, 20.0, 2, 0, 1002),
    "c4": Config("c4-index-build-bf16", torch.bfloat16, 8, 4, 128, 262144, 1024, 4096, 2048, 1024, 20.0, 2, 0, 1004),
    "c5": Config("c5-1M-bf16", torch.bfloat16, 8, 8, 128, 1048576, 2048, 16384, 4096, 2048, 30.0, 2, 4096, 1005),
}


def decode_lengths(n_seq: int = 64, lo: int = 8192, hi: int = 131072, seed: int = 1003):
    """Memory lengths of the varlen decode batch (config 3), with the
    per-sequence C = round(sqrt(N)), Z = round(4 sqrt(N))."""
    g = torch.Generator().manual_seed(seed)
    Ns = torch.randint(lo, hi + 1, (n_seq,), generator=g).tolist()
    return [(n, int(round(math.sqrt(n))), int(round(4 * math.sqrt(n)))) for n in Ns]


def _gen(device, seed: int) -> torch.Generator:
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    return g


def vmf_w(n: int, p: int, kappa: float, g: torch.Generator, device) -> torch.Tensor:
    """Cosines w = <x, mu> of n vMF(mu, kappa) samples in dimension p (Wood 1994).
    The proposal uses Beta((p-1)/2, (p-1)/2) drawn as a ratio of chi-squares."""
    b = (-2.0 * kappa + math.sqrt(4.0 * kappa * kappa + (p - 1) ** 2)) / (p - 1)
    x0 = (1.0 - b) / (1.0 + b)
    c = kappa * x0 + (p - 1) * math.log(1.0 - x0 * x0)
    w = torch.empty(n, device=device, dtype=torch.float32)
    todo = torch.arange(n, device=device)
    while todo.numel() > 0:
        m = todo.numel()
        # Beta(a,a) with a=(p-1)/2: X/(X+Y), X,Y ~ chi2(p-1)/2 = sum of (p-1) squared normals / 2
        x = torch.randn(m, p - 1, generator=g, device=device).square_().sum(-1)
        y = torch.randn(m, p - 1, generator=g, device=device).square_().sum(-1)
        z = x / (x + y)
        u = torch.rand(m, generator=g, device=device)
        ww = (1.0 - (1.0 + b) * z) / (1.0 - (1.0 - b) * z)
        ok = kappa * ww + (p - 1) * torch.log(1.0 - x0 * ww) - c >= torch.log(u)
        w[todo[ok]] = ww[ok]
        todo = todo[~ok]
    return w


def vmf_around(mu: torch.Tensor, kappa: float, g: torch.Generator, chunk: int = 1 << 18) -> torch.Tensor:
    """One vMF(mu_i, kappa) sample per row of ``mu [n,p]`` (unit rows) -> unit rows fp32."""
    n, p = mu.shape
    out = torch.empty_like(mu, dtype=torch.float32)
    for s in range(0, n, chunk):
        m = mu[s:s + chunk].float()
        w = vmf_w(m.shape[0], p, kappa, g, mu.device)
        t = torch.randn(m.shape, generator=g, device=mu.device)
        t = t - (t * m).sum(-1, keepdim=True) * m
        t = t / t.norm(dim=-1, keepdim=True)
        out[s:s + chunk] = w[:, None] * m + torch.sqrt((1.0 - w * w).clamp(min=0.0))[:, None] * t
    return out


def unit_centres(n: int, p: int, g: torch.Generator, device) -> torch.Tensor:
    c = torch.randn(n, p, generator=g, device=device)
    return c / c.norm(dim=-1, keepdim=True)


@dataclass
class Workload:
    cfg: Config
    keys: torch.Tensor                  # [H,N,d]
    values: torch.Tensor                # [H,N,d]
    queries: torch.Tensor               # [H,G*S,d]
    k_local: Optional[torch.Tensor]     # [H,L,d]
    v_local: Optional[torch.Tensor]


def make_workload(cfg: Config, device="cpu", N: Optional[int] = None, S: Optional[int] = None,
                  H: Optional[int] = None) -> Workload:
    """Inputs of one configuration; ``N``, ``S``, ``H`` may be overridden to
    produce a reduced case with the same statistics."""
    N = cfg.N if N is None else N
    S = cfg.S if S is None else S
    H = cfg.H if H is None else H
    d, G = cfg.d, cfg.G
    g = _gen(device, cfg.seed)
    if cfg.n_clusters == 0:
        keys = torch.randn(H, N, d, generator=g, device=device)
        values = torch.randn(H, N, d, generator=g, device=device)
        queries = torch.randn(H, G * S, d, generator=g, device=device)
        kl = vl = None
    else:
        keys = torch.empty(H, N, d, device=device, dtype=cfg.dtype)
        queries = torch.empty(H, G * S, d, device=device, dtype=cfg.dtype)
        L = min(cfg.local, N) if cfg.local else 0
        kl = torch.empty(H, L, d, device=device, dtype=cfg.dtype) if L else None
        for h in range(H):
            centres = unit_centres(cfg.n_clusters, d, g, device)
            comp = torch.randint(0, cfg.n_clusters, (N,), generator=g, device=device)
            x = vmf_around(centres[comp], cfg.kappa, g)
            norms = torch.exp(0.25 * torch.randn(N, generator=g, device=device))
            keys[h] = (x * norms[:, None]).to(cfg.dtype)
            qc = torch.randint(0, cfg.n_clusters, (G * S,), generator=g, device=device)
            queries[h] = (vmf_around(centres[qc], cfg.kappa, g) * math.sqrt(d)).to(cfg.dtype)
            if L:
                lc = torch.randint(0, cfg.n_clusters, (L,), generator=g, device=device)
                ln = torch.exp(0.25 * torch.randn(L, generator=g, device=device))
                kl[h] = (vmf_around(centres[lc], cfg.kappa, g) * ln[:, None]).to(cfg.dtype)
        values = torch.randn(H, N, d, generator=g, device=device).to(cfg.dtype)
        vl = torch.randn(H, L, d, generator=g, device=device).to(cfg.dtype) if L else None
    return Workload(cfg, keys.to(cfg.dtype), values.to(cfg.dtype), queries.to(cfg.dtype), kl, vl)
