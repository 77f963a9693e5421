"""Seeded synthetic populations for the five benchmark configurations.

Every generator draws on the CPU from ``torch.Generator("cpu").manual_seed(seed)`` so that a
CPU checker and the GPU path see identical bits; callers move the tensors to the device.

C1  N=200,    M=3, D=30,  topk=100     i.i.d. Uniform[0,1)
C2  N=2000,   M=2,        topk=1000    20 layered fronts on a 1/64 grid (exact ties, duplicate rows)
C3  N=20000,  M=3, D=100, topk=10000   i.i.d. Uniform[0,1)
C4  B=1024 x (N=512, M=3), topk=256    positive-orthant sphere direction x (1 + Exp(mean 0.1))
C5  N=200000, M=8,        topk=100000  positive-orthant sphere direction x (1 + Exp(mean 0.05))
"""

from typing import NamedTuple, Optional

import torch


class Workload(NamedTuple):
    name: str
    f: torch.Tensor  # (N, M) or (B, N, M) float32 fitness
    x: Optional[torch.Tensor]  # (N, D) float32 decision vectors, or None
    topk: int
    seed: int


def _gen(seed: int) -> torch.Generator:
    return torch.Generator("cpu").manual_seed(seed)


def uniform_population(n: int, m: int, d: int, seed: int):
    g = _gen(seed)
    f = torch.rand(n, m, generator=g, dtype=torch.float32)
    x = torch.rand(n, d, generator=g, dtype=torch.float32) if d > 0 else None
    return f, x


def layered_grid_population(layers: int, per_layer: int, seed: int, permute: bool = False):
    """Points on f1 + f2 = layer + 1 with f1 ~ U[0, layer+1] rounded to multiples of 1/64."""
    g = _gen(seed)
    rows = []
    for layer in range(layers):
        u = torch.rand(per_layer, generator=g, dtype=torch.float32)
        f1 = torch.round(u * float(layer + 1) * 64.0) / 64.0
        f2 = float(layer + 1) - f1
        rows.append(torch.stack([f1, f2], dim=1))
    f = torch.cat(rows, dim=0)
    if permute:
        f = f[torch.randperm(f.size(0), generator=g)]
    return f.contiguous()


def sphere_shell_population(shape, m: int, mean: float, seed: int):
    """|N(0,1)| direction normalised to the unit sphere, times radius 1 + Exponential(mean)."""
    g = _gen(seed)
    d = torch.randn(*shape, m, generator=g, dtype=torch.float32).abs()
    d = d / d.norm(dim=-1, keepdim=True)
    r = 1.0 + torch.empty(*shape, 1, dtype=torch.float32).exponential_(1.0 / mean, generator=g)
    return (d * r).contiguous()


def c1(seed: int = 0) -> Workload:
    f, x = uniform_population(200, 3, 30, seed)
    return Workload("C1", f, x, 100, seed)


def c2(seed: int = 0, permute: bool = False) -> Workload:
    f = layered_grid_population(20, 100, seed, permute)
    return Workload("C2p" if permute else "C2", f, None, 1000, seed)


def c3(seed: int = 0, n: int = 20000, d: int = 100) -> Workload:
    f, x = uniform_population(n, 3, d, seed)
    return Workload("C3", f, x, n // 2, seed)


def c4(seed: int = 1000, batch: int = 1024, n: int = 512) -> Workload:
    f = sphere_shell_population((batch, n), 3, 0.1, seed)
    return Workload("C4", f, None, n // 2, seed)


def c5(seed: int = 0, n: int = 200000) -> Workload:
    f = sphere_shell_population((n,), 8, 0.05, seed)
    return Workload("C5", f, None, n // 2, seed)
