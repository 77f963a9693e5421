"""Drop-in replacement for ``cal_hv`` of the reference's HypE (src/evox/algorithms/mo/hype.py:12-39): the
Monte-Carlo estimate of every point's hypervolume contribution, with which HypE breaks ties inside the
last admitted front (hype.py:140-143).
"""

import torch

from . import ops


def hv_alpha(n: int, pop_size, device) -> torch.Tensor:
    """The weights alpha[j] of a sample covered by j + 1 points (hype.py:14-24)."""
    idx = torch.arange(1, n, device=device)
    alpha = torch.cumprod(torch.cat([torch.ones(1, device=device), (pop_size - idx) / (n - idx)]), dim=0) / torch.arange(
        1, n + 1, device=device)
    return torch.nan_to_num(alpha)


def cal_hv(fit: torch.Tensor, ref: torch.Tensor, pop_size, n_sample: int) -> torch.Tensor:
    """Same contract as the reference's ``cal_hv``: ``fit`` (N, M), ``ref`` (M,) reference point, ``pop_size``
    the number of points to be kept, ``n_sample`` uniform samples drawn with ``torch.rand`` on ``fit.device``
    between the per-objective minimum and ``ref`` (a seeded generator gives the reference's samples)."""
    n, m = fit.size()
    alpha = hv_alpha(n, pop_size, fit.device)
    f_min = torch.min(fit, dim=0).values
    samples = torch.rand(n_sample, m, device=fit.device) * (ref - f_min) + f_min
    scale = torch.prod(ref - f_min) / n_sample
    return ops.hv_contributions(fit, samples, alpha.float(), 1.0) * scale
