"""Drop-in replacement for the reference's Monte-Carlo hypervolume metric (src/evox/metrics/hv.py:4-20)."""

import torch

from .. import ops


def hv(objs: torch.Tensor, ref: torch.Tensor, num_sample: int = 100000) -> torch.Tensor:
    """Same contract as the reference's ``hv``: ``objs`` (n_points, n_objs), ``ref`` (n_objs,) reference point,
    ``num_sample`` uniform samples in the bounding box of ``|objs - ref|``; returns the estimated hypervolume
    (0-d tensor on ``objs.device``).  The samples are drawn with ``torch.rand(num_sample, n_objs)`` on the
    default device exactly as the reference does (hv.py:17), so a seeded default generator gives the
    reference's samples; the sample-against-points test (hv.py:18) runs in the HIP kernel, without the
    (num_sample, n_points, n_objs) temporaries of the reference."""
    points = torch.abs(objs - ref)
    bound = torch.max(points, dim=0).values
    max_vol = torch.prod(bound)
    samples = torch.rand(num_sample, points.size(1)).to(bound.device) * bound
    covered = ops.hv_covered_count(points, samples)
    return covered / num_sample * max_vol
