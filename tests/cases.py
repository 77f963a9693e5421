"""Small seeded populations shared by the oracle tests, the golden-vector script and the GPU
parity tests.  Each case is (name, f float32 (N, M), topk list)."""

import numpy as np
import torch

NAN = float("nan")
INF = float("inf")


def _rand(n, m, seed):
    return torch.rand(n, m, generator=torch.Generator("cpu").manual_seed(seed), dtype=torch.float32)


def _randn(n, m, seed):
    return torch.randn(n, m, generator=torch.Generator("cpu").manual_seed(seed), dtype=torch.float32)


def _grid(n, m, levels, seed):
    g = torch.Generator("cpu").manual_seed(seed)
    return torch.randint(0, levels, (n, m), generator=g).to(torch.float32) / float(levels)


def edge_cases():
    """Tiny and degenerate inputs: N in {1,2,3,5,12,...}, M in {1,2,3,8}, duplicates, NaN/inf rows,
    constant objectives, signed zeros."""
    t = torch.tensor
    cases = [
        ("single", t([[0.5, 0.25, 0.75]]), [1]),
        ("pair_dominated", t([[0.0, 0.0], [1.0, 1.0]]), [1, 2]),
        ("pair_tradeoff", t([[0.0, 1.0], [1.0, 0.0]]), [1, 2]),
        ("pair_equal", t([[0.5, 0.5], [0.5, 0.5]]), [1, 2]),
        ("three_m1", t([[2.0], [1.0], [2.0]]), [1, 2, 3]),
        ("chain5", t([[float(i), float(i), float(i)] for i in range(5)]), [1, 3, 5]),
        ("chain5_rev", t([[float(4 - i), float(4 - i)] for i in range(5)]), [2, 5]),
        ("all_equal5", torch.full((5, 3), 0.25), [1, 3, 5]),
        ("front5_m2", t([[0.0, 4.0], [1.0, 3.0], [2.0, 2.0], [3.0, 1.0], [4.0, 0.0]]), [1, 2, 3, 4, 5]),
        ("front5_m2_shuffled", t([[2.0, 2.0], [4.0, 0.0], [0.0, 4.0], [3.0, 1.0], [1.0, 3.0]]), [3, 5]),
        ("const_objective", t([[0.0, 1.0, 5.0], [1.0, 0.0, 5.0], [0.5, 0.5, 5.0], [0.25, 0.75, 5.0],
                               [0.75, 0.25, 5.0]]), [2, 4, 5]),
        ("const_all_but_one", t([[1.0, 3.0], [1.0, 1.0], [1.0, 2.0], [1.0, 2.0], [1.0, 0.5]]), [1, 2, 3, 5]),
        ("signed_zero", t([[0.0, 1.0], [-0.0, 1.0], [0.0, -0.0], [-0.0, 0.0], [1.0, -0.0], [1.0, 0.0]]), [2, 3, 6]),
        ("nan_row", t([[0.1, 0.9], [NAN, 0.0], [0.5, 0.5], [0.9, 0.1], [0.6, 0.6], [0.0, NAN]]), [2, 3, 4, 6]),
        ("all_nan", torch.full((4, 2), NAN), [1, 2, 4]),
        ("inf_rows", t([[INF, 0.0], [0.0, INF], [-INF, 5.0], [1.0, 1.0], [INF, INF], [2.0, 0.5], [-INF, -INF]]),
         [1, 3, 5, 7]),
        ("dups_m2", t([[1.0, 2.0], [1.0, 2.0], [2.0, 1.0], [2.0, 1.0], [1.5, 1.5], [1.5, 1.5], [3.0, 3.0],
                       [3.0, 3.0]]), [1, 3, 4, 6, 8]),
        ("rand12_m3", _randn(12, 3, 12), [1, 6, 12]),
        ("rand12_m8", _randn(12, 8, 128), [6, 12]),
        ("rand64_m2", _rand(64, 2, 64), [32, 64]),
        ("rand65_m3", _rand(65, 3, 65), [1, 33, 65]),
        ("rand130_m4", _rand(130, 4, 130), [65, 129]),
        ("grid100_m2", _grid(100, 2, 8, 100), [10, 50, 99]),
        ("grid100_m3", _grid(100, 3, 4, 101), [37, 50]),
        ("grid200_m1", _grid(200, 1, 16, 102), [100, 200]),
        ("grid300_m5", _grid(300, 5, 3, 103), [150]),
        ("rand257_m3", _rand(257, 3, 257), [128, 200]),
    ]
    return [(name, f.contiguous(), ks) for name, f, ks in cases]


def as_np(t):
    return t.detach().cpu().numpy() if isinstance(t, torch.Tensor) else np.asarray(t)
