"""The CPU oracle against the golden vectors that the reference itself produced."""

import numpy as np
import pytest
import torch

from oracle import eager_restatement as er
from tests import golden_io
from tests.cases import as_np, edge_cases

EDGE = edge_cases()
IDS = [c[0] for c in EDGE]


def same_float(a, b):
    a, b = as_np(a), as_np(b)
    return a.shape == b.shape and np.array_equal(a, b, equal_nan=True)


@pytest.fixture(scope="module")
def edge_golden():
    return golden_io.load("edge_cases.npz")


@pytest.mark.parametrize("name,f,ks", EDGE, ids=IDS)
def test_edge_cases(edge_golden, name, f, ks):
    g = edge_golden
    assert same_float(f, g[f"{name}/f"])
    x = torch.arange(f.size(0), dtype=torch.float32)[:, None]
    assert np.array_equal(as_np(er.ranks_by_peeling(f)), g[f"{name}/rank"])
    for k in ks:
        _, rank, dist, order = er.environmental_selection(x, f, k, return_all=True)
        assert np.array_equal(as_np(rank), g[f"{name}/rank"])
        assert same_float(dist, g[f"{name}/dist@{k}"])
        assert np.array_equal(as_np(order), g[f"{name}/order@{k}"])
    assert same_float(er.crowding(f, None), g[f"{name}/cd_none"])
    for t in range(4):
        mask = torch.from_numpy(g[f"{name}/mask{t}"])
        assert same_float(er.crowding(f, mask), g[f"{name}/cd_mask{t}"])


@pytest.mark.parametrize("name", ["C1", "C2", "C2p"])
def test_configs(name):
    w, g = golden_io.config(name)
    x = w.x if w.x is not None else w.f
    _, rank, dist, order = er.environmental_selection(x, w.f, w.topk, return_all=True)
    assert np.array_equal(as_np(rank), g["rank"])
    assert same_float(dist, g["dist"])
    assert np.array_equal(as_np(order), g["order"])


def test_c4_first8():
    w, g = golden_io.c4_first8()
    batched = er.ranks_by_peeling_batched(w.f[:8])
    assert np.array_equal(as_np(batched), g["rank"])
    for b in range(8):
        _, rank, dist, order = er.environmental_selection(w.f[b], w.f[b], w.topk, return_all=True)
        assert np.array_equal(as_np(rank), g["rank"][b])
        assert same_float(dist, g["dist"][b])
        assert np.array_equal(as_np(order), g["order"][b])
