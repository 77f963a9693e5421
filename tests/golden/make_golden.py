"""Writes the golden vectors under tests/golden/ by running the reference itself, once, in the
build container (the reference is not present anywhere else).

    PYTHONPATH=/root/reference/src python tests/golden/make_golden.py

What is stored is data only: seeded inputs and the reference's outputs for them
(`non_dominate_rank`, `crowding_distance`, `nd_environmental_selection` and the selected order,
recomputed with the reference's own `lexsort`).  The reason an import is used at all: the
reference holds no known-answer vectors for this path, and the degenerate corners of its crowding
distance (zero range, NaN/inf costs, one or two valid rows, signed zeros, NaN distances flowing
into the final ordering) are properties of its exact operation sequence, which no textbook fixes.
"""

import json
import os
import sys
import time

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

from evox.operators.selection import crowding_distance, nd_environmental_selection, non_dominate_rank  # noqa: E402
from evox.utils import lexsort  # noqa: E402

from evox_amd import workloads  # noqa: E402
from tests.cases import edge_cases  # noqa: E402


def reference_outputs(f: torch.Tensor, topk: int):
    rank = non_dominate_rank(f)
    worst = torch.topk(rank, topk, largest=False)[0][-1]
    dist = crowding_distance(f, rank == worst)
    order = lexsort([-dist, rank])[:topk]
    x = torch.arange(f.size(0), dtype=torch.float32)[:, None].repeat(1, 2)
    xs, fs, rs, ds = nd_environmental_selection(x, f, topk)
    assert torch.equal(xs[:, 0].long(), order) and torch.equal(rs, rank[order])
    assert np.array_equal(fs.numpy(), f[order].numpy(), equal_nan=True)
    assert np.array_equal(ds.numpy(), dist[order].numpy(), equal_nan=True)
    return rank.numpy(), dist.numpy(), order.numpy()


def masks_for(n: int, seed: int):
    g = torch.Generator("cpu").manual_seed(seed)
    out = [torch.ones(n, dtype=torch.bool), torch.rand(n, generator=g) < 0.5, torch.rand(n, generator=g) < 0.15]
    one = torch.zeros(n, dtype=torch.bool)
    one[n // 2] = True
    out.append(one)
    return out


def main():
    torch.set_num_threads(os.cpu_count())
    timings = {}

    # --- edge cases: rank, per-topk distance/order, crowding under assorted masks (and mask=None)
    edge = {}
    for name, f, ks in edge_cases():
        edge[f"{name}/f"] = f.numpy()
        edge[f"{name}/ks"] = np.asarray(ks, dtype=np.int64)
        for k in ks:
            rank, dist, order = reference_outputs(f, k)
            edge[f"{name}/rank"] = rank
            edge[f"{name}/dist@{k}"] = dist
            edge[f"{name}/order@{k}"] = order
        edge[f"{name}/cd_none"] = crowding_distance(f, None).numpy()
        for t, mask in enumerate(masks_for(f.size(0), 11)):
            edge[f"{name}/mask{t}"] = mask.numpy()
            edge[f"{name}/cd_mask{t}"] = crowding_distance(f, mask).numpy()
    np.savez_compressed(os.path.join(HERE, "edge_cases.npz"), **edge)

    # --- the benchmark configurations that the reference can run
    for w in (workloads.c1(), workloads.c2(), workloads.c2(permute=True), workloads.c3()):
        t0 = time.perf_counter()
        rank, dist, order = reference_outputs(w.f, w.topk)
        timings[w.name] = {"n": int(w.f.size(0)), "m": int(w.f.size(1)), "topk": w.topk, "seed": w.seed,
                           "fronts": int(rank.max()) + 1,
                           "seconds_two_passes": round(time.perf_counter() - t0, 3)}
        # inputs are re-derived from the seed by evox_amd.workloads; a checksum guards the generator
        np.savez_compressed(os.path.join(HERE, f"{w.name.lower()}.npz"), rank=rank.astype(np.int32), dist=dist,
                            order=order.astype(np.int32), f_sum=np.float64(w.f.double().sum().item()),
                            f_head=w.f[:4].numpy())
        t0 = time.perf_counter()
        x = w.x if w.x is not None else w.f
        nd_environmental_selection(x, w.f, w.topk)
        timings[w.name]["nd_environmental_selection_seconds"] = round(time.perf_counter() - t0, 3)

    # --- first 8 populations of the batched configuration, each run un-batched
    w = workloads.c4()
    ranks, dists, orders = [], [], []
    for b in range(8):
        rank, dist, order = reference_outputs(w.f[b], w.topk)
        ranks.append(rank)
        dists.append(dist)
        orders.append(order)
    np.savez_compressed(os.path.join(HERE, "c4_first8.npz"), rank=np.stack(ranks).astype(np.int32),
                        dist=np.stack(dists), order=np.stack(orders).astype(np.int32),
                        f_sum=np.float64(w.f[:8].double().sum().item()))

    timings["host"] = {"cores": os.cpu_count(), "torch": torch.__version__, "threads": torch.get_num_threads()}
    with open(os.path.join(HERE, "reference_timings.json"), "w") as fh:
        json.dump(timings, fh, indent=1)
    print(json.dumps(timings, indent=1))


if __name__ == "__main__":
    main()
