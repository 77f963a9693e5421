"""TEST INFRASTRUCTURE ONLY -- independent numpy definitions used to pin the restatement.

Nothing here shares structure with ``oracle/eager_restatement.py``: dominance is a per-row scan,
rank is the longest dominator chain (and, separately, Deb's bookkeeping from the NSGA-II paper
cited at src/evox/algorithms/mo/nsga2.py:18-20), sorting is numpy's stable argsort / lexsort.
The rules specific to the reference that these definitions encode were read from
src/evox/operators/selection/non_dominate.py:217-229 and :250-254 and are stated where used.
"""

import numpy as np


def dominates_matrix(f: np.ndarray) -> np.ndarray:
    """A[i, j] = all_k f[i,k] <= f[j,k] and any_k f[i,k] < f[j,k]; any NaN makes the pair False."""
    n = f.shape[0]
    out = np.zeros((n, n), dtype=bool)
    with np.errstate(invalid="ignore"):
        for i in range(n):
            out[i] = np.all(f[i] <= f, axis=1) & np.any(f[i] < f, axis=1)
    return out


def rank_longest_chain(f: np.ndarray) -> np.ndarray:
    """rank[j] = 0 without dominators, else 1 + max rank of its dominators.

    Rows are visited in lexicographic order, a linear extension of dominance (i dominates j
    implies tuple(f_i) < tuple(f_j)), so dominators are always finished first.  Rows holding a
    NaN compare False against everything: they are isolated and get rank 0."""
    n = f.shape[0]
    rank = np.zeros(n, dtype=np.int32)
    has_nan = np.isnan(f).any(axis=1)
    clean = np.flatnonzero(~has_nan)
    order = clean[np.lexsort(f[clean].T[::-1])] if clean.size else clean
    done = []
    for j in order:
        if done:
            prev = np.asarray(done)
            d = np.all(f[prev] <= f[j], axis=1) & np.any(f[prev] < f[j], axis=1)
            if d.any():
                rank[j] = rank[prev[d]].max() + 1
        done.append(j)
    return rank


def rank_deb(f: np.ndarray) -> np.ndarray:
    """Fast non-dominated sort with explicit dominated-sets and domination counters."""
    n = f.shape[0]
    dom = dominates_matrix(f)
    counter = dom.sum(axis=0).astype(np.int64)
    rank = np.zeros(n, dtype=np.int32)
    current = [j for j in range(n) if counter[j] == 0]
    level = 0
    while current:
        nxt = []
        for i in current:
            rank[i] = level
            for j in np.flatnonzero(dom[i]):
                counter[j] -= 1
                if counter[j] == 0:
                    nxt.append(j)
        current = nxt
        level += 1
    return rank


def crowding_brute(costs: np.ndarray, mask) -> np.ndarray:
    """NSGA-II crowding distance over the masked rows, float32 arithmetic, -inf elsewhere.

    Per objective k the masked rows are ordered by (cost, row index), NaN costs last
    (stable sort).  The first and last row of that order are boundary rows; a row that is a
    boundary row of ANY objective has distance +inf (non_dominate.py:226-227 write whole rows).
    Every other masked row receives (next - previous) / (last - first) per objective, summed
    over objectives in column order (non_dominate.py:225, 229)."""
    costs = np.asarray(costs, dtype=np.float32)
    n, m = costs.shape
    mask = np.ones(n, dtype=bool) if mask is None else np.asarray(mask, dtype=bool)
    out = np.full(n, -np.inf, dtype=np.float32)
    rows = np.flatnonzero(mask)
    nv = rows.size
    if nv == 0:
        return out
    part = np.zeros((n, m), dtype=np.float32)
    boundary = np.zeros(n, dtype=bool)
    with np.errstate(invalid="ignore", divide="ignore"):
        for k in range(m):
            srt = rows[np.argsort(costs[rows, k], kind="stable")]
            c = costs[srt, k]
            span = np.float32(c[-1] - c[0])
            boundary[srt[0]] = True
            boundary[srt[-1]] = True
            for p in range(1, nv - 1):
                part[srt[p], k] = np.float32(np.float32(c[p + 1] - c[p - 1]) / span)
        for r in rows:
            if boundary[r]:
                out[r] = np.inf
            else:
                acc = np.float32(0.0)
                for k in range(m):
                    acc = np.float32(acc + part[r, k])
                out[r] = acc
    return out


def selection_order_brute(rank: np.ndarray, dist: np.ndarray, topk: int) -> np.ndarray:
    """First ``topk`` of: rank ascending, then distance descending with NaN after every number,
    then row index ascending (non_dominate.py:253 with jit_fix_operator.py:246-252)."""
    n = rank.shape[0]
    with np.errstate(invalid="ignore"):
        neg = -np.asarray(dist, dtype=np.float32)
    return np.lexsort((np.arange(n), neg, rank))[:topk]


def selection_brute(f: np.ndarray, topk: int):
    """(order, rank, dist) of nd_environmental_selection from the independent definitions."""
    rank = rank_longest_chain(np.asarray(f, dtype=np.float32))
    worst = np.sort(rank, kind="stable")[topk - 1]
    dist = crowding_brute(f, rank == worst)
    return selection_order_brute(rank, dist, topk), rank, dist


def tournament_winners_brute(parents: np.ndarray, keys: np.ndarray) -> np.ndarray:
    """Winner of each tournament by an explicit comparison of tuples (last key first, NaN as +inf plus
    one, then position).  parents: (n_round, t) ints; keys: (candidates, nkeys) floats."""
    out = np.empty(parents.shape[0], dtype=np.int64)
    for r, row in enumerate(parents):
        def sort_key(pos_cand):
            pos, cand = pos_cand
            parts = []
            for k in range(keys.shape[1] - 1, -1, -1):
                v = float(keys[cand, k])
                parts.append((1, 0.0) if v != v else (0, v + 0.0))
            return (tuple(parts), pos)
        out[r] = min(enumerate(row), key=sort_key)[1]
    return out


def hv_contributions_brute(fit: np.ndarray, ref: np.ndarray, pop_size: int, uniform: np.ndarray) -> np.ndarray:
    """HypE's sampled hypervolume contributions by explicit loops, in float64: a sample inside the box
    [min fit, ref] that is covered by c >= 1 points gives each of them alpha[c - 1], with
    alpha[j] = prod_{l=1..j} (pop_size - l) / (n - l) / (j + 1); the sums are scaled by box volume / samples."""
    fit = np.asarray(fit, dtype=np.float32)
    n, m = fit.shape
    alpha = np.zeros(n)
    for j in range(n):
        a = 1.0
        for l in range(1, j + 1):
            a *= (pop_size - l) / (n - l)
        alpha[j] = a / (j + 1)
    f_min = fit.min(axis=0)
    box = (np.asarray(ref, dtype=np.float32) - f_min).astype(np.float32)
    samples = (np.asarray(uniform, dtype=np.float32) * box + f_min).astype(np.float32)
    out = np.zeros(n)
    for s in range(samples.shape[0]):
        covering = [i for i in range(n) if all(fit[i, k] <= samples[s, k] for k in range(m))]
        for i in covering:
            out[i] += alpha[len(covering) - 1]
    return out * float(np.prod(box.astype(np.float64))) / samples.shape[0]


def hv_covered_brute(points: np.ndarray, samples: np.ndarray) -> int:
    """Number of samples that some point exceeds strictly in every objective, by explicit loops."""
    count = 0
    for s in range(samples.shape[0]):
        hit = False
        for i in range(points.shape[0]):
            if all(samples[s, k] < points[i, k] for k in range(points.shape[1])):
                hit = True
                break
        count += int(hit)
    return count


def staircase_area_2d(points: np.ndarray) -> float:
    """Exact area of the union of the boxes [0, p] over 2-D points p >= 0 (a staircase), in float64:
    sweep the points by descending first coordinate and add the strips that raise the running height."""
    pts = sorted(((float(p[0]), float(p[1])) for p in points), reverse=True)
    area, height = 0.0, 0.0
    for a, b in pts:
        if b > height:
            area += a * (b - height)
            height = b
    return area
