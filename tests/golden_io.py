"""Loaders for the committed golden vectors (outputs of the reference on seeded inputs)."""

import os

import numpy as np

from evox_amd import workloads

GOLDEN_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(name):
    return np.load(os.path.join(GOLDEN_DIR, name), allow_pickle=False)


def config(name):
    """(workload, golden dict) for C1, C2, C2p or C3; verifies that the seeded generator still
    produces the population the vectors were computed on."""
    w = {"C1": workloads.c1, "C2": workloads.c2, "C2p": lambda: workloads.c2(permute=True), "C3": workloads.c3}[name]()
    g = load(name.lower() + ".npz")
    assert float(w.f.double().sum()) == float(g["f_sum"]) and np.array_equal(w.f[:4].numpy(), g["f_head"])
    return w, g


def c4_first8():
    w = workloads.c4()
    g = load("c4_first8.npz")
    assert float(w.f[:8].double().sum()) == float(g["f_sum"])
    return w, g
