"""Helpers shared by the test modules: golden-fixture access and seeded inputs."""
import os

import numpy as np
import torch

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "int_cases.npz")
INT_CASES = ("tiny", "ragged", "wide", "tall")
INT32_MIN = np.iinfo(np.int32).min


def golden():
    return np.load(GOLDEN)


def golden_inputs(g, name):
    A = torch.from_numpy(g[name + "_A"].astype(np.float32))
    B = torch.from_numpy(g[name + "_B"].astype(np.float32))
    return A, B


def golden_topk_values(g, name, dim):
    v = g["%s_top%d_val" % (name, dim)].astype(np.float64)
    v[g["%s_top%d_val" % (name, dim)] == INT32_MIN] = -np.inf
    return torch.from_numpy(v.astype(np.float32))


def seeded(L, M, N, K, seed=0, dist="normal"):
    """A drawn before B from one CPU generator, as the measurement plan fixes."""
    gen = torch.Generator().manual_seed(seed)
    if dist == "normal":
        A = torch.randn(L, M, K, generator=gen)
        B = torch.randn(L, K, N, generator=gen)
    else:
        A = torch.rand(L, M, K, generator=gen) * 2 - 1
        B = torch.rand(L, K, N, generator=gen) * 2 - 1
    return A, B
