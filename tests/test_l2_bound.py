"""The inequality the matrix-pipe route of min_bmm's squared l2 rests on
(custom_matmul_kernels_amd/csrc/cmk_min.hip, l2_beta): with E the sequential
fmaf(x-y, x-y, c) sum and t = fmaf(-2, dot, |x|^2) built from an fp32 dot product,
|E - |y|^2 - t| <= (4K + 32) * 2^-24 * (|x|^2 + |y|^2).  Checked here, on the CPU,
against emulations of both an fp32 accumulator that rounds to nearest and one
that truncates, in two summation orders, on data chosen to make rounding bite
(offsets, mixed magnitudes, small integers, single terms)."""
import numpy as np
import pytest

U = 2.0 ** -24


def f32(a):
    return np.asarray(a, dtype=np.float64).astype(np.float32)


def trunc32(a):
    """float64 -> float32 rounding toward zero."""
    a = np.asarray(a, dtype=np.float64)
    r = a.astype(np.float32)
    over = np.abs(r.astype(np.float64)) > np.abs(a)
    return np.where(over, np.nextafter(r, np.float32(0)), r).astype(np.float32)


def exact_route(x, y):
    E = np.zeros((x.shape[0], y.shape[0]), np.float32)
    for k in range(x.shape[1]):
        d = (x[:, None, k] - y[None, :, k]).astype(np.float32)
        E = f32(d.astype(np.float64) * d.astype(np.float64) + E.astype(np.float64))   # one rounding, as fmaf
    return E


def dot_route(x, y, rnd, pairwise):
    prods = [rnd(x[:, None, k].astype(np.float64) * y[None, :, k].astype(np.float64)) for k in range(x.shape[1])]
    if pairwise:
        while len(prods) > 1:
            nxt = [rnd(prods[i].astype(np.float64) + prods[i + 1].astype(np.float64)) for i in range(0, len(prods) - 1, 2)]
            if len(prods) % 2:
                nxt.append(prods[-1])
            prods = nxt
        return prods[0]
    acc = np.zeros_like(prods[0])
    for p in prods:
        acc = rnd(acc.astype(np.float64) + p.astype(np.float64))
    return acc


@pytest.mark.parametrize("kind", ["normal", "offset", "scales", "integers"])
@pytest.mark.parametrize("K", [1, 2, 7, 64, 300])
def test_rounding_budget_of_the_l2_screen(K, kind):
    rng = np.random.default_rng(K * 7 + len(kind))
    x = rng.standard_normal((48, K))
    y = rng.standard_normal((40, K))
    if kind == "offset":
        x, y = x + 1000.0, y + 1000.0
    elif kind == "scales":
        x = x * 10.0 ** rng.integers(-6, 7, (48, 1))
        y = y * 10.0 ** rng.integers(-6, 7, (40, 1))
    elif kind == "integers":
        x = rng.integers(-3, 4, (48, K)).astype(float)
        y = rng.integers(-3, 4, (40, K)).astype(float)
    x, y = x.astype(np.float32), y.astype(np.float32)
    E = exact_route(x, y).astype(np.float64)
    nx32 = f32((x.astype(np.float64) ** 2).sum(1))            # summed in double, rounded once
    ny = (y.astype(np.float64) ** 2).sum(1)
    budget = (4 * K + 32) * U * (nx32.astype(np.float64)[:, None] + ny[None, :])
    for rnd in (f32, trunc32):
        for pairwise in (False, True):
            dot = dot_route(x, y, rnd, pairwise)
            t = f32(nx32.astype(np.float64)[:, None] - 2.0 * dot.astype(np.float64))   # fmaf(-2, dot, nx)
            err = np.abs(E - ny[None, :] - t.astype(np.float64))
            assert (err <= budget).all(), (rnd.__name__, pairwise, float((err / np.maximum(budget, 1e-300)).max()))
            # and it is not vacuous: the budget is within two orders of magnitude of what happens
            assert (err / np.maximum(budget, 1e-300)).max() > 1e-4 or kind == "integers"
