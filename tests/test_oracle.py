"""Pins the CPU oracle (oracle/) before anything is compared with it:
  * exact-integer golden fixtures computed with int64 numpy only;
  * float64 closed forms and brute-force Python loops on tiny shapes;
  * the sorting network against sorting by other means (0/1 inputs, random
    permutations, np.sort);
  * the two oracle layers (C restatement, PyTorch-CPU semantics) against
    each other.
The reference ships no golden vectors for this path, so these checks are what
anchors the oracle."""
import itertools

import numpy as np
import pytest
import torch

from oracle import oracle as O
from _cases import INT_CASES, golden, golden_inputs, golden_topk_values, seeded


@pytest.fixture(scope="module")
def g():
    return golden()


@pytest.mark.parametrize("name", INT_CASES)
def test_c_bmm_matches_integer_golden(g, name):
    A, B = golden_inputs(g, name)
    C = O.c_bmm(A.numpy(), B.numpy())
    assert np.array_equal(C, g[name + "_C"].astype(np.float32))
    assert torch.equal(O.ref_bmm(A, B), torch.from_numpy(g[name + "_C"].astype(np.float32)))


@pytest.mark.parametrize("name", INT_CASES)
@pytest.mark.parametrize("dim", [1, 2])
def test_min_matches_integer_golden(g, name, dim):
    A, B = golden_inputs(g, name)
    v, i = O.c_min_bmm(A.numpy(), B.numpy(), dim)
    assert np.array_equal(v, g["%s_min%d_val" % (name, dim)].astype(np.float32))
    assert np.array_equal(i, g["%s_min%d_idx" % (name, dim)].astype(np.int64))  # first index on ties
    rv, ri = O.ref_min_bmm(A, B, dim)
    assert np.array_equal(rv.numpy(), v)
    assert np.array_equal(ri.numpy(), i)


@pytest.mark.parametrize("name", INT_CASES)
@pytest.mark.parametrize("dim", [1, 2])
def test_topk_values_match_integer_golden(g, name, dim):
    A, B = golden_inputs(g, name)
    want = golden_topk_values(g, name, dim)
    v, i = O.c_topk_bmm(A.numpy(), B.numpy(), 128, dim)
    assert torch.equal(torch.from_numpy(v), want)
    # indices: every finite value sits at its index (ties make the choice free)
    C = torch.from_numpy(g[name + "_C"].astype(np.float32))
    Cr = C if dim == 2 else C.transpose(1, 2)
    it = torch.from_numpy(i)
    ok = it >= 0
    assert torch.equal(ok, torch.isfinite(want))
    assert torch.equal(torch.gather(Cr, 2, it.clamp(min=0))[ok], want[ok])
    red = Cr.shape[2]
    rv, _ = O.ref_topk_bmm(A, B, min(128, red), dim)
    assert torch.equal(rv, want[..., :min(128, red)])


@pytest.mark.parametrize("name", INT_CASES)
def test_mbmm_matches_integer_golden(g, name):
    A, B = golden_inputs(g, name)
    mask = torch.from_numpy(g[name + "_mask"])
    bm, tm, em = O.ref_derive_masks(mask)
    C = O.c_mbmm(A.numpy(), B.numpy(), bm.numpy(), tm.numpy(), em.numpy(), True)
    want = g[name + "_Cmasked"].astype(np.float32)
    assert np.array_equal(C, want)
    full = mask[None].expand(A.shape[0], -1, -1)
    assert np.array_equal(O.ref_mbmm(A, B, full).numpy(), want)


def test_bmm_bruteforce_and_float64():
    A, B = seeded(2, 9, 11, 13, seed=3)
    C = O.c_bmm(A.numpy(), B.numpy())
    for l, m, n in itertools.product(range(2), range(9), range(11)):
        acc = np.float32(0)
        for k in range(13):  # one fp32 accumulator, k ascending, fused multiply-add
            acc = np.float32(np.float64(A[l, m, k].item()) * np.float64(B[l, k, n].item()) + np.float64(acc))
        assert C[l, m, n] == acc
    exact = torch.bmm(A.double(), B.double()).numpy()
    assert np.abs(C - exact).max() < 1e-5


def test_c_layer_agrees_with_torch_layer_on_floats():
    A, B = seeded(2, 150, 300, 40, seed=5)
    C = torch.from_numpy(O.c_bmm(A.numpy(), B.numpy()))
    O.check_values(C, O.ref_bmm(A, B), 40)
    for dim in (1, 2):
        v, i = O.c_min_bmm(A.numpy(), B.numpy(), dim)
        assert O.check_min(torch.from_numpy(v), torch.from_numpy(i), A, B, dim) <= 2
        v, i = O.c_topk_bmm(A.numpy(), B.numpy(), 128, dim)
        assert O.check_topk(torch.from_numpy(v), torch.from_numpy(i), A, B, 128, dim) <= 8


@pytest.mark.parametrize("code,p", [(1, 2), (2, 1)])
def test_distances_against_closed_forms(code, p):
    """(a-b)^2 and |a-b| accumulation (reference kernels/bmm_helpers.cu:28-35,
    46-52).  The reference's notebooks never run these, so they are pinned by
    what the mathematics fixes: integer inputs computed exactly in int64, a
    brute-force loop in the reference's order of operations, torch.cdist in
    float64, and special cases (identical vectors, a single k)."""
    rng = np.random.default_rng(5)
    # exact: small integers, every partial sum is an integer below 2^24
    Ai = rng.integers(-9, 10, size=(2, 17, 13))
    Bi = rng.integers(-9, 10, size=(2, 13, 21))
    diff = Ai[:, :, :, None] - Bi[:, None, :, :]                     # [l, m, k, n]
    D = (diff ** 2 if p == 2 else np.abs(diff)).sum(2)               # int64 [l, m, n]
    for dim in (1, 2):
        v, i = O.c_min_bmm(Ai.astype(np.float32), Bi.astype(np.float32), dim, code)
        assert np.array_equal(v, D.min(dim).astype(np.float32))
        assert np.array_equal(i, D.argmin(dim))                      # first minimum = lowest index
        tv, ti = O.c_topk_bmm(Ai.astype(np.float32), Bi.astype(np.float32), 128, dim, code)
        red = D.shape[dim]
        want = -np.sort(-D, axis=dim).swapaxes(dim, 2)[..., :red]    # largest first
        assert np.array_equal(tv[..., :red], want.astype(np.float32))
        assert np.isneginf(tv[..., red:]).all()
        picked = np.take_along_axis(D.swapaxes(dim, 2), ti[..., :red], axis=2)
        assert np.array_equal(picked, want)                          # indices point at their values
    # brute force in the reference's order: one accumulator, k ascending
    A, B = seeded(1, 6, 5, 11, seed=9)
    v, i = O.c_min_bmm(A.numpy(), B.numpy(), 2, code)
    for m in range(6):
        best = None
        for n in range(5):
            acc = np.float32(0)
            for k in range(11):
                d = np.float32(A[0, m, k].item()) - np.float32(B[0, k, n].item())
                if p == 2:   # fmaf(d, d, acc): one rounding
                    acc = np.float32(np.float64(d) * np.float64(d) + np.float64(acc))
                else:
                    acc = np.float32(acc + np.abs(d))
            if best is None or acc < best[0]:
                best = (acc, n)
        assert v[0, m] == best[0] and i[0, m] == best[1]
    # float64 closed form on random floats
    A, B = seeded(2, 40, 50, 33, seed=10)
    cd = torch.cdist(A.double(), B.double().transpose(1, 2), p=p)
    cd = cd ** 2 if p == 2 else cd
    for dim in (1, 2):
        v, i = O.c_min_bmm(A.numpy(), B.numpy(), dim, code)
        assert np.allclose(v, cd.min(dim)[0].numpy(), rtol=1e-5, atol=1e-4)
        tv, ti = O.c_topk_bmm(A.numpy(), B.numpy(), 128, dim, code)
        red = cd.shape[dim]
        assert np.allclose(tv[..., :red], cd.topk(red, dim)[0].transpose(dim, 2).numpy()[..., :red], rtol=1e-5, atol=1e-4)
    # identical vectors are at distance exactly 0 and win the minimum
    A = torch.randn(1, 4, 7)
    B = A[0].t().contiguous()[None]                                  # column j of B = row j of A
    v, i = O.c_min_bmm(A.numpy(), B.numpy(), 2, code)
    assert (v == 0).all() and np.array_equal(i[0], np.arange(4))


def test_mask_precedence():
    """block mask beats thread mask beats element mask; the element mask byte
    multiplies (reference kernels/mbmm.cu:127-128, 251-255, 360-363)."""
    A, B = seeded(1, 130, 140, 8, seed=7)
    C = O.c_bmm(A.numpy(), B.numpy())[0]
    bm = np.ones((1, 2, 2), np.uint8)
    tm = np.ones((1, 17, 18), np.uint8)
    em = np.ones((1, 130, 140), np.uint8)
    bm[0, 1, 0] = 0          # rows 128.., cols 0..127 skipped
    tm[0, 0, 1] = 0          # rows 0..7, cols 8..15 never accumulated
    em[0, 20, 30] = 0
    em[0, 21, 31] = 3        # the byte multiplies
    out = O.c_mbmm(A.numpy(), B.numpy(), bm, tm, em, False)[0]
    want = C.copy()
    want[128:, :128] = 0
    want[0:8, 8:16] = 0
    want[20, 30] = 0
    want[21, 31] *= 3
    assert np.array_equal(out, want)


def test_sorting_network_zero_one_and_random():
    rng = np.random.default_rng(11)
    idx = np.arange(128)
    # 0/1 inputs: a comparator network that sorts all of them sorts everything;
    # 2^128 is out of reach, so take every count of ones in several shuffles
    for ones in range(129):
        base = np.array([0.0] * (128 - ones) + [1.0] * ones, np.float32)
        for _ in range(4):
            p = rng.permutation(128)
            v, _i = O.c_bitonic_sort_128(base[p], idx)
            assert np.array_equal(v, base)
    for _ in range(200):
        x = rng.standard_normal(128).astype(np.float32)
        v, i = O.c_bitonic_sort_128(x, idx)
        assert np.array_equal(v, np.sort(x))
        assert np.array_equal(x[i], v)           # payload follows its key
        assert np.array_equal(np.sort(i), idx)   # distinct keys: a permutation


def test_topk_1d_against_sort():
    rng = np.random.default_rng(12)
    for n in (1, 5, 128, 129, 1000, 5000):
        x = rng.standard_normal(n).astype(np.float32)
        v, i = O.c_topk_1d(x, 128)
        want = np.sort(x)[::-1][:128]
        assert np.array_equal(v[:min(n, 128)], want)
        assert np.array_equal(x[i[:min(n, 128)]], want)
        if n < 128:
            assert np.all(np.isneginf(v[n:])) and np.all(i[n:] == -1)


def test_comparators_reject_wrong_answers():
    A, B = seeded(1, 40, 300, 16, seed=2)
    v, i = O.ref_min_bmm(A, B, 2)
    O.check_min(v, i, A, B, 2)
    bad = i.clone()
    bad[0, 3] = (bad[0, 3] + 1) % 300
    with pytest.raises(AssertionError):
        O.check_min(v, bad, A, B, 2)
    with pytest.raises(AssertionError):
        O.check_min(v + 1.0, i, A, B, 2)
    tv, ti = O.ref_topk_bmm(A, B, 128, 2)
    O.check_topk(tv, ti, A, B, 128, 2)
    swapped = ti.clone()
    swapped[0, 0, 0], swapped[0, 0, 100] = ti[0, 0, 100], ti[0, 0, 0]
    with pytest.raises(AssertionError):
        O.check_topk(tv, swapped, A, B, 128, 2)
    dup = ti.clone()
    dup[0, 1, 5] = dup[0, 1, 4]
    with pytest.raises(AssertionError):
        O.check_topk(tv, dup, A, B, 128, 2)
