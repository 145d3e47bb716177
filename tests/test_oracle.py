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
    from custom_matmul_kernels_amd.masks import derive_masks
    A, B = golden_inputs(g, name)
    mask = torch.from_numpy(g[name + "_mask"])
    bm, tm, em = derive_masks(mask)
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
