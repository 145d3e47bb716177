"""Edge cases of the HIP path, through the operator classes and the C ABI:
products that are all equal (every tie rule and the more-than-256-ties branch
of the selection), empty and short reduced axes, non-finite operands, the
masked product in all four layouts, a fixed-seed randomized sweep over every
operator, and the full-size configurations checked over all of their output."""
import os
import random

import numpy as np
import pytest
import torch

from custom_matmul_kernels_amd import (BMMCUDA, MBMMCUDA, MinBMMCUDA, TopkBMMCUDA, BitonicSort,
                                       derive_masks)
from oracle import oracle as O
from _cases import seeded
from test_parity_gpu import MODES, place, random_masks, say

pytestmark = pytest.mark.gpu


# ------------------------------------------------ all products equal --------
# (l, m, n, k, dim): reduced axis of 1024 (one chunk), 5000 (several chunks),
# 300 (fewer than one chunk), and a long axis that is split and merged
EQUAL_SHAPES = [(1, 70, 1024, 8, 2), (2, 33, 5000, 4, 2), (1, 40, 300, 16, 2),
                (1, 1024, 70, 8, 1), (1, 40000, 48, 4, 1), (1, 200000, 8, 2, 1)]


@pytest.mark.parametrize("const", [0.0, 1.0, -2.5])
@pytest.mark.parametrize("shape", EQUAL_SHAPES)
def test_all_equal_products_resolve_to_the_lowest_indices(device, shape, const):
    """A = const, B = 1: every product of a row equals const * k.  top-k must
    return that value 128 times with indices 0..127 in ascending order (more
    than 256 candidates share the threshold key, in every chunk and in the
    merge of a split axis), min must return index 0."""
    say("all equal", shape, const)
    L, M, N, K, dim = shape
    A = torch.full((L, M, K), const, device=device)
    B = torch.ones(L, K, N, device=device)
    kept = N if dim == 1 else M
    red = M if dim == 1 else N
    kk = min(128, red)
    v, i = TopkBMMCUDA()(A, B, k=128, dim=dim)
    assert v.shape == (L, kept, 128)
    assert (v[..., :kk] == const * K).all()
    assert torch.equal(i[..., :kk], torch.arange(kk, device=device).expand(L, kept, kk))
    if kk < 128:
        assert torch.isinf(v[..., kk:]).all() and (v[..., kk:] < 0).all() and (i[..., kk:] == -1).all()
    mv, mi = MinBMMCUDA()(A, B, dim=dim)
    assert (mv == const * K).all() and (mi == 0).all()


def test_ties_at_the_threshold_keep_the_lowest_indices_across_chunks(device):
    """Two distinct values only: the larger one fills fewer than 128 slots, the
    rest are ties at the threshold spread over several chunks; the lowest
    indices must win whatever chunk they sit in."""
    L, M, N, K = 1, 64, 4096, 1
    gen = torch.Generator().manual_seed(17)
    B = torch.ones(L, K, N)
    hot = torch.randperm(N, generator=gen)[:50]
    B[0, 0, hot] = 2.0
    A = torch.ones(L, M, K)
    v, i = TopkBMMCUDA()(A.to(device), B.to(device), k=128, dim=2)
    want_i = torch.cat([hot.sort().values, torch.tensor([j for j in range(N) if j not in set(hot.tolist())][:78])])
    want_v = torch.cat([torch.full((50,), 2.0), torch.full((78,), 1.0)])
    assert torch.equal(v.cpu(), want_v.expand(L, M, 128))
    assert torch.equal(i.cpu(), want_i.expand(L, M, 128))
    # the same along the split axis (dim=1: B^T A^T), long enough to be cut and merged
    At = torch.ones(1, 60000, 1)
    hot2 = torch.randperm(60000, generator=gen)[:50]
    At[0, hot2, 0] = 2.0
    Bt = torch.ones(1, 1, 24)
    v, i = TopkBMMCUDA()(At.to(device), Bt.to(device), k=128, dim=1)
    rest = np.setdiff1d(np.arange(60000), hot2.numpy())[:78]
    want_i = torch.cat([hot2.sort().values, torch.from_numpy(rest)])
    assert torch.equal(v.cpu(), want_v.expand(1, 24, 128))
    assert torch.equal(i.cpu(), want_i.expand(1, 24, 128))
    # and for the 1-D top-k
    x = torch.ones(300000)
    hot3 = torch.randperm(300000, generator=gen)[:50]
    x[hot3] = 2.0
    v, i = BitonicSort()(x.to(device), k=128)
    rest = np.setdiff1d(np.arange(300000), hot3.numpy())[:78]
    assert torch.equal(v.cpu(), want_v)
    assert torch.equal(i.cpu(), torch.cat([hot3.sort().values, torch.from_numpy(rest)]))


def test_long_reduced_axis_with_exact_products_matches_a_stable_sort(device):
    """Forty chunks of candidates per row, products that are small integers
    (exact in fp32, full of ties): the result must be the first 128 of a stable
    descending sort, i.e. equal values by ascending index.  The patterns make
    late chunks bring no newcomer (descending ramp), only newcomers (ascending
    ramp), a few (random digits) and ties with the list's smallest entry."""
    N = 40000
    gen = torch.Generator().manual_seed(23)
    ramps = {
        "digits": torch.randint(0, 10, (N,), generator=gen).float(),
        "ascending": torch.arange(N).float(),
        "descending": torch.arange(N, 0, -1).float(),
        "steps": (torch.arange(N) // 300).float(),
        "sawtooth": (torch.arange(N) % 1500).float(),
        "rare": (torch.rand(N, generator=gen) < 0.002).float() * torch.randint(1, 4, (N,), generator=gen).float(),
    }
    scale = torch.tensor([1.0, -1.0, 2.0, -3.0, 0.0]).repeat(14)[:68]      # 68 rows: two strips, the second ragged
    for name, b in ramps.items():
        say("long axis", name)
        A = scale.view(1, -1, 1).clone()
        B = b.view(1, 1, N).clone()
        C = torch.bmm(A, B)
        want = C.sort(dim=2, descending=True, stable=True)
        v, i = TopkBMMCUDA()(A.to(device), B.to(device), k=128, dim=2)
        assert torch.equal(v.cpu(), want.values[..., :128]), name
        assert torch.equal(i.cpu(), want.indices[..., :128]), name
        # the same products with the long axis first (dim=1), cut into splits and merged
        v, i = TopkBMMCUDA()(B.transpose(1, 2).contiguous().to(device), A.transpose(1, 2).contiguous().to(device),
                             k=128, dim=1)
        assert torch.equal(v.cpu(), want.values[..., :128]), name + " dim=1"
        assert torch.equal(i.cpu(), want.indices[..., :128]), name + " dim=1"


# ------------------------------------------------ empty / short axes --------
def test_topk_over_an_empty_or_short_reduced_axis(device):
    op = TopkBMMCUDA()
    # reduced axis of extent 0: nothing to select, every slot is -inf / -1
    for (A, B, dim, shape) in [(torch.zeros(2, 5, 3), torch.zeros(2, 3, 0), 2, (2, 5, 7)),
                               (torch.zeros(1, 0, 3), torch.zeros(1, 3, 9), 1, (1, 9, 7))]:
        v, i = op(A.to(device), B.to(device), k=7, dim=dim)
        assert v.shape == shape and i.shape == shape
        assert torch.isinf(v).all() and (v < 0).all() and (i == -1).all()
    # fewer candidates than k
    A, B = seeded(2, 9, 5, 12, seed=31)
    for dim, red in ((2, 5), (1, 9)):
        v, i = op(A.to(device), B.to(device), k=128, dim=dim)
        O.check_topk(v, i, A, B, 128, dim)
        assert (i[..., red:] == -1).all()
    # K = 0: every product is 0, indices 0..k-1
    v, i = op(torch.zeros(1, 4, 0, device=device), torch.zeros(1, 0, 300, device=device), k=16, dim=2)
    assert (v == 0).all() and torch.equal(i.cpu(), torch.arange(16).expand(1, 4, 16))
    mv, mi = MinBMMCUDA()(torch.zeros(1, 4, 0, device=device), torch.zeros(1, 0, 300, device=device), dim=2)
    assert (mv == 0).all() and (mi == 0).all()


# ------------------------------------------------ non-finite operands -------
def test_non_finite_products_min(device):
    """min_bmm compares with a strict '<' starting from +inf, like the reference
    kernel (kernels/minbmm.cu:37-51): NaN products never win, -inf wins at its
    first index, and a row whose products are all NaN or +inf reports +inf at
    index 0."""
    A, B = seeded(1, 300, 700, 32, seed=41)
    A[0, 3] = float("nan")                     # row 3: every product NaN
    A[0, 4] = 0.0
    A[0, 4, 0] = float("inf")                  # row 4: products are +-inf or NaN (inf * 0 never: B has no zeros)
    B[0, 0].abs_()                             # make B[0, 0, :] positive: row 4 is all +inf
    A[0, 5] = 0.0
    A[0, 5, 0] = float("-inf")                 # row 5: all -inf
    A[0, 6] = 0.0
    A[0, 6, 1] = 1.0                           # row 6 = B[0, 1, :]
    B[0, 1, 200] = float("nan")                # one NaN product in column 200 of every row whose A[.,1] != 0
    B[0, 1, 333] = float("-inf")
    C = torch.bmm(A, B)[0]
    want_v, want_i = torch.nan_to_num(C, nan=float("inf"), posinf=float("inf"), neginf=float("-inf")).min(1)
    for mode in ("nn", "tt"):
        Ad, Bd = place(A, B, mode, device)
        v, i = MinBMMCUDA()(Ad, Bd, dim=2)
        v, i = v.cpu()[0], i.cpu()[0]
        assert v[3] == float("inf") and i[3] == 0
        assert v[4] == float("inf") and i[4] == 0
        assert v[5] == float("-inf") and i[5] == 0
        assert v[6] == float("-inf") and i[6] == 333
        # every other row: the minimum over its products that are not NaN (column 200
        # is NaN everywhere, column 333 is -inf or +inf by the sign of A[., 1])
        O.check_values(v, want_v, 32, "minimum over the products that are not NaN")
        neg = want_v == float("-inf")
        neg[5] = False
        assert (i[neg] == 333).all()


def test_nan_products_do_not_hide_their_neighbours_in_min(device):
    """A NaN product at any position of a tile - the first one included - loses
    every comparison and nothing else: the minimum over the other products is
    still found.  NaNs are planted in whole columns of B (every row of the
    product has them) at positions that are first, last and in between for the
    lanes of the kernel's tiles."""
    A, B = seeded(1, 260, 1000, 16, seed=44)
    cols = [0, 4, 31, 32, 64, 127, 128, 132, 255, 256, 511, 512, 640, 999]
    B[0, :, cols] = float("nan")
    C = torch.bmm(A, B)[0]
    want_v, want_i = torch.nan_to_num(C, nan=float("inf")).min(1)
    for mode in MODES:
        Ad, Bd = place(A, B, mode, device)
        v, i = MinBMMCUDA()(Ad, Bd, dim=2)
        O.check_values(v.cpu()[0], want_v, 16, "minimum over the products that are not NaN")
        assert torch.equal(i.cpu()[0], want_i)
    # the same along dim=1 (NaN rows of A)
    A2, B2 = seeded(1, 1000, 260, 16, seed=45)
    A2[0, cols, :] = float("nan")
    C2 = torch.bmm(A2, B2)[0]
    want_v, want_i = torch.nan_to_num(C2, nan=float("inf")).min(0)
    v, i = MinBMMCUDA()(A2.to(device), B2.to(device), dim=1)
    O.check_values(v.cpu()[0], want_v, 16, "minimum over the products that are not NaN, dim=1")
    assert torch.equal(i.cpu()[0], want_i)


def test_non_finite_products_topk(device):
    """top-k orders by the fp32 bit pattern: +inf above every finite value, -inf
    below, NaN with a clear sign bit above +inf (torch.topk also ranks NaN
    largest), NaN with the sign bit set below -inf."""
    A, B = seeded(1, 200, 1500, 16, seed=42)
    A[0, 4] = 0.0
    A[0, 4, 0] = float("inf")
    B[0, 0].abs_()                             # row 4: all +inf -> indices 0..127
    A[0, 5] = 0.0
    A[0, 5, 0] = float("-inf")                 # row 5: all -inf -> indices 0..127
    v, i = TopkBMMCUDA()(A.to(device), B.to(device), k=128, dim=2)
    v, i = v.cpu()[0], i.cpu()[0]
    assert (v[4] == float("inf")).all() and torch.equal(i[4], torch.arange(128))
    assert (v[5] == float("-inf")).all() and torch.equal(i[5], torch.arange(128))
    A, B = seeded(1, 200, 1500, 16, seed=42)
    A[0, 6] = 0.0
    A[0, 6, 1] = 1.0                           # row 6 = B[0, 1, :]
    B[0, 1, 700] = float("inf")
    B[0, 1, 701] = float("-inf")
    v, i = TopkBMMCUDA()(A.to(device), B.to(device), k=128, dim=2)
    v, i = v.cpu()[0], i.cpu()[0]
    assert v[6, 0] == float("inf") and i[6, 0] == 700 and (i[6] != 701).all()
    row6 = B[0, 1].clone()
    row6[700] = float("-inf")
    assert torch.equal(v[6, 1:], row6.topk(127).values)
    # every other row has one +-inf product at 700 and one at 701: the +inf one comes first
    rv, ri = torch.bmm(A, B)[0].topk(128, dim=-1)
    assert torch.equal(torch.isinf(v), torch.isinf(rv)) and torch.equal(i[:, 0], ri[:, 0])
    # a NaN bit pattern with a clear sign bit ranks first, one with the sign bit set is never selected
    x = torch.randn(5000, generator=torch.Generator().manual_seed(2))
    xi = x.view(torch.int32)
    xi[1234] = 0x7FC00000
    xi[4321] = -0x400000                        # 0xFFC00000
    v1, i1 = BitonicSort()(x.to(device), k=128)
    assert torch.isnan(v1[0]) and i1[0] == 1234 and (i1 != 4321).all()
    y = x.clone()
    y[1234] = float("-inf")
    y[4321] = float("-inf")
    assert torch.equal(v1.cpu()[1:], y.topk(127).values)


def test_non_finite_products_mbmm(device):
    """The element mask is a 0/1 multiplier (reference kernels/mbmm.cu:127-128):
    a non-finite product under a zero element byte gives NaN, while positions
    dropped by the thread mask or the block mask are exact zeros and their
    operands are not even read for skipped tiles."""
    L, M, N, K = 1, 256, 256, 8
    A, B = seeded(L, M, N, K, seed=43)
    A[0, 10, 0] = float("inf")                  # row 10 of C is +-inf everywhere
    A[0, 200] = float("nan")                    # row 200 of C is NaN everywhere
    fm = torch.ones(M, N, dtype=torch.bool)
    fm[10, 5] = False                           # dropped by the element mask only: inf * 0 = NaN
    fm[8:16, 64:72] = False                     # a whole 8x8 micro-tile: thread mask 0 -> exact zeros
    fm[128:, :128] = False                      # a whole 128x128 tile: block mask 0 -> skipped, zeros
    bm, tm, em = derive_masks(fm.to(device))
    C = MBMMCUDA(share_mask=True)(A.to(device), B.to(device), bm, tm, em).cpu()[0]
    assert torch.isnan(C[10, 5])
    assert (C[8:16, 64:72] == 0).all()
    assert (C[128:, :128] == 0).all()           # includes row 200, whose operands are NaN
    assert torch.isnan(C[200, 128:]).all()
    assert torch.isinf(C[10, 6:64]).all()
    want = torch.from_numpy(O.c_mbmm(A.numpy(), B.numpy(), bm.cpu().numpy(), tm.cpu().numpy(),
                                     em.cpu().numpy(), True))[0]
    finite = torch.isfinite(want)
    assert torch.equal(torch.isnan(C), torch.isnan(want)) and torch.equal(C[~finite & ~torch.isnan(want)],
                                                                           want[~finite & ~torch.isnan(want)])
    O.check_values(C[finite], want[finite], K, "finite part")


# ------------------------------------------------ mbmm in all layouts -------
@pytest.mark.parametrize("share", [False, True])
@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("shape", [(2, 130, 140, 8), (1, 256, 384, 40), (3, 77, 200, 33), (1, 512, 128, 64)])
def test_mbmm_layouts_match_oracle(device, shape, mode, share):
    """`mode` as the reference documents it (mbmm.py:163-170): "t" for A means A
    is passed as [l, k, m], "t" for B that B is passed as [l, n, k]."""
    say("mbmm layout", shape, mode, share)
    L, M, N, K = shape
    A, B = seeded(L, M, N, K, seed=51)
    fm = random_masks(L, M, N, seed=52, share=share)
    bm, tm, em = derive_masks(fm.to(device))
    Ain = A.to(device) if mode[0] == "n" else A.transpose(1, 2).contiguous().to(device)
    Bin = B.to(device) if mode[1] == "n" else B.transpose(1, 2).contiguous().to(device)
    C = MBMMCUDA(share_mask=share)(Ain, Bin, bm, tm, em, mode=mode)
    assert C.shape == (L, M, N)
    full = fm[None].expand(L, -1, -1) if share else fm
    O.check_values(C.cpu(), O.ref_mbmm(A, B, full), K, "mbmm " + mode)
    assert (C.cpu()[~full] == 0).all()
    cbm, ctm, cem = O.ref_derive_masks(fm)
    O.check_values(C.cpu(), torch.from_numpy(O.c_mbmm(A.numpy(), B.numpy(), cbm.numpy(), ctm.numpy(),
                                                      cem.numpy(), share)), K, "mbmm vs C")
    # a strided view in mode "nn" is consumed in place and gives the same bits
    Ad, Bd = place(A, B, mode, device)
    assert torch.equal(MBMMCUDA(share_mask=share)(Ad, Bd, bm, tm, em), C)
    # 2-D operands
    if L == 1:
        masks2 = (bm, tm, em) if share else (bm[0], tm[0], em[0])
        C2 = MBMMCUDA(share_mask=share)(Ain[0], Bin[0], *masks2, mode=mode)
        assert C2.shape == (M, N) and torch.equal(C2, C[0])


# ------------------------------------------------ randomized sweep ----------
def _dims(rng):
    L = rng.choice([1, 1, 2, 3, 40])
    M = rng.choice([1, 7, 64, 100, 128, 129, 255, 256, 300, 513, 640, 1500])
    N = rng.choice([1, 5, 64, 96, 128, 130, 256, 384, 500, 1024, 1100, 2500, 9000])
    K = rng.choice([1, 3, 8, 31, 32, 33, 36, 64, 65, 96, 100, 128, 160, 200, 257])
    if L == 40 and M * N * K > 3e7:
        L = 4
    return L, M, N, K


def test_randomized_sweep_fixed_seed(device):
    """120 cases drawn from one fixed seed: every operator, layout, axis and
    distance on ragged shapes, against the oracle; stops at the first failure and
    names it.  CMK_SWEEP_CASES / CMK_SWEEP_SEED run a longer or different sweep by hand."""
    rng = random.Random(int(os.environ.get("CMK_SWEEP_SEED", "20240607")))
    for it in range(int(os.environ.get("CMK_SWEEP_CASES", "120"))):
        L, M, N, K = _dims(rng)
        mode = rng.choice(MODES)
        dim = rng.choice([1, 2])
        op = rng.choice(["bmm", "min", "topk", "mbmm", "minl2", "minl1", "topkl1", "topkl2"])
        if op in ("minl2", "minl1", "topkl1", "topkl2") and L * M * N * K > 1e8:
            K = 33                                 # the vector-unit paths are slower; keep the case small
        say("sweep", it, op, (L, M, N, K), mode, dim)
        g = torch.Generator().manual_seed(it)
        A = torch.randn(L, M, K, generator=g)
        B = torch.randn(L, K, N, generator=g)
        Ad, Bd = place(A, B, mode, device)
        if op == "bmm":
            O.check_values(BMMCUDA()(Ad, Bd).cpu(), O.ref_bmm(A, B), K, "bmm")
        elif op == "mbmm":
            fm = torch.rand(L, M, N, generator=g) < 0.4
            fm &= (torch.rand(L, (M + 127) // 128, (N + 127) // 128, generator=g) < 0.6) \
                .repeat_interleave(128, 1).repeat_interleave(128, 2)[:, :M, :N]
            bm, tm, em = derive_masks(fm.to(device))
            C = MBMMCUDA()(Ad, Bd, bm, tm, em).cpu()
            O.check_values(C, O.ref_mbmm(A, B, fm), K, "mbmm")
            assert (C[~fm] == 0).all()
        elif op == "min":
            v, i = MinBMMCUDA()(Ad, Bd, dim=dim)
            O.check_min(v, i, A, B, dim)
        elif op == "topk":
            k = rng.choice([1, 17, 128])
            v, i = TopkBMMCUDA()(Ad, Bd, k=k, dim=dim)
            O.check_topk(v, i, A, B, k, dim)
        elif op in ("minl2", "minl1"):
            dist = op[3:]
            v, i = MinBMMCUDA(distance=dist)(Ad, Bd, dim=dim)
            cv, ci = O.c_min_bmm(A.numpy(), B.numpy(), dim, 1 if dist == "l2" else 2)
            assert torch.equal(v.cpu(), torch.from_numpy(cv)), "%s values" % op
            assert torch.equal(i.cpu(), torch.from_numpy(ci).long()), "%s indices" % op
        else:
            dist = op[4:]
            v, i = TopkBMMCUDA(distance=dist)(Ad, Bd, k=128, dim=dim)
            cv, ci = O.c_topk_bmm(A.numpy(), B.numpy(), 128, dim, 1 if dist == "l2" else 2)
            kk = min(128, M if dim == 1 else N)
            assert torch.equal(v.cpu()[..., :kk], torch.from_numpy(cv)[..., :kk]), "%s values" % op


# ------------------------------------------------ full-size configurations --
def test_bmm_config_2_all_batches(device):
    """A[128,1024,128] @ B[128,128,1024], U(-1,1): every batch against torch.bmm on the CPU."""
    say("bmm config 2, all batches")
    A, B = seeded(128, 1024, 1024, 128, seed=0, dist="uniform")
    C = BMMCUDA()(A.to(device), B.to(device)).cpu()
    for b0 in range(0, 128, 16):
        O.check_values(C[b0:b0 + 16], torch.bmm(A[b0:b0 + 16], B[b0:b0 + 16]), 128, "bmm batches %d.." % b0)


def test_mbmm_config_3_all_batches(device):
    """A[128,1024,64] @ B[128,64,1024] under tril AND tile-Bernoulli(0.5): every
    batch against torch.bmm + masked_fill on the CPU, in all four layouts."""
    say("mbmm config 3, all batches")
    L, M, N, K = 128, 1024, 1024, 64
    A, B = seeded(L, M, N, K, seed=0)
    fm = random_masks(L, M, N, seed=1, share=False)
    bm, tm, em = derive_masks(fm.to(device))
    want = O.ref_mbmm(A, B, fm)
    first = None
    for mode in MODES:
        Ad, Bd = place(A, B, mode, device)
        C = MBMMCUDA(share_mask=False)(Ad, Bd, bm, tm, em).cpu()
        for b0 in range(0, L, 32):
            O.check_values(C[b0:b0 + 32], want[b0:b0 + 32], K, "mbmm %s batches %d.." % (mode, b0))
        assert (C[~fm] == 0).all()
        first = C if first is None else first
        assert torch.equal(C, first)               # the layouts only change how operands are fetched


def test_topk_config_5_every_row(device):
    """Full config 5: for all 2^20 rows, every reported value is the product at
    its index and no unselected product exceeds the smallest selected value
    (checked against torch.bmm on the GPU, an independent implementation, in
    slabs of rows), besides order and uniqueness."""
    say("topk config 5, every row")
    gen = torch.Generator().manual_seed(0)
    A = torch.randn(1, 1048576, 256, generator=gen)
    B = torch.randn(1, 256, 1024, generator=gen)
    Ad, Bd = A.to(device), B.to(device)
    v, i = TopkBMMCUDA()(Ad, Bd, k=128, dim=-1)
    tol = O.atol_for(256)
    step = 32768
    for r0 in range(0, 1048576, step):
        C = torch.bmm(Ad[:, r0:r0 + step], Bd)
        vs, is_ = v[:, r0:r0 + step], i[:, r0:r0 + step]
        at = torch.gather(C, 2, is_)
        assert ((at - vs).abs() <= tol + O.RTOL * at.abs()).all(), "value at index, rows %d.." % r0
        # nothing outside the selection beats the smallest selected value
        C.scatter_(2, is_, float("-inf"))
        assert (C.max(-1).values <= vs[..., -1] + tol).all(), "an unselected product is larger, rows %d.." % r0
        assert (vs[..., :-1] >= vs[..., 1:]).all()
    # a sample of rows in float64 on the CPU
    rows = torch.arange(0, 1048576, 8209)
    at = O.gather_products(A[:, rows], B, 2, i[:, rows].cpu())
    O.check_values(v[:, rows].cpu(), at, 256, "value at index (float64)")
