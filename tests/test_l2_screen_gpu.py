"""Squared-l2 min_bmm through the matrix pipe: the screening route must return,
bit for bit, what the vector route and the C oracle return (values and
indices), also where |x|^2 + |y|^2 - 2 x.y cancels, where points are
duplicated, and where the input is not finite."""
import numpy as np
import pytest
import torch

import custom_matmul_kernels_amd.minbmm as minbmm
from custom_matmul_kernels_amd import MinBMMCUDA, _lib
from oracle import oracle as O
from _cases import seeded

pytestmark = pytest.mark.gpu


def say(*a):
    print("[l2 screen]", *a, flush=True)


def place(A, B, mode, dev):
    Ad, Bd = A.to(dev), B.to(dev)
    if mode[0] == "t":
        Ad = Ad.transpose(1, 2).contiguous().transpose(1, 2)
    if mode[1] == "t":
        Bd = Bd.transpose(1, 2).contiguous().transpose(1, 2)
    return Ad, Bd


def both_routes(monkeypatch, Ad, Bd, dim):
    op = MinBMMCUDA(distance="l2")
    monkeypatch.setattr(minbmm, "L2_SCREEN_MIN_WORK", 1 << 62)
    vv, vi = op(Ad, Bd, dim=dim)
    monkeypatch.setattr(minbmm, "L2_SCREEN_MIN_WORK", 0)
    sv, si = op(Ad, Bd, dim=dim)
    torch.cuda.synchronize()
    return (vv.cpu(), vi.cpu()), (sv.cpu(), si.cpu())


def same(got, want):
    gv, gi = got
    wv, wi = want
    # bit patterns, so that NaN and signed zeros count too
    assert torch.equal(gv.view(torch.int32), wv.view(torch.int32)), (gv != wv).nonzero()[:5]
    assert torch.equal(gi, wi), ((gi != wi).nonzero()[:5], gi[gi != wi][:5], wi[gi != wi][:5])


SHAPES = [(1, 5, 7, 3), (2, 130, 140, 33), (1, 300, 260, 64), (1, 64, 1100, 40), (1, 1000, 1500, 100),
          (3, 257, 129, 1), (1, 2048, 2048, 16), (2, 700, 900, 401)]


def test_the_screening_workspace_is_the_larger_one():
    lib = _lib.load()
    for (L, M, N, K) in SHAPES + [(1, 16384, 16384, 256)]:
        for dim in (1, 2):
            small = lib.cmk_workspace_bytes(_lib.OP_MIN_BMM, L, M, N, K, dim)
            big = lib.cmk_workspace_bytes(_lib.OP_MIN_BMM_L2, L, M, N, K, dim)
            assert big > small
    assert lib.cmk_workspace_bytes(_lib.OP_MIN_BMM_L2, 1, 64, 64, 0, 1) == 0   # K = 0: vector route only


@pytest.mark.parametrize("dim", [1, 2])
@pytest.mark.parametrize("mode", ["nn", "tt", "nt", "tn"])
@pytest.mark.parametrize("shape", SHAPES)
def test_screened_l2_equals_oracle_and_vector_route(device, monkeypatch, shape, mode, dim):
    say("random", shape, mode, dim)
    L, M, N, K = shape
    A, B = seeded(L, M, N, K, seed=21)
    Ad, Bd = place(A, B, mode, device)
    vec, scr = both_routes(monkeypatch, Ad, Bd, dim)
    same(scr, vec)
    cv, ci = O.c_min_bmm(A.numpy(), B.numpy(), dim, 1)
    same(scr, (torch.from_numpy(cv), torch.from_numpy(ci).long()))


@pytest.mark.parametrize("dim", [1, 2])
def test_screened_l2_under_cancellation(device, monkeypatch, dim):
    """Points far from the origin and close to each other: the expanded form loses
    every significant digit, all rows go to the exact route (more than the
    one-by-one limit, so the vector route over the whole problem)."""
    say("cancellation", dim)
    g = torch.Generator().manual_seed(5)
    A = 1000.0 + 1e-2 * torch.randn(1, 900, 24, generator=g)
    B = 1000.0 + 1e-2 * torch.randn(1, 24, 700, generator=g)
    vec, scr = both_routes(monkeypatch, A.to(device), B.to(device), dim)
    same(scr, vec)
    cv, ci = O.c_min_bmm(A.numpy(), B.numpy(), dim, 1)
    same(scr, (torch.from_numpy(cv), torch.from_numpy(ci).long()))


def test_screened_l2_mild_cancellation_takes_the_row_route(device, monkeypatch):
    """An offset that makes some but not all rows undecidable (a few hundred at
    most): those are recomputed one by one."""
    say("mild cancellation")
    g = torch.Generator().manual_seed(6)
    A = 3.0 + torch.randn(1, 3000, 32, generator=g)
    B = 3.0 + torch.randn(1, 32, 2000, generator=g)
    for dim in (1, 2):
        vec, scr = both_routes(monkeypatch, A.to(device), B.to(device), dim)
        same(scr, vec)


@pytest.mark.parametrize("K", [48, 450])     # either kernel that recomputes single rows
@pytest.mark.parametrize("dim", [1, 2])
def test_screened_l2_with_duplicated_points(device, monkeypatch, dim, K):
    """Exact ties: three copies of some reduced-axis points, and kept-axis points
    that coincide with them (distance 0 three times).  The lowest index wins."""
    say("duplicates", dim, K)
    A, B = seeded(1, 1200, 900, K, seed=22)
    X, Y = (A[0], B[0].t()) if dim == 1 else (B[0].t(), A[0])    # X = reduced axis, rows
    X, Y = X.clone(), Y.clone()
    X[500] = X[17]; X[1] = X[17]; X[800] = X[640]; X[700] = X[640]
    for j, src in enumerate([17, 640, 17, 640, 1]):
        Y[11 * j + 3] = X[src]
    if dim == 1:
        A2, B2 = X[None], Y.t().contiguous()[None]
    else:
        A2, B2 = Y[None], X.t().contiguous()[None]
    vec, scr = both_routes(monkeypatch, A2.to(device), B2.to(device), dim)
    same(scr, vec)
    assert scr[1][0, 3].item() == 1 and scr[1][0, 14].item() == 640 and scr[0][0, 3].item() == 0.0
    cv, ci = O.c_min_bmm(A2.numpy(), B2.numpy(), dim, 1)
    same(scr, (torch.from_numpy(cv), torch.from_numpy(ci).long()))


def test_screened_l2_all_points_equal(device, monkeypatch):
    """Every distance is the same: everything is a tie, index 0 everywhere."""
    say("all equal")
    A = torch.full((2, 300, 20), 0.5)
    B = torch.full((2, 20, 400), 0.25)
    for dim in (1, 2):
        vec, scr = both_routes(monkeypatch, A.to(device), B.to(device), dim)
        same(scr, vec)
        assert int(scr[1].max()) == 0


@pytest.mark.parametrize("dim", [1, 2])
def test_screened_l2_with_non_finite_input(device, monkeypatch, dim):
    say("non-finite", dim)
    A, B = seeded(1, 400, 500, 24, seed=23)
    A, B = A.clone(), B.clone()
    A[0, 5, 3] = float("nan"); A[0, 77, 0] = float("inf"); A[0, 200, 7] = 3e38
    B[0, 2, 9] = float("-inf"); B[0, 11, 300] = float("nan"); B[0, 4, 123] = -3e38
    vec, scr = both_routes(monkeypatch, A.to(device), B.to(device), dim)
    same(scr, vec)
    cv, ci = O.c_min_bmm(A.numpy(), B.numpy(), dim, 1)
    same(scr, (torch.from_numpy(cv), torch.from_numpy(ci).long()))


def test_screened_l2_tiny_magnitudes(device, monkeypatch):
    """Squares that underflow: the screening steps aside."""
    say("tiny")
    A, B = seeded(1, 300, 200, 16, seed=24)
    vec, scr = both_routes(monkeypatch, (A * 1e-21).to(device), (B * 1e-21).to(device), 2)
    same(scr, vec)


def test_screened_l2_full_size_equals_vector_route(device, monkeypatch):
    """A[1,16384,256] x B[1,256,16384], every output of both routes; 48 rows
    against the C oracle."""
    say("16384 x 16384 x 256")
    A, B = seeded(1, 16384, 16384, 256, seed=3)
    vec, scr = both_routes(monkeypatch, A.to(device), B.to(device), 2)
    same(scr, vec)
    rows = np.linspace(0, 16383, 48).astype(np.int64)
    cv, ci = O.c_min_bmm(A.numpy()[:, rows], B.numpy(), 2, 1)
    same((scr[0][:, rows], scr[1][:, rows]), (torch.from_numpy(cv), torch.from_numpy(ci).long()))


def test_default_threshold_uses_the_screening_for_large_problems(device):
    """Without any patching: large problem, results equal the oracle's on a sample."""
    say("default route")
    A, B = seeded(1, 4096, 8192, 64, seed=4)
    assert 4096 * 8192 * 64 >= minbmm.L2_SCREEN_MIN_WORK
    v, i = MinBMMCUDA(distance="l2")(A.to(device), B.to(device), dim=1)
    cols = np.linspace(0, 8191, 32).astype(np.int64)
    cv, ci = O.c_min_bmm(A.numpy(), np.ascontiguousarray(B.numpy()[:, :, cols]), 1, 1)
    same((v.cpu()[:, cols], i.cpu()[:, cols]), (torch.from_numpy(cv), torch.from_numpy(ci).long()))


def _sweep_case(rng):
    L = int(rng.choice([1, 1, 2, 3]))
    M = int(rng.integers(1, 700))
    N = int(rng.integers(1, 700))
    K = int(rng.choice([1, 2, 7, 16, 31, 64, 100, 257, 420]))
    kind = rng.choice(["normal", "clustered", "integers", "offset", "scales", "sparse"])
    g = torch.Generator().manual_seed(int(rng.integers(1 << 30)))
    if kind == "normal":
        A, B = torch.randn(L, M, K, generator=g), torch.randn(L, K, N, generator=g)
    elif kind == "clustered":
        # a handful of centres, points are centres plus noise at the rounding level: near ties everywhere
        C = torch.randn(L, 5, K, generator=g)
        ia = torch.randint(0, 5, (L, M), generator=g)
        ib = torch.randint(0, 5, (L, N), generator=g)
        A = torch.gather(C, 1, ia[..., None].expand(L, M, K)) + 1e-6 * torch.randn(L, M, K, generator=g)
        B = (torch.gather(C, 1, ib[..., None].expand(L, N, K)) + 1e-6 * torch.randn(L, N, K, generator=g)).transpose(1, 2)
    elif kind == "integers":
        A = torch.randint(-3, 4, (L, M, K), generator=g).float()
        B = torch.randint(-3, 4, (L, K, N), generator=g).float()
    elif kind == "offset":
        off = float(rng.choice([10.0, 300.0, 1e4]))
        A = off + torch.randn(L, M, K, generator=g)
        B = off + torch.randn(L, K, N, generator=g)
    elif kind == "scales":
        A = torch.randn(L, M, K, generator=g) * 10.0 ** torch.randint(-6, 7, (L, M, 1), generator=g).float()
        B = torch.randn(L, K, N, generator=g) * 10.0 ** torch.randint(-6, 7, (L, 1, N), generator=g).float()
    else:
        A = torch.randn(L, M, K, generator=g) * (torch.rand(L, M, K, generator=g) < 0.1)
        B = torch.randn(L, K, N, generator=g) * (torch.rand(L, K, N, generator=g) < 0.1)
    return kind, A.contiguous(), B.contiguous()


def test_screened_l2_seeded_sweep_over_shapes_and_data(device, monkeypatch):
    """Sixty seeded cases over shapes, layouts, axes and kinds of data that stress
    the screen in different ways (near ties, exact ties, cancellation, mixed
    magnitudes, many zeros): both routes return the same bits, and the oracle
    agrees on every fourth case."""
    rng = np.random.default_rng(2024)
    for case in range(60):
        kind, A, B = _sweep_case(rng)
        mode = str(rng.choice(["nn", "tt", "nt", "tn"]))
        dim = int(rng.choice([1, 2]))
        say("sweep", case, kind, tuple(A.shape), tuple(B.shape), mode, dim)
        Ad, Bd = place(A, B, mode, device)
        vec, scr = both_routes(monkeypatch, Ad, Bd, dim)
        same(scr, vec)
        if case % 4 == 0:
            cv, ci = O.c_min_bmm(A.numpy(), B.numpy(), dim, 1)
            same(scr, (torch.from_numpy(cv), torch.from_numpy(ci).long()))


def test_screened_l2_on_strided_views_and_a_shared_operand(device, monkeypatch):
    """Operands that are windows of wider tensors (leading dimension beyond the
    row length, consumed in place) and an operand shared by all batches (batch
    stride 0)."""
    say("views")
    g = torch.Generator().manual_seed(31)
    wideA = torch.randn(3, 260, 96, generator=g)
    wideB = torch.randn(3, 80, 400, generator=g)
    A, B = wideA[:, 4:250, 8:72], wideB[:, 16:80, 40:360]          # [3,246,64] and [3,64,320]
    Ad, Bd = wideA.to(device)[:, 4:250, 8:72], wideB.to(device)[:, 16:80, 40:360]
    for dim in (1, 2):
        vec, scr = both_routes(monkeypatch, Ad, Bd, dim)
        same(scr, vec)
        cv, ci = O.c_min_bmm(A.contiguous().numpy(), B.contiguous().numpy(), dim, 1)
        same(scr, (torch.from_numpy(cv), torch.from_numpy(ci).long()))
    shared = wideB[:1, 16:80, 40:360]
    Bs = shared.to(device).expand(3, -1, -1)
    for dim in (1, 2):
        vec, scr = both_routes(monkeypatch, Ad, Bs, dim)
        same(scr, vec)
        cv, ci = O.c_min_bmm(A.contiguous().numpy(), shared.expand(3, -1, -1).contiguous().numpy(), dim, 1)
        same(scr, (torch.from_numpy(cv), torch.from_numpy(ci).long()))


def test_screened_l2_replays_in_a_hip_graph(device, monkeypatch):
    """The screening route is kernel launches only (its counter is cleared by its
    first kernel): captured once, every replay on new inputs - one of them with
    duplicated points, so that rows are queued - equals the eager vector route."""
    say("graph replay")
    monkeypatch.setattr(minbmm, "L2_SCREEN_MIN_WORK", 0)
    L, M, N, K = 2, 300, 520, 72
    gen = torch.Generator().manual_seed(41)
    A = torch.randn(L, M, K, generator=gen).to(device)
    B = torch.randn(L, K, N, generator=gen).to(device)
    op = MinBMMCUDA(distance="l2")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            op(A, B, dim=2)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = op(A, B, dim=2)
    for step in range(3):
        a = torch.randn(L, M, K, generator=gen)
        b = torch.randn(L, K, N, generator=gen)
        if step == 1:
            b[:, :, 100] = b[:, :, 7]
            b[:, :, 300] = b[:, :, 7]
            a[:, 5] = b[:, :, 7]
        A.copy_(a)
        B.copy_(b)
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in captured]
        monkeypatch.setattr(minbmm, "L2_SCREEN_MIN_WORK", 1 << 62)
        want = op(A, B, dim=2)
        monkeypatch.setattr(minbmm, "L2_SCREEN_MIN_WORK", 0)
        torch.cuda.synchronize()
        same((got[0].cpu(), got[1].cpu()), (want[0].cpu(), want[1].cpu()))
        if step == 1:
            assert int(got[1][0, 5]) == 7
