"""Parity of the HIP path with the CPU oracle, through the operator classes and
therefore through the C ABI of libcmk.so.  Values: rtol 1e-4, atol
1e-3*sqrt(K).  Indices: exact, except where the competing products are closer
than that tolerance.  Integer-valued cases must match bit for bit."""
import numpy as np
import pytest
import torch

from custom_matmul_kernels_amd import (BMMCUDA, MBMMCUDA, MinBMMCUDA, TopkBMMCUDA, BitonicSort,
                                       derive_masks)
from oracle import oracle as O
from _cases import INT_CASES, golden, golden_inputs, golden_topk_values, seeded

pytestmark = pytest.mark.gpu

MODES = ("nn", "nt", "tn", "tt")


def place(A, B, mode, dev):
    """Device copies of A [l,m,k] / B [l,k,n] stored in the given layout; the
    returned tensors have the logical shapes, only their strides differ."""
    Ad = A.to(dev) if mode[0] == "n" else A.transpose(1, 2).contiguous().to(dev).transpose(1, 2)
    Bd = B.to(dev) if mode[1] == "n" else B.transpose(1, 2).contiguous().to(dev).transpose(1, 2)
    return Ad, Bd


def say(*a):
    print(*a, flush=True)


# ---------------------------------------------------------------- bmm --------
# the last three have enough 128x128 tiles for the large-tile kernel (ragged edges included),
# the others take the 64x64-tile kernel
BMM_SHAPES = [(1, 1, 1, 1), (2, 37, 300, 19), (3, 129, 257, 33), (1, 128, 128, 64),
              (2, 200, 136, 70), (1, 256, 384, 100), (5, 64, 64, 32),
              (70, 300, 520, 33), (13, 1000, 1100, 40), (1, 4000, 3100, 24)]


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("shape", BMM_SHAPES)
def test_bmm_matches_oracle(device, shape, mode):
    say("bmm", shape, mode)
    L, M, N, K = shape
    A, B = seeded(L, M, N, K, seed=1, dist="uniform")
    Ad, Bd = place(A, B, mode, device)
    op = BMMCUDA()
    assert op.get_mode(Ad, Bd) == mode or 1 in (M, N, K)
    C = op(Ad, Bd)
    assert C.shape == (L, M, N) and C.dtype == torch.float32 and C.device == Ad.device
    O.check_values(C.cpu(), torch.from_numpy(O.c_bmm(A.numpy(), B.numpy())), K, "bmm")


# few tiles and a long contraction: k is cut into ranges whose partial products go
# to a workspace and are summed by a second kernel
BMM_LONG_K = [(1, 200, 136, 1000), (3, 129, 257, 517), (1, 64, 64, 4099), (2, 300, 70, 2048), (1, 1, 1, 300)]


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("shape", BMM_LONG_K)
def test_bmm_long_contraction_few_tiles(device, shape, mode):
    from custom_matmul_kernels_amd import _lib
    say("bmm long k", shape, mode)
    L, M, N, K = shape
    lib = _lib.load()
    assert lib.cmk_workspace_bytes(_lib.OP_BMM, L, M, N, K, 0) > 0
    A, B = seeded(L, M, N, K, seed=2, dist="uniform")
    Ad, Bd = place(A, B, mode, device)
    op = BMMCUDA()
    C = op(Ad, Bd)
    O.check_values(C.cpu(), torch.from_numpy(O.c_bmm(A.numpy(), B.numpy())), K, "bmm long k")
    assert torch.equal(C, op(Ad, Bd)), "two runs differ"
    # small integers: every partial sum is exact, so the cut must not show
    gen = torch.Generator().manual_seed(K)
    Ai = torch.randint(-3, 4, (L, M, K), generator=gen).float()
    Bi = torch.randint(-3, 4, (L, K, N), generator=gen).float()
    Aid, Bid = place(Ai, Bi, mode, device)
    assert torch.equal(op(Aid, Bid).cpu(), torch.bmm(Ai.double(), Bi.double()).float())


def test_bmm_workspace_entry_point_through_the_abi(device):
    """cmk_bmm_ws_f32 against cmk_bmm_f32 on the same operands: equal within fp32
    rounding where k is cut, bit-equal where it is not; too small a workspace is
    refused with a message and nothing is launched."""
    from custom_matmul_kernels_amd import _lib
    lib = _lib.load()
    stream = torch.cuda.current_stream(device).cuda_stream
    for (L, M, N, K) in [(1, 256, 256, 2048), (2, 100, 90, 700), (4, 512, 512, 512)]:
        say("bmm ws abi", (L, M, N, K))
        A, B = seeded(L, M, N, K, seed=5, dist="uniform")
        Ad, Bd = A.to(device), B.to(device)
        d = _lib.GemmDesc(L, M, N, K, 0, 0, K, N, M * K, K * N)
        plain = torch.full((L, M, N), float("nan"), device=device)
        _lib.check(lib.cmk_bmm_f32(Ad.data_ptr(), Bd.data_ptr(), plain.data_ptr(), d, stream))
        need = lib.cmk_workspace_bytes(_lib.OP_BMM, L, M, N, K, 0)
        ws = torch.empty(max(need, 1), dtype=torch.uint8, device=device)
        cut = torch.full((L, M, N), float("nan"), device=device)
        _lib.check(lib.cmk_bmm_ws_f32(Ad.data_ptr(), Bd.data_ptr(), cut.data_ptr(), d, ws.data_ptr(), need, stream))
        torch.cuda.synchronize()
        if need == 0:
            assert torch.equal(cut, plain)
        else:
            O.check_values(cut.cpu(), plain.cpu(), K, "bmm ws against plain")
            untouched = torch.full((L, M, N), 7.0, device=device)
            rc = lib.cmk_bmm_ws_f32(Ad.data_ptr(), Bd.data_ptr(), untouched.data_ptr(), d, ws.data_ptr(), need - 1,
                                    stream)
            torch.cuda.synchronize()
            assert rc == _lib.ERR_WORKSPACE and b"workspace" in lib.cmk_last_error()
            assert (untouched == 7.0).all()


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("name", INT_CASES)
def test_bmm_integer_cases_are_bit_exact(device, name, mode):
    say("bmm int", name, mode)
    g = golden()
    A, B = golden_inputs(g, name)
    Ad, Bd = place(A, B, mode, device)
    C = BMMCUDA()(Ad, Bd)
    assert torch.equal(C.cpu(), torch.from_numpy(g[name + "_C"].astype(np.float32)))


def test_bmm_2d_views_and_empty(device):
    A, B = seeded(1, 50, 60, 24, seed=4)
    C = BMMCUDA()(A[0].to(device), B[0].to(device))
    assert C.shape == (50, 60)
    O.check_values(C.cpu(), torch.bmm(A, B)[0], 24)
    # a strided window of a larger tensor is consumed in place
    big = torch.randn(2, 80, 96, generator=torch.Generator().manual_seed(9))
    win = big[:, 5:55, 8:32]
    Bw = torch.randn(2, 24, 33, generator=torch.Generator().manual_seed(10))
    C = BMMCUDA()(big.to(device)[:, 5:55, 8:32], Bw.to(device))
    O.check_values(C.cpu(), torch.bmm(win, Bw), 24)
    # K = 0 gives zeros, empty outputs stay empty
    Z = BMMCUDA()(torch.zeros(2, 5, 0, device=device), torch.zeros(2, 0, 7, device=device))
    assert Z.shape == (2, 5, 7) and (Z == 0).all()
    assert BMMCUDA()(torch.zeros(0, 5, 3, device=device), torch.zeros(0, 3, 7, device=device)).shape == (0, 5, 7)


def test_bmm_config_shape(device):
    """A[128,1024,128] @ B[128,128,1024], U(-1,1): sampled against float64."""
    say("bmm config")
    A, B = seeded(128, 1024, 1024, 128, seed=0, dist="uniform")
    C = BMMCUDA()(A.to(device), B.to(device)).cpu()
    for b in (0, 63, 127):
        want = (A[b].double() @ B[b].double()).float()
        O.check_values(C[b], want, 128, "bmm batch %d" % b)


# ---------------------------------------------------------------- mbmm -------
def random_masks(L, M, N, seed, share):
    gen = torch.Generator().manual_seed(seed)
    lead = 1 if share else L
    tiles = torch.rand(lead, -(-M // 128), -(-N // 128), generator=gen) < 0.5
    keep = tiles.repeat_interleave(128, 1).repeat_interleave(128, 2)[:, :M, :N]
    fm = torch.tril(torch.ones(M, N)).bool()[None] & keep
    return fm[0] if share else fm


@pytest.mark.parametrize("share", [False, True])
@pytest.mark.parametrize("shape", [(2, 130, 140, 8), (3, 256, 384, 40), (1, 1024, 1024, 64), (2, 77, 9, 5)])
def test_mbmm_matches_oracle(device, shape, share):
    say("mbmm", shape, share)
    L, M, N, K = shape
    A, B = seeded(L, M, N, K, seed=6)
    fm = random_masks(L, M, N, seed=7, share=share)
    bm, tm, em = O.ref_derive_masks(fm)
    dbm, dtm, dem = derive_masks(fm.to(device))
    assert torch.equal(dbm.cpu(), bm) and torch.equal(dtm.cpu(), tm) and torch.equal(dem.cpu(), em)
    C = MBMMCUDA(share_mask=share)(A.to(device), B.to(device), dbm, dtm, dem)
    full = fm[None].expand(L, -1, -1) if share else fm
    want = O.ref_mbmm(A, B, full)
    O.check_values(C.cpu(), want, K, "mbmm")
    assert (C.cpu()[~full] == 0).all()                      # masked-out entries are exactly 0
    if M * N * K <= 3 * 256 * 384 * 40:
        O.check_values(C.cpu(), torch.from_numpy(
            O.c_mbmm(A.numpy(), B.numpy(), bm.numpy(), tm.numpy(), em.numpy(), share)), K, "mbmm vs C")


MASK_SHAPES = [(1, 1, 1), (2, 130, 140), (1, 128, 128), (3, 256, 384), (2, 77, 9), (1, 1000, 1040),
               (2, 136, 272), (1, 8, 2049)]


@pytest.mark.parametrize("kind", ["bernoulli", "tril", "sparse", "bytes"])
@pytest.mark.parametrize("shape", MASK_SHAPES)
def test_derive_masks_matches_oracle(device, shape, kind):
    """Bit-exact against the oracle's derivation: aligned and unaligned row
    pitches, ragged extents, 2-D (shared) masks, a storage offset that breaks
    16-byte alignment, and uint8 masks whose kept bytes are not 1."""
    say("derive_masks", shape, kind)
    L, M, N = shape
    g = torch.Generator().manual_seed(11)
    if kind == "bernoulli":
        fm = torch.rand(L, M, N, generator=g) < 0.5
    elif kind == "tril":
        fm = torch.tril(torch.ones(M, N)).bool()[None].expand(L, -1, -1).contiguous()
    elif kind == "sparse":
        fm = torch.rand(L, M, N, generator=g) < 0.0005
    else:
        fm = (torch.randint(0, 256, (L, M, N), generator=g, dtype=torch.int32)
              * (torch.rand(L, M, N, generator=g) < 0.3)).to(torch.uint8)
    for mask in (fm, fm[0]):
        bm, tm, em = O.ref_derive_masks(mask)
        dbm, dtm, dem = derive_masks(mask.to(device))
        assert dbm.dtype == dtm.dtype == dem.dtype == torch.uint8
        assert torch.equal(dbm.cpu(), bm) and torch.equal(dtm.cpu(), tm) and torch.equal(dem.cpu(), em)
    # the same mask at an odd byte offset inside a larger allocation
    flat = torch.zeros(fm.numel() + 3, dtype=fm.dtype, device=device)
    flat[3:] = fm.to(device).reshape(-1)
    bm, tm, em = O.ref_derive_masks(fm)
    dbm, dtm, dem = derive_masks(flat[3:].view(L, M, N))
    assert torch.equal(dbm.cpu(), bm) and torch.equal(dtm.cpu(), tm) and torch.equal(dem.cpu(), em)


def test_derive_masks_full_size_properties(device):
    """At the mbmm benchmark's size: counts add up to the number of kept
    elements, a block is flagged exactly when one of its counts is non-zero,
    and the result equals the oracle's."""
    L, M, N = 128, 1024, 1024
    g = torch.Generator().manual_seed(5)
    keep = torch.rand(L, M // 128, N // 128, generator=g) < 0.5
    fm = torch.tril(torch.ones(M, N)).bool()[None] & keep.repeat_interleave(128, 1).repeat_interleave(128, 2)
    dbm, dtm, dem = derive_masks(fm.to(device))
    assert int(dtm.sum(dtype=torch.int64)) == int(fm.sum())
    per_block = dtm.view(L, M // 128, 16, N // 128, 16).sum(dim=(2, 4), dtype=torch.int32)
    assert torch.equal(per_block > 0, dbm.bool())
    bm, tm, em = O.ref_derive_masks(fm)
    assert torch.equal(dbm.cpu(), bm) and torch.equal(dtm.cpu(), tm)


def test_mbmm_mask_precedence_and_integer_exactness(device):
    g = golden()
    for name in INT_CASES:
        A, B = golden_inputs(g, name)
        bm, tm, em = derive_masks(torch.from_numpy(g[name + "_mask"]).to(device))
        C = MBMMCUDA(share_mask=True)(A.to(device), B.to(device), bm, tm, em)
        assert torch.equal(C.cpu(), torch.from_numpy(g[name + "_Cmasked"].astype(np.float32)))
    # inconsistent masks: block beats thread beats element, the byte multiplies
    A, B = seeded(1, 130, 140, 8, seed=7)
    bm = torch.ones(1, 2, 2, dtype=torch.uint8)
    tm = torch.ones(1, 17, 18, dtype=torch.uint8)
    em = torch.ones(1, 130, 140, dtype=torch.uint8)
    bm[0, 1, 0] = 0
    tm[0, 0, 1] = 0
    em[0, 20, 30] = 0
    em[0, 21, 31] = 3
    C = MBMMCUDA()(A.to(device), B.to(device), bm.to(device), tm.to(device), em.to(device)).cpu()
    want = torch.from_numpy(O.c_mbmm(A.numpy(), B.numpy(), bm.numpy(), tm.numpy(), em.numpy(), False))
    O.check_values(C, want, 8)
    assert (C[0, 128:, :128] == 0).all() and (C[0, :8, 8:16] == 0).all() and C[0, 20, 30] == 0
    # the same on a shape whose kept tiles take their masks through LDS (N % 16 == 0)
    A2, B2 = seeded(1, 256, 256, 8, seed=8)
    bm2 = torch.ones(1, 2, 2, dtype=torch.uint8)
    tm2 = torch.ones(1, 32, 32, dtype=torch.uint8)
    em2 = torch.ones(1, 256, 256, dtype=torch.uint8)
    bm2[0, 1, 0] = 0
    tm2[0, 0, 1] = 0
    tm2[0, 31, 31] = 0
    em2[0, 20, 30] = 0
    em2[0, 21, 31] = 3
    em2[0, 200, 250] = 7
    C2 = MBMMCUDA()(A2.to(device), B2.to(device), bm2.to(device), tm2.to(device), em2.to(device)).cpu()
    want2 = torch.from_numpy(O.c_mbmm(A2.numpy(), B2.numpy(), bm2.numpy(), tm2.numpy(), em2.numpy(), False))
    O.check_values(C2, want2, 8)
    assert (C2[0, 128:, :128] == 0).all() and (C2[0, :8, 8:16] == 0).all() and C2[0, 20, 30] == 0
    assert (C2[0, 248:, 248:] == 0).all()
    # all-ones masks reproduce bmm, an all-zero block mask gives zeros
    ones = [torch.ones_like(t).to(device) for t in (bm, tm, em)]
    assert torch.equal(MBMMCUDA()(A.to(device), B.to(device), *ones), BMMCUDA()(A.to(device), B.to(device)))
    zb = torch.zeros_like(bm).to(device)
    assert (MBMMCUDA()(A.to(device), B.to(device), zb, ones[1], ones[2]) == 0).all()


def test_mbmm_config_3_properties(device):
    """A[128,1024,64] @ B[128,64,1024] under tril AND tile-Bernoulli(0.5) masks, at
    full size: dropped elements are exactly zero, kept elements equal the dense
    product of the same library bit for bit, three batches are checked against
    float64, and a skipped tile never touches its operands (NaNs planted there
    do not leak)."""
    say("mbmm config 3")
    L, M, N, K = 128, 1024, 1024, 64
    A, B = seeded(L, M, N, K, seed=0)
    fm = random_masks(L, M, N, seed=1, share=False)
    Ad, Bd, fd = A.to(device), B.to(device), fm.to(device)
    bm, tm, em = derive_masks(fd)
    C = MBMMCUDA(share_mask=False)(Ad, Bd, bm, tm, em)
    assert (C[~fd] == 0).all()
    dense = BMMCUDA()(Ad, Bd)
    assert torch.equal(C[fd], dense[fd])
    for b in (0, 77, 127):
        want = (A[b].double() @ B[b].double()).float() * fm[b]
        O.check_values(C[b].cpu(), want, K, "mbmm batch %d" % b)
    # batch 5, tile row 0: rows 0..127 of A feed only tiles (0, 0) (tril); if that
    # tile is skipped, NaNs in those rows must not show anywhere in the output
    if bm[5, 0, 0] == 0:
        A2 = Ad.clone()
        A2[5, :128] = float("nan")
        C2 = MBMMCUDA(share_mask=False)(A2, Bd, bm, tm, em)
        assert torch.equal(C2[5], C[5])


# ---------------------------------------------------------------- min_bmm ----
MIN_SHAPES = [(1, 1, 1, 1), (2, 37, 300, 19), (1, 129, 257, 33), (3, 128, 128, 64),
              (1, 200, 1000, 70), (1, 1000, 200, 12), (2, 64, 2000, 32)]


@pytest.mark.parametrize("dim", [1, 2])
@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("shape", MIN_SHAPES)
def test_min_bmm_matches_oracle(device, shape, mode, dim):
    say("min", shape, mode, dim)
    L, M, N, K = shape
    A, B = seeded(L, M, N, K, seed=2)
    Ad, Bd = place(A, B, mode, device)
    v, i = MinBMMCUDA()(Ad, Bd, dim=dim)
    kept = N if dim == 1 else M
    assert v.shape == (L, kept) and i.shape == (L, kept) and i.dtype == torch.int64
    cv, ci = O.c_min_bmm(A.numpy(), B.numpy(), dim)
    O.check_min(v, i, A, B, dim, ref=(torch.from_numpy(cv), torch.from_numpy(ci)))
    O.check_min(v, i, A, B, dim)


@pytest.mark.parametrize("dim", [1, 2])
@pytest.mark.parametrize("name", INT_CASES)
def test_min_bmm_integer_cases_and_ties(device, name, dim):
    """Exact products with many ties: values bit-exact, lowest index wins."""
    say("min int", name, dim)
    g = golden()
    A, B = golden_inputs(g, name)
    for mode in ("nn", "tt"):
        Ad, Bd = place(A, B, mode, device)
        v, i = MinBMMCUDA()(Ad, Bd, dim=dim)
        assert torch.equal(v.cpu(), torch.from_numpy(g["%s_min%d_val" % (name, dim)].astype(np.float32)))
        assert torch.equal(i.cpu(), torch.from_numpy(g["%s_min%d_idx" % (name, dim)].astype(np.int64)))


DIST_SHAPES = [(1, 5, 7, 3), (2, 130, 140, 33), (1, 300, 260, 64), (1, 64, 1100, 40)]


@pytest.mark.parametrize("distance", ["l2", "l1"])
@pytest.mark.parametrize("dim", [1, 2])
@pytest.mark.parametrize("mode", ["nn", "tt", "nt"])
@pytest.mark.parametrize("shape", DIST_SHAPES)
def test_min_bmm_distances_match_oracle(device, shape, mode, dim, distance):
    """(a-b)^2 and |a-b| accumulate on the vector unit in the reference's order
    of operations: values are bit-equal to the C oracle, ties go to the lowest
    index."""
    say("min", distance, shape, mode, dim)
    L, M, N, K = shape
    A, B = seeded(L, M, N, K, seed=12)
    Ad, Bd = place(A, B, mode, device)
    v, i = MinBMMCUDA(distance=distance)(Ad, Bd, dim=dim)
    code = {"l2": 1, "l1": 2}[distance]
    cv, ci = O.c_min_bmm(A.numpy(), B.numpy(), dim, code)
    assert torch.equal(v.cpu(), torch.from_numpy(cv))
    assert torch.equal(i.cpu(), torch.from_numpy(ci).long())
    # closed form: torch.cdist between the rows of A and the columns of B
    p = 2 if distance == "l2" else 1
    D = torch.cdist(A.double(), B.double().transpose(1, 2), p=p)
    if p == 2:
        D = D ** 2
    want = D.min(dim)[0]
    assert torch.allclose(v.cpu().double(), want, rtol=1e-4, atol=1e-3 * K ** 0.5)


@pytest.mark.parametrize("distance", ["euclidean", "manhattan"])
@pytest.mark.parametrize("dim", [1, 2])
@pytest.mark.parametrize("shape", [(1, 5, 7, 3), (2, 130, 300, 33), (1, 70, 2500, 16)])
def test_topk_bmm_distances_match_oracle(device, shape, dim, distance):
    """Largest k of the accumulated distances, as the reference's kernels would
    select them (its top-k always keeps the largest values)."""
    say("topk", distance, shape, dim)
    L, M, N, K = shape
    A, B = seeded(L, M, N, K, seed=13)
    v, i = TopkBMMCUDA(distance=distance)(A.to(device), B.to(device), k=128, dim=dim)
    code = {"euclidean": 1, "manhattan": 2}[distance]
    cv, ci = O.c_topk_bmm(A.numpy(), B.numpy(), 128, dim, code)
    red = M if dim == 1 else N
    kk = min(128, red)
    assert torch.equal(v.cpu()[..., :kk], torch.from_numpy(cv)[..., :kk])
    # indices: equal wherever the value is not repeated in the row
    gv = v.cpu()[..., :kk]
    uniq = torch.ones_like(gv, dtype=torch.bool)
    uniq[..., 1:] &= gv[..., 1:] != gv[..., :-1]
    uniq[..., :-1] &= gv[..., :-1] != gv[..., 1:]
    uniq &= gv != gv[..., -1:]          # a tie with the first value left out may pick either
    gi, wi = i.cpu()[..., :kk], torch.from_numpy(ci).long()[..., :kk]
    bad = (gi != wi) & uniq
    assert not bad.any(), (bad.nonzero()[:5], gi[bad][:5], wi[bad][:5], gv[bad][:5])


def test_min_bmm_dims_2d_negative_and_determinism(device):
    A, B = seeded(1, 300, 500, 48, seed=8)
    op = MinBMMCUDA()
    v2, i2 = op(A[0].to(device), B[0].to(device), dim=1)       # 2-D: dim 1 = over n
    v3, i3 = op(A.to(device), B.to(device), dim=2)
    vn, i_n = op(A.to(device), B.to(device), dim=-1)
    assert v2.shape == (300,) and torch.equal(v2, v3[0]) and torch.equal(i2, i3[0])
    assert torch.equal(vn, v3) and torch.equal(i_n, i3)
    v0, i0 = op(A[0].to(device), B[0].to(device), dim=0)
    v1, i1 = op(A.to(device), B.to(device), dim=1)
    assert v0.shape == (500,) and torch.equal(v0, v1[0]) and torch.equal(i0, i1[0])
    for _ in range(3):                                         # run-to-run identical
        w, j = op(A.to(device), B.to(device), dim=2)
        assert torch.equal(w, v3) and torch.equal(j, i3)
    with pytest.raises(ValueError):
        op(torch.zeros(1, 4, 3, device=device), torch.zeros(1, 3, 0, device=device), dim=2)


def test_min_bmm_config_1(device):
    """A[1,4096,64] @ B[1,64,4096], N(0,1), min over dim=-1, vs torch on the CPU."""
    say("min config 1")
    A, B = seeded(1, 4096, 4096, 64, seed=0)
    v, i = MinBMMCUDA()(A.to(device), B.to(device), dim=-1)
    mism = O.check_min(v, i, A, B, 2)
    assert mism <= 4


def test_min_bmm_large_rows_sampled(device):
    """Config-4 geometry with fewer rows of A (A[1,2048,256] @ B[1,256,65536]):
    every output row still walks all 65536 columns; checked in full on the CPU."""
    say("min large")
    A, B = seeded(1, 2048, 65536, 256, seed=0)
    v, i = MinBMMCUDA()(A.to(device), B.to(device), dim=2)
    assert O.check_min(v, i, A, B, 2) <= 4


def test_min_bmm_config_4_properties(device):
    """Full config 4 (65536 x 65536 x 256): the product has 2^32 entries, so the
    check is by properties - sampled rows against the CPU, value-at-index for
    all rows, and agreement of dim=1 on the transposed problem."""
    say("min config 4")
    gen = torch.Generator().manual_seed(0)
    A = torch.randn(1, 65536, 256, generator=gen)
    B = torch.randn(1, 256, 65536, generator=gen)
    Ad, Bd = A.to(device), B.to(device)
    v, i = MinBMMCUDA()(Ad, Bd, dim=-1)
    torch.cuda.synchronize()
    v, i = v.cpu(), i.cpu()
    rows = torch.arange(0, 65536, 257)
    rv, ri = O.ref_min_bmm(A[:, rows], B, 2)
    O.check_min(v[:, rows], i[:, rows], A[:, rows], B, 2, ref=(rv, ri))
    at = O.gather_products(A, B, 2, i)
    O.check_values(v, at, 256, "value at index")
    # transposed problem, reduced over dim=1: same answer
    vt, it = MinBMMCUDA()(Bd.transpose(1, 2), Ad.transpose(1, 2), dim=1)
    assert torch.equal(vt.cpu(), v) and torch.equal(it.cpu(), i)


# ---------------------------------------------------------------- topk_bmm ---
TOPK_SHAPES = [(1, 1, 1, 1), (2, 37, 300, 19), (1, 129, 257, 33), (2, 64, 1024, 64),
               (1, 40, 2500, 24), (1, 2500, 40, 24), (3, 33, 100, 8), (1, 70, 5000, 16)]


@pytest.mark.parametrize("dim", [1, 2])
@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("shape", TOPK_SHAPES)
def test_topk_bmm_matches_oracle(device, shape, mode, dim):
    say("topk", shape, mode, dim)
    L, M, N, K = shape
    A, B = seeded(L, M, N, K, seed=3)
    Ad, Bd = place(A, B, mode, device)
    v, i = TopkBMMCUDA()(Ad, Bd, k=128, dim=dim)
    kept = N if dim == 1 else M
    assert v.shape == (L, kept, 128) and i.shape == (L, kept, 128) and i.dtype == torch.int64
    O.check_topk(v, i, A, B, 128, dim)
    red = M if dim == 1 else N
    if L * kept * red * K <= 2 * 64 * 1024 * 64:
        cv, ci = O.c_topk_bmm(A.numpy(), B.numpy(), 128, dim)
        O.check_values(v.cpu(), torch.from_numpy(cv), K, "topk vs C oracle")


@pytest.mark.parametrize("dim", [1, 2])
@pytest.mark.parametrize("name", INT_CASES)
def test_topk_bmm_integer_cases_and_ties(device, name, dim):
    say("topk int", name, dim)
    g = golden()
    A, B = golden_inputs(g, name)
    want = golden_topk_values(g, name, dim)
    C = torch.from_numpy(g[name + "_C"].astype(np.float32))
    Cr = C if dim == 2 else C.transpose(1, 2)
    v, i = TopkBMMCUDA()(A.to(device), B.to(device), k=128, dim=dim)
    v, i = v.cpu(), i.cpu()
    assert torch.equal(v, want)                                   # bit-exact values, -inf padding
    ok = torch.isfinite(want)
    assert torch.equal(i >= 0, ok) and (i[~ok] == -1).all()
    assert torch.equal(torch.gather(Cr, 2, i.clamp(min=0))[ok], want[ok])
    s = torch.where(ok, i, torch.arange(128).expand_as(i) + 10 ** 6).sort(-1).values
    assert (s[..., 1:] != s[..., :-1]).all()                      # no index twice
    # equal values come out by ascending index
    same = ok[..., 1:] & (v[..., 1:] == v[..., :-1])
    assert (i[..., 1:][same] > i[..., :-1][same]).all()


def test_topk_bmm_k_prefix_2d_and_determinism(device):
    A, B = seeded(1, 100, 3000, 32, seed=5)
    op = TopkBMMCUDA()
    v128, i128 = op(A.to(device), B.to(device), k=128, dim=2)
    for k in (1, 7, 64, 100):
        v, i = op(A.to(device), B.to(device), k=k, dim=2)
        assert v.shape == (1, 100, k) and v.is_contiguous()
        assert torch.equal(v, v128[..., :k]) and torch.equal(i, i128[..., :k])
    v2, i2 = op(A[0].to(device), B[0].to(device), k=128, dim=1)    # 2-D: dim 1 = over n
    assert v2.shape == (100, 128) and torch.equal(v2, v128[0]) and torch.equal(i2, i128[0])
    vn, i_n = op(A.to(device), B.to(device), k=128, dim=-1)
    assert torch.equal(vn, v128) and torch.equal(i_n, i128)
    for _ in range(3):
        w, j = op(A.to(device), B.to(device), k=128, dim=2)
        assert torch.equal(w, v128) and torch.equal(j, i128)


def test_topk_bmm_config_5_slice(device):
    """Config-5 geometry with fewer rows (A[1,8192,256] @ B[1,256,1024], k=128)."""
    say("topk config 5 slice")
    A, B = seeded(1, 8192, 1024, 256, seed=0)
    v, i = TopkBMMCUDA()(A.to(device), B.to(device), k=128, dim=-1)
    assert O.check_topk(v, i, A, B, 128, 2) <= 64


def test_topk_bmm_long_axis_split(device):
    """The notebook's benchmark geometry (top-128 over the long axis, dim=1) at
    reduced length: A[1,65536,64] @ B[1,64,256]."""
    say("topk long axis")
    A, B = seeded(1, 65536, 256, 64, seed=1)
    v, i = TopkBMMCUDA()(A.to(device), B.to(device), k=128, dim=1)
    assert v.shape == (1, 256, 128)
    assert O.check_topk(v, i, A, B, 128, 1) <= 16


def test_topk_bmm_config_5_properties(device):
    """Full config 5 (2^20 rows): sampled rows against the CPU plus
    size-independent properties over all rows."""
    say("topk config 5")
    gen = torch.Generator().manual_seed(0)
    A = torch.randn(1, 1048576, 256, generator=gen)
    B = torch.randn(1, 256, 1024, generator=gen)
    Ad, Bd = A.to(device), B.to(device)
    v, i = TopkBMMCUDA()(Ad, Bd, k=128, dim=-1)
    torch.cuda.synchronize()
    assert (v[..., :-1] >= v[..., 1:]).all()
    assert ((i >= 0) & (i < 1024)).all()
    s = i.sort(-1).values
    assert (s[..., 1:] != s[..., :-1]).all()
    del s
    # the smallest selected value bounds the row maximum from below and the
    # largest equals the row maximum of A@B (checked on a slab of rows on the GPU)
    Cs = torch.bmm(Ad[:, :65536], Bd)
    O.check_values(v[:, :65536, 0].cpu(), Cs.max(-1).values.cpu(), 256, "row maximum")
    del Cs
    rows = torch.arange(0, 1048576, 4099)
    vs, is_ = v[:, rows].cpu(), i[:, rows].cpu()
    assert O.check_topk(vs, is_, A[:, rows], B, 128, 2) <= 8


def test_bitonic_sort_1d(device):
    op = BitonicSort()
    gen = torch.Generator().manual_seed(4)
    for n in (1, 100, 128, 1000, 100000, 3000000):
        x = torch.randn(n, generator=gen)
        v, i = op(x.to(device), k=128)
        kk = min(n, 128)
        want = x.sort(descending=True).values[:kk]
        assert torch.equal(v.cpu()[:kk], want)
        assert torch.equal(x[i.cpu()[:kk]], want)
        if n < 128:
            assert torch.isinf(v.cpu()[n:]).all() and (i.cpu()[n:] == -1).all()
        cv, ci = O.c_topk_1d(x.numpy(), 128)
        assert np.array_equal(cv, v.cpu().numpy())


def test_non_default_stream(device):
    A, B = seeded(1, 512, 512, 64, seed=11)
    Ad, Bd = A.to(device), B.to(device)
    want = BMMCUDA()(Ad, Bd)
    s = torch.cuda.Stream(device=device)
    s.wait_stream(torch.cuda.current_stream(device))
    with torch.cuda.stream(s):
        got = BMMCUDA()(Ad, Bd)
        mv, mi = MinBMMCUDA()(Ad, Bd, dim=2)
    s.synchronize()
    assert torch.equal(got, want)
    mv0, mi0 = MinBMMCUDA()(Ad, Bd, dim=2)
    assert torch.equal(mv, mv0) and torch.equal(mi, mi0)


def test_entry_points_replay_in_a_hip_graph(device):
    """The entry points only enqueue kernels on the given stream, so a sequence of
    them can be captured once and replayed: every replay, with new inputs copied
    into the captured buffers and eager work in between, matches the eager result."""
    say("graph replay")
    L, M, N, K = 2, 300, 520, 72
    gen = torch.Generator().manual_seed(21)
    A = torch.randn(L, M, K, generator=gen).to(device)
    B = torch.randn(L, K, N, generator=gen).to(device)
    ops = (BMMCUDA(), MinBMMCUDA(), TopkBMMCUDA())

    def run_all():
        return (ops[0](A, B), *ops[1](A, B, dim=2), *ops[2](A, B, k=128, dim=1))

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            run_all()                                   # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = run_all()
    for step in range(3):
        A.copy_(torch.randn(L, M, K, generator=gen))
        B.copy_(torch.randn(L, K, N, generator=gen))
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in captured]
        want = run_all()                                # eager, between the replays
        torch.cuda.synchronize()
        for g, w in zip(got, want):
            assert torch.equal(g, w), "replay %d differs from the eager result" % step


def test_two_host_threads_on_two_streams(device):
    """The library keeps no state between calls except the thread-local error
    string: two host threads, each on a stream of its own, get the results they
    get when run one after the other."""
    import threading
    say("host threads")
    gen = torch.Generator().manual_seed(33)
    inputs = [(torch.randn(1, 700, 96, generator=gen).to(device), torch.randn(1, 96, 900, generator=gen).to(device))
              for _ in range(2)]
    want = [(MinBMMCUDA()(a, b, dim=2), TopkBMMCUDA()(a, b, k=64, dim=2)) for a, b in inputs]
    torch.cuda.synchronize()
    got = [None, None]
    errors = []

    def work(i):
        try:
            s = torch.cuda.Stream()
            with torch.cuda.stream(s):
                a, b = inputs[i]
                for _ in range(20):
                    r = (MinBMMCUDA()(a, b, dim=2), TopkBMMCUDA()(a, b, k=64, dim=2))
                s.synchronize()
                got[i] = r
        except Exception as e:  # noqa: BLE001 - reported below
            errors.append(e)

    threads = [threading.Thread(target=work, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for i in range(2):
        for (gv, gi), (wv, wi) in zip(got[i], want[i]):
            assert torch.equal(gv, wv) and torch.equal(gi, wi)
