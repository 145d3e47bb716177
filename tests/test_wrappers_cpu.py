"""Host logic of the operator classes, checked without a GPU against the
reference's wrappers read as text (bmm.py:56-90, minbmm.py:86-100,
topkbmm.py:89-104, mbmm.py:62-72)."""
import pytest
import torch

from custom_matmul_kernels_amd import (BMMCUDA, MBMMCUDA, MinBMMCUDA, TopkBMMCUDA, _common,
                                       derive_masks)
from oracle import oracle as O


def test_mode_from_strides():
    A = torch.zeros(2, 5, 7)
    B = torch.zeros(2, 7, 3)
    assert BMMCUDA().get_mode(A, B) == "nn"
    assert BMMCUDA().get_mode(torch.zeros(2, 7, 5).transpose(1, 2), B) == "tn"
    assert BMMCUDA().get_mode(A, torch.zeros(2, 3, 7).transpose(1, 2)) == "nt"
    assert MinBMMCUDA().get_mode(torch.zeros(2, 7, 5).transpose(1, 2),
                                 torch.zeros(2, 3, 7).transpose(1, 2)) == "tt"
    assert _common.get_mode(A[:, :, ::2], B) == [None, "n"]


def test_descriptor_for_each_layout():
    A = torch.zeros(2, 5, 7)
    B = torch.zeros(2, 7, 3)
    _, _, d = _common.make_desc(A, B)
    assert (d.L, d.M, d.N, d.K, d.transA, d.transB) == (2, 5, 3, 7, 0, 0)
    assert (d.lda, d.ldb, d.strideA, d.strideB) == (7, 3, 35, 21)
    At = torch.zeros(2, 7, 5).transpose(1, 2)
    Bt = torch.zeros(2, 3, 7).transpose(1, 2)
    _, _, d = _common.make_desc(At, Bt)
    assert (d.transA, d.transB, d.lda, d.ldb) == (1, 1, 5, 7)
    # a row-sliced view keeps its parent's leading dimension
    big = torch.zeros(2, 10, 16)
    _, _, d = _common.make_desc(big[:, 2:7, 4:11], B)
    assert (d.transA, d.lda, d.strideA, d.K) == (0, 16, 160, 7)
    # strides that fit neither layout are copied
    A2, _, d = _common.make_desc(torch.zeros(2, 5, 14)[:, :, ::2], B)
    assert A2.is_contiguous() and (d.transA, d.lda) == (0, 7)
    # a batch broadcast by expand() has batch stride 0
    _, _, d = _common.make_desc(torch.zeros(1, 5, 7).expand(2, 5, 7), B)
    assert d.strideA == 0


def test_dim_convention():
    # 3-D: 1 = over m, 2 = over n; 2-D inputs shift by one; negatives count from the end
    assert _common.normalize_dim(1, False) == 1
    assert _common.normalize_dim(2, False) == 2
    assert _common.normalize_dim(0, True) == 1
    assert _common.normalize_dim(1, True) == 2
    assert _common.normalize_dim(-1, False) == 2
    assert _common.normalize_dim(-1, True) == 2
    assert _common.normalize_dim(-2, True) == 1
    for bad, two in ((0, False), (3, False), (2, True), (-3, False)):
        with pytest.raises(AssertionError):
            _common.normalize_dim(bad, two)


def test_unknown_distance_raises():
    with pytest.raises(ValueError):
        MinBMMCUDA(distance="cosine")
    with pytest.raises(ValueError):
        TopkBMMCUDA(distance="cosine")
    assert MinBMMCUDA(distance="euclidean").distance == "euclidean"


def test_shape_and_dtype_checks_fire_before_any_launch():
    bmm = BMMCUDA()
    with pytest.raises(ValueError):
        bmm(torch.zeros(2, 2, 2, 2), torch.zeros(2, 2, 2, 2))
    with pytest.raises(AssertionError):
        bmm(torch.zeros(2, 3), torch.zeros(2, 3, 4))
    with pytest.raises(AssertionError):
        bmm(torch.zeros(2, 5, 7), torch.zeros(3, 7, 3))       # batch mismatch
    with pytest.raises(AssertionError):
        bmm(torch.zeros(2, 5, 7), torch.zeros(2, 6, 3))       # contraction mismatch
    with pytest.raises(TypeError):
        bmm(torch.zeros(2, 5, 7, dtype=torch.half), torch.zeros(2, 7, 3, dtype=torch.half))
    with pytest.raises(AssertionError):
        bmm(torch.zeros(2, 5, 7), torch.zeros(2, 7, 3))       # CPU tensors are refused
    with pytest.raises(AssertionError):
        TopkBMMCUDA()(torch.zeros(2, 5, 7), torch.zeros(2, 7, 3), k=129, dim=2)
    with pytest.raises(AssertionError):
        MinBMMCUDA()(torch.zeros(2, 5, 7), torch.zeros(2, 7, 3), dim=3)
    with pytest.raises(AssertionError):
        MBMMCUDA(share_mask=1)
    mb = MBMMCUDA()
    u8 = torch.uint8
    # every mode is dispatched ("tn": A is [l, k, m]); CPU tensors are refused after the shape checks
    with pytest.raises(AssertionError):
        mb(torch.zeros(1, 8, 8), torch.zeros(1, 8, 8), torch.zeros(1, 1, 1, dtype=u8),
           torch.zeros(1, 1, 1, dtype=u8), torch.zeros(1, 8, 8, dtype=u8), mode="tn")
    with pytest.raises(AssertionError):
        mb(torch.zeros(1, 5, 8), torch.zeros(1, 8, 8), torch.zeros(1, 1, 1, dtype=u8),
           torch.zeros(1, 1, 1, dtype=u8), torch.zeros(1, 8, 8, dtype=u8), mode="tn")   # k: 5 vs 8
    with pytest.raises(KeyError):
        mb(torch.zeros(1, 8, 8), torch.zeros(1, 8, 8), torch.zeros(1, 1, 1, dtype=u8),
           torch.zeros(1, 1, 1, dtype=u8), torch.zeros(1, 8, 8, dtype=u8), mode="xx")


def test_derive_masks_rejects_host_tensors_and_other_dtypes():
    with pytest.raises(ValueError):
        derive_masks(torch.ones(8, 8, dtype=torch.bool))
    with pytest.raises(TypeError):
        derive_masks(torch.ones(8, 8))
    with pytest.raises(ValueError):
        derive_masks(torch.ones(8, dtype=torch.bool))


def test_oracle_mask_derivation_follows_the_notebook_rule():
    m, n = 256, 384
    fm = torch.tril(torch.ones(m, n)).bool()
    bm, tm, em = O.ref_derive_masks(fm)
    # colab/test_mbmm.ipynb:1303-1313 for shapes that are multiples of 8 / 128
    want_tm = fm.view(m // 8, 8, n // 8, 8).sum(dim=1).sum(dim=-1).to(torch.uint8)
    want_bm = fm.view(m // 128, 128, n // 128, 128).sum(dim=1).sum(dim=-1).bool().to(torch.uint8)
    assert torch.equal(tm, want_tm) and torch.equal(bm, want_bm)
    assert torch.equal(em, fm.to(torch.uint8))
    assert tm.max() == 64 and tm.dtype == torch.uint8
    # ragged extents are padded with zeros
    fm = torch.ones(2, 130, 9).bool()
    bm, tm, em = O.ref_derive_masks(fm)
    assert bm.shape == (2, 2, 1) and tm.shape == (2, 17, 2) and em.shape == (2, 130, 9)
    assert tm[0, 16, 1] == 2 and tm[0, 0, 0] == 64 and bm.all()
    # hand-counted: a single kept element, and a kept column that crosses micro-tiles
    fm = torch.zeros(136, 260, dtype=torch.bool)
    fm[129, 257] = True
    fm[3:21, 9] = True
    bm, tm, em = O.ref_derive_masks(fm)
    assert bm.tolist() == [[1, 0, 0], [0, 0, 1]]
    assert int(tm.sum()) == 19 and tm[16, 32] == 1
    assert [int(tm[i, 1]) for i in range(3)] == [5, 8, 5]


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from custom_matmul_kernels_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "libcmk.so"))
    with pytest.raises(ImportError):
        BMMCUDA()


def test_unaligned_operands_are_copied_to_padded_rows_when_it_pays():
    """A large operand whose leading dimension is not a multiple of four would rule
    out 16-byte loads in the kernels: make_desc hands over a padded copy (same
    values, aligned pitch); small or already aligned operands are passed as they are."""
    g = torch.Generator().manual_seed(0)
    A = torch.randn(2, 300, 129, generator=g)            # k = 129: rows of 129 floats
    B = torch.randn(2, 129, 301, generator=g)            # n = 301
    A2, B2, d = _common.make_desc(A, B)
    assert (d.lda, d.ldb, d.transA, d.transB) == (132, 304, 0, 0)
    assert d.strideA == 300 * 132 and d.strideB == 129 * 304
    assert torch.equal(A2, A) and torch.equal(B2, B) and A2.data_ptr() % 16 == 0
    assert A2.stride() == (300 * 132, 132, 1)
    # the "t" layouts keep their orientation
    At = A.transpose(1, 2).contiguous().transpose(1, 2)  # m contiguous, m = 300 is a multiple of 4
    Bt = B.transpose(1, 2).contiguous().transpose(1, 2)  # k contiguous, k = 129 is not
    A3, B3, d = _common.make_desc(At, Bt)
    assert (d.transA, d.transB, d.lda, d.ldb) == (1, 1, 300, 132)
    assert A3.data_ptr() == At.data_ptr() and torch.equal(B3, B) and B3.stride()[1] == 1
    # small operands are left alone
    _, _, d = _common.make_desc(torch.zeros(1, 5, 7), torch.zeros(1, 7, 9))
    assert (d.lda, d.ldb) == (7, 9)


def test_shared_unaligned_operand_is_copied_once():
    """An operand that every batch shares (batch stride 0) and that is not 16-byte
    aligned is copied as one matrix, not once per batch, and keeps its stride of 0."""
    import torch
    from custom_matmul_kernels_amd import _common
    base = torch.arange(300 * 250 + 1, dtype=torch.float32)
    one = base[1:].view(300, 250)                      # data pointer off by 4 bytes
    assert one.data_ptr() % 16 != 0
    T = one[None].expand(8, 300, 250)
    out, trans, ld, stride = _common._aligned(T, 0, 250, 0)
    assert (trans, ld, stride) == (0, 252, 0)
    assert out.shape == T.shape and out.stride(0) == 0 and torch.equal(out, T)
    assert out.data_ptr() % 16 == 0
    # the size window looks at what is physically there: a small shared matrix is left alone
    small = base[1:1 + 40 * 50].view(40, 50)[None].expand(4096, 40, 50)
    same, _, _, _ = _common._aligned(small, 0, 50, 0)
    assert same is small
