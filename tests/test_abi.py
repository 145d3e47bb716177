"""The C-ABI library loads, exports every symbol include/cmk.h declares, and
rejects bad arguments before touching the GPU (none of these calls launches a
kernel)."""
import ctypes
import os
import re

import pytest

from custom_matmul_kernels_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(_lib.LIB_PATH):
        _lib.build()
    return _lib.load()


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "cmk.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(cmk_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_list_agree():
    assert declared_symbols() == sorted(_lib.EXPORTS)


def test_every_declared_symbol_is_exported(lib):
    for name in declared_symbols():
        assert hasattr(lib, name), name


def test_abi_version(lib):
    text = open(os.path.join(ROOT, "include", "cmk.h")).read()
    assert lib.cmk_abi_version() == int(re.search(r"#define CMK_ABI_VERSION (\d+)", text).group(1))


def test_desc_layout_matches_header():
    # int x6 then long long x4: 24 + 32 bytes, naturally aligned
    assert ctypes.sizeof(_lib.GemmDesc) == 56
    assert _lib.GemmDesc.lda.offset == 24


def test_workspace_sizes(lib):
    # a small reduced operand with many strips: no split, no workspace
    assert lib.cmk_workspace_bytes(_lib.OP_MIN_BMM, 1, 65536, 1024, 256, 2) == 0
    assert lib.cmk_workspace_bytes(_lib.OP_TOPK_BMM, 1, 1048576, 1024, 256, 2) == 0
    # a large reduced operand is cut in a few ranges for L2 locality: 8 bytes per row and range
    w = lib.cmk_workspace_bytes(_lib.OP_MIN_BMM, 1, 65536, 65536, 256, 2)
    assert 0 < w <= 16 * 65536 * 8 and w % (65536 * 8) == 0
    assert lib.cmk_workspace_bytes(_lib.OP_BMM, 128, 1024, 1024, 128, 0) == 0
    # few strips: the reduced axis is split and partials need room
    w = lib.cmk_workspace_bytes(_lib.OP_MIN_BMM, 1, 4096, 4096, 64, 2)
    assert w > 0 and w % (4096 * 8) == 0
    w = lib.cmk_workspace_bytes(_lib.OP_TOPK_BMM, 1, 1048576, 1024, 256, 1)
    assert w > 0 and w % (1024 * 128 * 8) == 0
    assert lib.cmk_workspace_bytes(_lib.OP_TOPK_1D, 1, 1000, 0, 0, 0) == 128 * 8
    assert lib.cmk_workspace_bytes(_lib.OP_MIN_BMM, 1, 8, 8, 8, 3) == 0   # bad dim
    # squared l2 on the matrix pipe: norms, the queue, a copy of the reduced-axis operand and
    # 20 bytes per row and range; always more than the vector route asks for, nothing when K is 0
    for shape in ((1, 16384, 16384, 256), (1, 4096, 4096, 64), (2, 300, 500, 17)):
        for dim in (1, 2):
            small = lib.cmk_workspace_bytes(_lib.OP_MIN_BMM, *shape, dim)
            big = lib.cmk_workspace_bytes(_lib.OP_MIN_BMM_L2, *shape, dim)
            assert big > small and big % 256 == 0
            L, M, N, K = shape
            x, y = (N, M) if dim == 2 else (M, N)
            assert big >= 4 * L * (x * K + x + y) + 20 * L * y
    assert lib.cmk_workspace_bytes(_lib.OP_MIN_BMM_L2, 1, 64, 64, 0, 2) == 0
    assert lib.cmk_workspace_bytes(_lib.OP_MIN_BMM_L2, 1, 64, 64, 8, 0) == 0
    assert _lib.OP_MIN_BMM_L2 == 5


def _desc(L=1, M=8, N=8, K=8, tA=0, tB=0, lda=None, ldb=None):
    return _lib.GemmDesc(L, M, N, K, tA, tB, lda if lda is not None else K,
                         ldb if ldb is not None else N, M * K, K * N)


def test_argument_errors_return_codes_without_launching(lib):
    fake = ctypes.c_void_p(0x1000)  # never dereferenced: every call fails validation first
    assert lib.cmk_bmm_f32(fake, fake, fake, None, None) == _lib.ERR_INVALID_ARG
    assert b"descriptor" in lib.cmk_last_error()
    assert lib.cmk_bmm_f32(fake, fake, fake, _desc(M=-1), None) == _lib.ERR_INVALID_ARG
    assert lib.cmk_bmm_f32(fake, fake, fake, _desc(lda=4), None) == _lib.ERR_INVALID_ARG
    assert lib.cmk_bmm_f32(fake, fake, fake, _desc(tA=2), None) == _lib.ERR_INVALID_ARG
    assert lib.cmk_bmm_f32(None, fake, fake, _desc(), None) == _lib.ERR_INVALID_ARG
    assert lib.cmk_mbmm_f32(fake, fake, fake, fake, fake, fake, 0, _desc(tA=1, M=16, lda=8), None) \
        == _lib.ERR_INVALID_ARG            # "t" layout of A: lda must cover m
    assert lib.cmk_mbmm_f32(fake, fake, fake, None, fake, fake, 0, _desc(), None) == _lib.ERR_INVALID_ARG
    assert lib.cmk_min_bmm_f32(fake, fake, fake, fake, _desc(), 3, 0, None, 0, None) \
        == _lib.ERR_INVALID_ARG
    assert lib.cmk_min_bmm_f32(fake, fake, fake, fake, _desc(), 2, 7, None, 0, None) \
        == _lib.ERR_INVALID_ARG
    assert lib.cmk_min_bmm_f32(fake, fake, fake, fake, _desc(N=0, ldb=1), 2, 0, None, 0, None) \
        == _lib.ERR_INVALID_ARG            # empty reduction
    assert lib.cmk_topk_bmm_f32(fake, fake, fake, fake, _desc(), 2, 0, 0, None, 0, None) \
        == _lib.ERR_INVALID_ARG
    assert lib.cmk_topk_bmm_f32(fake, fake, fake, fake, _desc(), 2, 129, 0, None, 0, None) \
        == _lib.ERR_INVALID_ARG
    # a split reduction without its workspace is refused, not launched
    big = _desc(M=4096, N=4096, K=64)
    assert lib.cmk_min_bmm_f32(fake, fake, fake, fake, big, 2, 0, None, 0, None) == _lib.ERR_WORKSPACE
    assert b"workspace" in lib.cmk_last_error()
    assert lib.cmk_topk_1d_f32(fake, 10, fake, fake, 200, None, 0, None) == _lib.ERR_INVALID_ARG
    assert lib.cmk_topk_1d_f32(fake, 10, fake, fake, 5, None, 0, None) == _lib.ERR_WORKSPACE


def test_empty_problems_succeed_without_launching(lib):
    fake = ctypes.c_void_p(0x1000)
    assert lib.cmk_bmm_f32(fake, fake, fake, _desc(L=0), None) == 0
    assert lib.cmk_bmm_f32(fake, fake, fake, _desc(M=0), None) == 0
    assert lib.cmk_min_bmm_f32(fake, fake, fake, fake, _desc(M=0), 2, 0, None, 0, None) == 0
    assert lib.cmk_topk_bmm_f32(fake, fake, fake, fake, _desc(L=0), 2, 5, 0, None, 0, None) == 0


def test_check_maps_codes_to_exceptions(lib):
    lib.cmk_bmm_f32(None, None, None, None, None)
    with pytest.raises(ValueError):
        _lib.check(_lib.ERR_INVALID_ARG)
    with pytest.raises(NotImplementedError):
        _lib.check(_lib.ERR_UNSUPPORTED)
    with pytest.raises(_lib.CmkError):
        _lib.check(_lib.ERR_WORKSPACE)
    _lib.check(0)
