"""CPU oracle for the fused batched-matmul family.  TEST INFRASTRUCTURE ONLY:
imported by tests/, by the smoke run and by the CPU-baseline leg of bench.py as
the checker; the product package never imports it.

Two layers:

* ``c_*`` functions call oracle/cmk_oracle.c (built into
  oracle/_build/liboracle.so), a restatement of the reference's algorithms:
  sequential fp32 FMA accumulation, mask precedence, first-index argmin and the
  128-wide bitonic sort / merge network.
* ``ref_*`` functions are the reference's *semantics* as its notebooks state
  them - ``torch.bmm`` followed by ``masked_fill`` / ``min`` / ``topk`` on the
  CPU (reference colab/test_bmm.ipynb:2121, colab/test_mbmm.ipynb:1342-1343,
  colab/test_minbmm.ipynb:2131-2132, colab/test_topkbmm.ipynb:2673-2677) -
  chunked over rows so that large products never exist in memory.

``check_*`` functions compare a result with the oracle under the parity rule:
values within rtol 1e-4 / atol 1e-3*sqrt(K); indices equal, or pointing at a
product value within that tolerance of the oracle's.
"""
import ctypes
import math
import os
import subprocess

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "liboracle.so")
_clib = None

RTOL = 1e-4


def atol_for(K):
    return 1e-3 * math.sqrt(max(K, 1))


class _Desc(ctypes.Structure):
    _fields_ = [("L", ctypes.c_int), ("M", ctypes.c_int), ("N", ctypes.c_int), ("K", ctypes.c_int),
                ("transA", ctypes.c_int), ("transB", ctypes.c_int),
                ("lda", ctypes.c_longlong), ("ldb", ctypes.c_longlong),
                ("strideA", ctypes.c_longlong), ("strideB", ctypes.c_longlong)]


def build():
    subprocess.run(["make", "-C", _HERE, "-B"], check=True, stdout=subprocess.DEVNULL)
    return _SO


def clib():
    global _clib
    if _clib is None:
        if not os.path.exists(_SO):
            build()
        _clib = ctypes.CDLL(_SO)
    return _clib


def _f32(a):
    return np.ascontiguousarray(np.asarray(a, dtype=np.float32))


def _ptr(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _desc(A, B):
    """A [L,M,K], B [L,K,N] as C-contiguous numpy arrays ("nn")."""
    L, M, K = A.shape
    N = B.shape[2]
    return _Desc(L, M, N, K, 0, 0, K, N, M * K, K * N)


def c_bmm(A, B):
    A, B = _f32(A), _f32(B)
    d = _desc(A, B)
    C = np.empty((d.L, d.M, d.N), np.float32)
    clib().orc_bmm(_ptr(A), _ptr(B), _ptr(C), ctypes.byref(d))
    return C


def c_mbmm(A, B, block_mask, thread_mask, element_mask, share_mask):
    A, B = _f32(A), _f32(B)
    d = _desc(A, B)
    bm = np.ascontiguousarray(block_mask, dtype=np.uint8)
    tm = np.ascontiguousarray(thread_mask, dtype=np.uint8)
    em = np.ascontiguousarray(element_mask, dtype=np.uint8)
    C = np.empty((d.L, d.M, d.N), np.float32)
    clib().orc_mbmm(_ptr(A), _ptr(B), _ptr(C), _ptr(bm), _ptr(tm), _ptr(em),
                    1 if share_mask else 0, ctypes.byref(d))
    return C


def c_min_bmm(A, B, dim, distance=0):
    A, B = _f32(A), _f32(B)
    d = _desc(A, B)
    kept = d.N if dim == 1 else d.M
    v = np.empty((d.L, kept), np.float32)
    i = np.empty((d.L, kept), np.int64)
    clib().orc_min_bmm(_ptr(A), _ptr(B), _ptr(v), _ptr(i), ctypes.byref(d), dim, distance)
    return v, i


def c_topk_bmm(A, B, k, dim, distance=0):
    A, B = _f32(A), _f32(B)
    d = _desc(A, B)
    kept = d.N if dim == 1 else d.M
    v = np.empty((d.L, kept, k), np.float32)
    i = np.empty((d.L, kept, k), np.int64)
    clib().orc_topk_bmm(_ptr(A), _ptr(B), _ptr(v), _ptr(i), ctypes.byref(d), dim, k, distance)
    return v, i


def c_bitonic_sort_128(values, indices):
    v = _f32(values).copy()
    i = np.ascontiguousarray(indices, dtype=np.int64).copy()
    assert v.shape == (128,) and i.shape == (128,)
    clib().orc_bitonic_sort_128(_ptr(v), _ptr(i))
    return v, i


def c_topk_1d(arr, k):
    a = _f32(arr)
    v = np.empty((k,), np.float32)
    i = np.empty((k,), np.int64)
    clib().orc_topk_1d(_ptr(a), ctypes.c_longlong(a.shape[0]), _ptr(v), _ptr(i), k)
    return v, i


# ---- reference semantics with PyTorch on the CPU ---------------------------

def ref_bmm(A, B):
    return torch.bmm(A, B)


def ref_derive_masks(final_mask):
    """(block_mask, thread_mask, element_mask), uint8, from a bool mask [m, n] or
    [l, m, n]: counts per 8x8 micro-tile and any-kept flags per 128x128 tile, as
    reference colab/test_mbmm.ipynb:1295-1313 forms them, with zero padding for
    extents that are not multiples of 8 / 128."""
    fm = final_mask != 0
    squeeze = fm.dim() == 2
    if squeeze:
        fm = fm[None]
    l, m, n = fm.shape
    m8, n8 = math.ceil(m / 8), math.ceil(n / 8)
    m128, n128 = math.ceil(m / 128), math.ceil(n / 128)
    u = fm.to(torch.uint8)
    pad = torch.nn.functional.pad
    p8 = pad(u, (0, n8 * 8 - n, 0, m8 * 8 - m))
    thread_mask = p8.view(l, m8, 8, n8, 8).sum(dim=(2, 4), dtype=torch.int32).to(torch.uint8)
    p128 = pad(u, (0, n128 * 128 - n, 0, m128 * 128 - m))
    block_mask = (p128.view(l, m128, 128, n128, 128).sum(dim=(2, 4), dtype=torch.int32) > 0).to(torch.uint8)
    element_mask = (final_mask.to(torch.uint8) if final_mask.dtype == torch.bool else final_mask).contiguous()
    if squeeze:
        return block_mask[0], thread_mask[0], element_mask
    return block_mask, thread_mask, element_mask


def ref_mbmm(A, B, final_mask):
    """final_mask: bool, True = keep (colab/test_mbmm.ipynb:1342-1343)."""
    C = torch.bmm(A, B)
    return C.masked_fill_(~final_mask, 0)


def ref_min_bmm(A, B, dim, chunk=4096):
    """min/argmin of A@B along axis `dim` of C[l,m,n], chunked over kept rows."""
    if dim == 1:
        A, B = B.transpose(1, 2), A.transpose(1, 2)   # C^T = B^T A^T, reduce over its last axis
    kept = A.shape[1]
    vals, idxs = [], []
    for r0 in range(0, kept, chunk):
        v, i = torch.bmm(A[:, r0:r0 + chunk], B).min(dim=-1)
        vals.append(v)
        idxs.append(i)
    return torch.cat(vals, 1), torch.cat(idxs, 1)


def ref_topk_bmm(A, B, k, dim, chunk=65536):
    """k largest of A@B along axis `dim`, sorted descending; dim == 1 results are
    laid out [l, n, k] (colab/test_topkbmm.ipynb:2673-2677)."""
    if dim == 1:
        A, B = B.transpose(1, 2), A.transpose(1, 2)
    kept = A.shape[1]
    vals, idxs = [], []
    for r0 in range(0, kept, chunk):
        v, i = torch.bmm(A[:, r0:r0 + chunk], B).topk(k, dim=-1)
        vals.append(v)
        idxs.append(i)
    return torch.cat(vals, 1), torch.cat(idxs, 1)


# ---- comparators ------------------------------------------------------------

def check_values(got, want, K, what="values"):
    got = torch.as_tensor(got).double()
    want = torch.as_tensor(want).double()
    assert got.shape == want.shape, "%s: shape %s vs %s" % (what, tuple(got.shape), tuple(want.shape))
    same_inf = torch.isinf(want) & (got == want)
    err = (got - want).abs()
    tol = atol_for(K) + RTOL * want.abs()
    bad = ~((err <= tol) | same_inf)
    if bad.any():
        w = bad.nonzero()[0].tolist()
        raise AssertionError("%s: %d of %d outside tolerance, first at %s: got %r want %r" % (
            what, int(bad.sum()), bad.numel(), w, got[tuple(w)].item(), want[tuple(w)].item()))


def gather_products(A, B, dim, indices):
    """C[l, y, indices[l, y, ...]] recomputed in float64 without forming C.
    A [l,m,k], B [l,k,n] CPU tensors; indices [l, kept] or [l, kept, q]."""
    if dim == 1:
        A, B = B.transpose(1, 2), A.transpose(1, 2)
    idx = indices if indices.dim() == 3 else indices[..., None]
    l, kept, q = idx.shape
    out = torch.empty(l, kept, q, dtype=torch.float64)
    safe = idx.clamp(min=0)
    step = max(1, (1 << 24) // max(1, q * A.shape[2]))
    bt = B.transpose(1, 2)                                       # [l, X, K]
    for r0 in range(0, kept, step):
        a = A[:, r0:r0 + step].double()                          # [l, r, K]
        # only the gathered columns are widened, never the whole operand
        sel = torch.stack([bt[b][safe[b, r0:r0 + step]] for b in range(l)]).double()  # [l, r, q, K]
        out[:, r0:r0 + step] = (a[:, :, None, :] * sel).sum(-1)
    return out if indices.dim() == 3 else out[..., 0]


def check_min(values, indices, A, B, dim, ref=None):
    """values/indices from the device (any device) against the oracle."""
    K = A.shape[2]
    values = values.cpu()
    indices = indices.cpu()
    rv, ri = ref if ref is not None else ref_min_bmm(A, B, dim)
    check_values(values, rv, K, "min values")
    red = A.shape[1] if dim == 1 else B.shape[2]
    assert indices.dtype == torch.int64
    assert ((indices >= 0) & (indices < red)).all(), "min indices out of range"
    diff = indices != ri
    if diff.any():
        # allowed only where the competing products are closer than the tolerance
        at_got = gather_products(A, B, dim, indices)
        gap = (at_got - rv.double()).abs()
        tol = atol_for(K) + RTOL * rv.double().abs()
        bad = diff & (gap > tol)
        assert not bad.any(), "min indices: %d mismatches beyond tolerance" % int(bad.sum())
    return int(diff.sum())


def check_topk(values, indices, A, B, k, dim, ref=None):
    K = A.shape[2]
    values = values.cpu()
    indices = indices.cpu()
    red = A.shape[1] if dim == 1 else B.shape[2]
    kk = min(k, red)
    rv, ri = ref if ref is not None else ref_topk_bmm(A, B, kk, dim)
    assert values.shape[-1] == k and indices.shape[-1] == k
    assert indices.dtype == torch.int64
    if kk < k:
        assert torch.isinf(values[..., kk:]).all() and (values[..., kk:] < 0).all()
        assert (indices[..., kk:] == -1).all()
    v, i = values[..., :kk], indices[..., :kk]
    check_values(v, rv, K, "topk values")
    assert (v[..., :-1] >= v[..., 1:]).all(), "topk values not sorted descending"
    assert ((i >= 0) & (i < red)).all(), "topk indices out of range"
    s = i.sort(dim=-1).values
    assert (s[..., 1:] != s[..., :-1]).all(), "topk indices repeat within a row"
    # every reported value is the product at its index
    at_got = gather_products(A, B, dim, i)
    check_values(v, at_got, K, "topk value-at-index")
    diff = i != ri
    if diff.any():
        gap = (at_got - rv.double()).abs()
        tol = atol_for(K) + RTOL * rv.double().abs()
        bad = diff & (gap > tol)
        assert not bad.any(), "topk indices: %d mismatches beyond tolerance" % int(bad.sum())
    return int(diff.sum())
