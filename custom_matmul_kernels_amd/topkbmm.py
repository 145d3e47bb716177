"""Fused sorted top-k of a batched fp32 product along one axis."""
import torch

from . import _common, _lib


# The vector-unit distance kernels of top-k run 40 % faster when the operand of
# the reduced axis is stored with that axis contiguous (its points are then LDS
# columns that a half-wave reads as broadcasts without extra address registers;
# the other form spills at the kernel's 128 registers per lane).  From this many
# multiply-adds on, an operand stored the other way is copied once: the copy
# moves the operand, the kernel does l*m*n*k vector operations on it.
DIST_RELAYOUT_MIN_WORK = 1 << 24


def _reduced_axis_contiguous(A, B, dim):
    """A[l,m,k], B[l,k,n] with the operand of the reduced axis (A for dim 1, B for
    dim 2) stored with that axis contiguous; same values, other strides.  (Copying
    the other, larger operand into its preferred form as well costs more than the
    10 % it gives.)"""
    if dim == 1 and A.stride(-1) == 1 and A.stride(-2) != 1:
        A = A.transpose(1, 2).contiguous().transpose(1, 2)
    elif dim == 2 and B.stride(-2) == 1 and B.stride(-1) != 1:
        B = B.contiguous()
    return A, B


class TopkBMMCUDA:
    """Drop-in for the reference's ``TopkBMMCUDA`` (reference topkbmm.py:7-156):
    same constructor keywords, same ``__call__(A, B, k=128, dim=1)`` returning
    ``(values, indices)``, the k largest entries of A@B along `dim`, sorted
    descending; ``0 < k <= 128``.

    `dim` counts axes of A@B as in the reference (3-D: 1 = over m, result
    [l, n, k]; 2 = over n, result [l, m, k]); negative dims are accepted too.
    Any m and n work (the reference needs multiples of 128,
    colab/test_topkbmm.ipynb:2620-2623); when fewer than k candidates exist the
    trailing slots hold -inf / -1.
    """

    def __init__(self, patch_m=4, patch_n=4, distance="inner"):
        self.patch_m = patch_m
        self.patch_n = patch_n
        self._distance = _common.distance_code(distance)
        self.distance = distance
        self._lib = _lib.load()

    def get_mode(self, A, B):
        a, b = _common.get_mode(A, B)
        return "".join([a or "n", b or "n"])

    def __call__(self, A, B, k=128, dim=1):
        A, B, two_dimensional = _common.promote(A, B)
        dim = _common.normalize_dim(dim, two_dimensional)
        _common.check_operands(A, B)
        assert 0 < k <= 128
        l, m, d = A.shape
        n = B.shape[2]
        kept = n if dim == 1 else m
        values = torch.empty([l, kept, k], device=A.device, dtype=A.dtype)
        indices = torch.empty([l, kept, k], device=A.device, dtype=torch.int64)
        if values.numel():
            if self._distance != _lib.DIST_INNER and l * m * n * d >= DIST_RELAYOUT_MIN_WORK:
                A, B = _reduced_axis_contiguous(A, B, dim)
            A2, B2, desc = _common.make_desc(A, B)
            ws, ws_bytes = _common.workspace(_lib.OP_TOPK_BMM, l, m, n, d, dim, A.device)
            with torch.cuda.device(A.device):
                _lib.check(self._lib.cmk_topk_bmm_f32(
                    A2.data_ptr(), B2.data_ptr(), values.data_ptr(), indices.data_ptr(), desc,
                    dim, k, self._distance, ws.data_ptr() if ws is not None else None, ws_bytes,
                    _common.stream_ptr(A.device)))
        if two_dimensional:
            indices = indices[0]
            values = values[0]
        return values, indices


class BitonicSort:
    """Top-k (largest, sorted descending, k <= 128) of a 1-D fp32 tensor; the
    counterpart of the notebook class around the reference's standalone
    ``bitonic_sort`` kernel (colab/test_topkbmm.ipynb:1027-1069,
    kernels/bitonic_sort.cu:182-216)."""

    def __init__(self):
        self._lib = _lib.load()

    def __call__(self, arr, k=128):
        assert arr.dim() == 1
        assert 0 < k <= 128
        if arr.dtype != torch.float32:
            raise TypeError("only torch.float32 is supported, got %s" % arr.dtype)
        assert arr.device.type == "cuda"
        arr = arr.contiguous()
        values = torch.empty([k], device=arr.device, dtype=arr.dtype)
        indices = torch.empty([k], device=arr.device, dtype=torch.int64)
        ws, ws_bytes = _common.workspace(_lib.OP_TOPK_1D, 1, arr.numel(), 0, 0, 0, arr.device)
        with torch.cuda.device(arr.device):
            _lib.check(self._lib.cmk_topk_1d_f32(
                arr.data_ptr(), arr.numel(), values.data_ptr(), indices.data_ptr(), k,
                ws.data_ptr() if ws is not None else None, ws_bytes,
                _common.stream_ptr(arr.device)))
        return values, indices
