"""Fused min / argmin of a batched fp32 product along one axis."""
import torch

from . import _common, _lib


# Squared l2 goes through the matrix pipe (screening there, exact evaluation of
# the surviving candidates, bit-equal results) from this many multiply-adds
# L*m*n*k on; below, the extra launches cost more than the vector route saves.
# Measured on MI355X: the screening route takes 0.034 ms at least, the vector
# route 0.025 ms at k = 16 and 0.042 ms at k = 64 for 2^26 multiply-adds.
L2_SCREEN_MIN_WORK = 1 << 26


def screens_l2(l, m, n, k):
    """Whether MinBMMCUDA(distance="l2") takes the matrix pipe for this shape."""
    work = l * m * n * k
    return work >= L2_SCREEN_MIN_WORK and (k >= 48 or work >= 4 * L2_SCREEN_MIN_WORK)


class MinBMMCUDA:
    """Drop-in for the reference's ``MinBMMCUDA`` (reference minbmm.py:7-148):
    same constructor keywords, same ``__call__(A, B, dim=1)`` returning
    ``(values, indices)``.

    `dim` is an axis of A@B as the reference counts it (for 3-D inputs 1 reduces
    over m, 2 over n; for 2-D inputs 0 and 1); negative dims are accepted as
    well.  Every output element is written, ties resolve to the lowest index
    (the reference's index write is racy, kernels/minbmm.cu:76-79), and an
    unknown `distance` raises (the reference only builds the exception,
    minbmm.py:19).
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

    def __call__(self, A, B, dim=1):
        A, B, two_dimensional = _common.promote(A, B)
        dim = _common.normalize_dim(dim, two_dimensional)
        _common.check_operands(A, B)
        l, m, k = A.shape
        n = B.shape[2]
        kept, reduced = (n, m) if dim == 1 else (m, n)
        if reduced == 0:
            raise ValueError("min_bmm: cannot reduce over an axis of extent 0")
        values = torch.empty([l, kept], device=A.device, dtype=A.dtype)
        indices = torch.empty([l, kept], device=A.device, dtype=torch.int64)
        if values.numel():
            A2, B2, desc = _common.make_desc(A, B)
            op = _lib.OP_MIN_BMM
            if self._distance == _lib.DIST_L2 and screens_l2(l, m, n, k):
                op = _lib.OP_MIN_BMM_L2
            ws, ws_bytes = _common.workspace(op, l, m, n, k, dim, A.device)
            if op == _lib.OP_MIN_BMM_L2 and ws is None:   # shape outside the screening route
                ws, ws_bytes = _common.workspace(_lib.OP_MIN_BMM, l, m, n, k, dim, A.device)
            with torch.cuda.device(A.device):
                _lib.check(self._lib.cmk_min_bmm_f32(
                    A2.data_ptr(), B2.data_ptr(), values.data_ptr(), indices.data_ptr(), desc,
                    dim, self._distance, ws.data_ptr() if ws is not None else None, ws_bytes,
                    _common.stream_ptr(A.device)))
        if two_dimensional:
            indices = indices[0]
            values = values[0]
        return values, indices
