"""Masked batched fp32 product: tiles whose block mask is zero are skipped."""
import math

import torch

from . import _common, _lib


class MBMMCUDA:
    """Drop-in for the reference's ``MBMMCUDA`` (reference mbmm.py:7-197):
    same constructor keywords and the same
    ``__call__(A, B, block_mask, thread_mask, element_mask, mode="nn")``.

    The reference class cannot be constructed as shipped (it opens a kernel
    file that does not exist, mbmm.py:18); its intended behaviour is taken from
    kernels/mbmm.cu:208-374: C = (A@B) * element_mask where the tile's
    block_mask and the 8x8 micro-tile's thread_mask are non-zero, 0 elsewhere.
    All four modes run (the reference's `_call_tt/_tn/_nt` raise
    NotImplementedError, mbmm.py:100-107, and its kernels for them are empty):
    `mode` says how A and B are stored, as the reference documents it
    (mbmm.py:163-170): "tn" takes A as [l, k, m] and computes A.T @ B, "nt" takes B
    as [l, n, k] and computes A @ B.T, "tt" both.  Operands whose strides already
    describe one of the two layouts are consumed in place.
    """

    def __init__(self, patch_m=4, patch_n=4, share_mask=False):
        assert type(share_mask) == bool
        self.patch_m = patch_m
        self.patch_n = patch_n
        self.share_mask = share_mask
        self._lib = _lib.load()

    def _call(self, A, B, block_mask, thread_mask, element_mask):
        """A [l, m, k] and B [l, k, n] as logical views with any strides."""
        _common.check_operands(A, B)
        l, m, k = A.shape
        n = B.shape[2]
        # mask checks follow reference mbmm.py:62-72
        assert block_mask.dtype == torch.uint8
        assert thread_mask.dtype == torch.uint8
        assert element_mask.dtype == torch.uint8
        lead = () if self.share_mask else (l,)
        assert tuple(block_mask.shape) == lead + (math.ceil(m / 128), math.ceil(n / 128))
        assert tuple(thread_mask.shape) == lead + (math.ceil(m / 8), math.ceil(n / 8))
        assert tuple(element_mask.shape) == lead + (m, n)
        for t in (block_mask, thread_mask, element_mask):
            assert t.device == A.device
        block_mask = block_mask.contiguous()
        thread_mask = thread_mask.contiguous()
        element_mask = element_mask.contiguous()

        C = torch.empty(l, m, n, device=A.device, dtype=A.dtype)
        if C.numel():
            A2, B2, desc = _common.make_desc(A, B)
            with torch.cuda.device(A.device):
                _lib.check(self._lib.cmk_mbmm_f32(
                    A2.data_ptr(), B2.data_ptr(), C.data_ptr(),
                    block_mask.data_ptr(), thread_mask.data_ptr(), element_mask.data_ptr(),
                    1 if self.share_mask else 0, desc, _common.stream_ptr(A.device)))
        return C

    def _call_nn(self, A, B, block_mask, thread_mask, element_mask):
        return self._call(A, B, block_mask, thread_mask, element_mask)

    def _call_tt(self, A, B, block_mask, thread_mask, element_mask):
        return self._call(A.transpose(1, 2), B.transpose(1, 2), block_mask, thread_mask, element_mask)

    def _call_tn(self, A, B, block_mask, thread_mask, element_mask):
        return self._call(A.transpose(1, 2), B, block_mask, thread_mask, element_mask)

    def _call_nt(self, A, B, block_mask, thread_mask, element_mask):
        return self._call(A, B.transpose(1, 2), block_mask, thread_mask, element_mask)

    def __call__(self, A, B, block_mask, thread_mask, element_mask, mode="nn"):
        """
        Performs C = (A @ B) masked.
        A: float32 [m, k] or [l, m, k];  B: float32 [k, n] or [l, k, n]
        element_mask: uint8 [m, n] (share_mask) or [l, m, n]
        block_mask:   uint8 [ceil(m/128), ceil(n/128)] or with leading l
        thread_mask:  uint8 [ceil(m/8), ceil(n/8)] or with leading l
        mode: {"nn", "tn", "nt", "tt"}: "t" for A means it is given as [l, k, m],
              "t" for B that it is given as [l, n, k]
        returns C: float32 [m, n] or [l, m, n]
        """
        assert len(A.shape) == len(B.shape)
        two_dimensional = A.dim() == 2 and B.dim() == 2
        if two_dimensional:
            A2, B2 = A[None], B[None]
            if not self.share_mask:
                block_mask = block_mask[None]
                thread_mask = thread_mask[None]
                element_mask = element_mask[None]
        elif A.dim() == 3 and B.dim() == 3:
            A2, B2 = A, B
        else:
            raise ValueError("shape of A and B need to be 2d or 3d")
        call = {"nn": self._call_nn, "tt": self._call_tt,
                "tn": self._call_tn, "nt": self._call_nt}[mode]
        C = call(A2, B2, block_mask, thread_mask, element_mask)
        if two_dimensional:
            C = C[0]
        return C
