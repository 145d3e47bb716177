"""The three mask levels MBMMCUDA takes, derived on the GPU from one boolean
mask by libcmk's ``cmk_derive_masks_u8``: the element mask is the mask itself,
the thread mask counts kept elements per 8x8 micro-tile (0..64) and the block
mask flags 128x128 tiles with any kept element -- the rule callers of the
reference apply with tensor reductions (reference
colab/test_mbmm.ipynb:1295-1313).  Extents that are not multiples of 8 / 128
are padded with zeros (the notebook only handles multiples)."""
import math

import torch

from . import _lib


def derive_masks(final_mask):
    """final_mask: bool or uint8 device tensor [m, n] or [l, m, n] ->
    (block_mask, thread_mask, element_mask), all uint8 on the same device, in
    the argument order of MBMMCUDA.__call__.  A bool mask is reinterpreted, not
    copied; a uint8 mask is used as given (any non-zero byte counts as kept,
    and the product is multiplied by the byte, as reference
    kernels/mbmm.cu:127-128 does)."""
    if final_mask.dtype not in (torch.bool, torch.uint8):
        raise TypeError("the mask must be torch.bool or torch.uint8, got %s" % final_mask.dtype)
    if final_mask.dim() not in (2, 3):
        raise ValueError("the mask needs to be 2d or 3d")
    if final_mask.device.type != "cuda":
        raise ValueError("the mask must be a device tensor (got device %s)" % final_mask.device)
    lib = _lib.load()
    em = final_mask.contiguous()
    if em.dtype == torch.bool:
        em = em.view(torch.uint8)
    squeeze = em.dim() == 2
    e3 = em[None] if squeeze else em
    l, m, n = e3.shape
    dev = em.device
    block_mask = torch.empty((l, math.ceil(m / 128), math.ceil(n / 128)), dtype=torch.uint8, device=dev)
    thread_mask = torch.empty((l, math.ceil(m / 8), math.ceil(n / 8)), dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        stream = torch.cuda.current_stream(dev).cuda_stream
        _lib.check(lib.cmk_derive_masks_u8(e3.data_ptr(), block_mask.data_ptr(), thread_mask.data_ptr(),
                                           l, m, n, stream))
    if squeeze:
        return block_mask[0], thread_mask[0], em
    return block_mask, thread_mask, em
