"""Derivation of the three mask levels MBMMCUDA takes from one boolean mask,
following colab/test_mbmm.ipynb:1295-1313 of the reference: the element mask is
the mask itself, the thread mask counts kept elements per 8x8 micro-tile
(0..64) and the block mask flags 128x128 tiles with any kept element.  Extents
that are not multiples of 8 / 128 are padded with zeros (the notebook only
handles multiples)."""
import math

import torch
import torch.nn.functional as F


def derive_masks(final_mask):
    """final_mask: bool [m, n] or [l, m, n] -> (block_mask, thread_mask,
    element_mask), all uint8, in the argument order of MBMMCUDA.__call__."""
    fm = final_mask.bool()
    squeeze = fm.dim() == 2
    if squeeze:
        fm = fm[None]
    l, m, n = fm.shape
    m8, n8 = math.ceil(m / 8), math.ceil(n / 8)
    m128, n128 = math.ceil(m / 128), math.ceil(n / 128)
    u = fm.to(torch.uint8)
    p8 = F.pad(u, (0, n8 * 8 - n, 0, m8 * 8 - m))
    thread_mask = p8.view(l, m8, 8, n8, 8).sum(dim=(2, 4), dtype=torch.int32).to(torch.uint8)
    p128 = F.pad(u, (0, n128 * 128 - n, 0, m128 * 128 - m))
    block_mask = (p128.view(l, m128, 128, n128, 128).sum(dim=(2, 4), dtype=torch.int32) > 0)
    block_mask = block_mask.to(torch.uint8)
    element_mask = u.contiguous()
    if squeeze:
        return block_mask[0], thread_mask[0], element_mask[0]
    return block_mask, thread_mask, element_mask
