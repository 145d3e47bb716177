"""MI355X (gfx950) fused batched-matmul family: bmm, mbmm, min_bmm, topk_bmm.

The operator classes keep the call surface of DeMoriarty/custom_matmul_kernels;
the kernels are hand-written HIP behind a C ABI (include/cmk.h) loaded with
ctypes."""
from ._lib import build, load, LIB_PATH, CmkError
from .bmm import BMMCUDA
from .mbmm import MBMMCUDA
from .minbmm import MinBMMCUDA
from .topkbmm import TopkBMMCUDA, BitonicSort
from .masks import derive_masks

__all__ = ["BMMCUDA", "MBMMCUDA", "MinBMMCUDA", "TopkBMMCUDA", "BitonicSort",
           "derive_masks", "build", "load", "LIB_PATH", "CmkError"]
