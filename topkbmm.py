"""Import shim: ``from topkbmm import TopkBMMCUDA`` keeps working as with the reference
(reference topkbmm.py), the class now lives in custom_matmul_kernels_amd."""
from custom_matmul_kernels_amd.topkbmm import TopkBMMCUDA  # noqa: F401
