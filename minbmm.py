"""Import shim: ``from minbmm import MinBMMCUDA`` keeps working as with the reference
(reference minbmm.py), the class now lives in custom_matmul_kernels_amd."""
from custom_matmul_kernels_amd.minbmm import MinBMMCUDA  # noqa: F401
