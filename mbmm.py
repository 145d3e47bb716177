"""Import shim: ``from mbmm import MBMMCUDA`` keeps working as with the reference
(reference mbmm.py), the class now lives in custom_matmul_kernels_amd."""
from custom_matmul_kernels_amd.mbmm import MBMMCUDA  # noqa: F401
