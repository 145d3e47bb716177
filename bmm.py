"""Import shim: ``from bmm import BMMCUDA`` keeps working as with the reference
(reference bmm.py), the class now lives in custom_matmul_kernels_amd."""
from custom_matmul_kernels_amd.bmm import BMMCUDA  # noqa: F401
