"""ctypes binding of libcmk.so, the hipcc-built C-ABI library.

Takes the place of the reference's CuPy ``RawKernel`` loader
(reference custom_kernel.py:12-43): kernels are compiled ahead of time for
gfx950, device memory comes from PyTorch's allocator (the intent of
``_torch_alloc``, custom_kernel.py:17-22) and the stream handle is read at
every call instead of once at construction (custom_kernel.py:15).
"""
import ctypes
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libcmk.so")
CSRC_DIR = os.path.join(_HERE, "csrc")

ABI_VERSION = 1

OP_BMM, OP_MBMM, OP_MIN_BMM, OP_TOPK_BMM, OP_TOPK_1D, OP_MIN_BMM_L2 = range(6)
DIST_INNER, DIST_L2, DIST_L1 = range(3)
ERR_INVALID_ARG, ERR_UNSUPPORTED, ERR_WORKSPACE = -1, -2, -3

# every symbol include/cmk.h declares
EXPORTS = (
    "cmk_bmm_f32",
    "cmk_bmm_ws_f32",
    "cmk_mbmm_f32",
    "cmk_derive_masks_u8",
    "cmk_min_bmm_f32",
    "cmk_min_bmm_f32_static",
    "cmk_topk_bmm_f32",
    "cmk_topk_1d_f32",
    "cmk_workspace_bytes",
    "cmk_last_error",
    "cmk_abi_version",
)


class GemmDesc(ctypes.Structure):
    """Mirror of ``cmk_gemm_desc`` in include/cmk.h."""

    _fields_ = [
        ("L", ctypes.c_int),
        ("M", ctypes.c_int),
        ("N", ctypes.c_int),
        ("K", ctypes.c_int),
        ("transA", ctypes.c_int),
        ("transB", ctypes.c_int),
        ("lda", ctypes.c_longlong),
        ("ldb", ctypes.c_longlong),
        ("strideA", ctypes.c_longlong),
        ("strideB", ctypes.c_longlong),
    ]


class CmkError(RuntimeError):
    """A libcmk entry point returned a non-zero status."""

    def __init__(self, code, message):
        super().__init__("libcmk error %d: %s" % (code, message))
        self.code = code


_lib = None


def build(verbose=False):
    """Compile libcmk.so in-tree with hipcc for gfx950 (no GPU needed)."""
    cmd = ["make", "-C", CSRC_DIR, "-j8", "-B"]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if verbose or res.returncode != 0:
        print(res.stdout)
    if res.returncode != 0:
        raise RuntimeError("building libcmk.so failed (exit %d)" % res.returncode)
    return LIB_PATH


def load():
    """Load libcmk.so once and declare the argument types of its entry points.

    There is no fallback: without the library every operator raises.
    """
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            "libcmk.so not found at %s; build it with `make -C %s` "
            "(or custom_matmul_kernels_amd.build())" % (LIB_PATH, CSRC_DIR)
        )
    lib = ctypes.CDLL(LIB_PATH)
    p, i, sz, ll = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t, ctypes.c_longlong
    dp = ctypes.POINTER(GemmDesc)
    lib.cmk_bmm_f32.argtypes = [p, p, p, dp, p]
    lib.cmk_bmm_ws_f32.argtypes = [p, p, p, dp, p, sz, p]
    lib.cmk_mbmm_f32.argtypes = [p, p, p, p, p, p, i, dp, p]
    lib.cmk_derive_masks_u8.argtypes = [p, p, p, i, i, i, p]
    lib.cmk_min_bmm_f32.argtypes = [p, p, p, p, dp, i, i, p, sz, p]
    lib.cmk_min_bmm_f32_static.argtypes = [p, p, p, p, dp, i, i, p]
    lib.cmk_topk_bmm_f32.argtypes = [p, p, p, p, dp, i, i, i, p, sz, p]
    lib.cmk_topk_1d_f32.argtypes = [p, ll, p, p, i, p, sz, p]
    for name in ("cmk_bmm_f32", "cmk_bmm_ws_f32", "cmk_mbmm_f32", "cmk_derive_masks_u8", "cmk_min_bmm_f32", "cmk_min_bmm_f32_static",
                 "cmk_topk_bmm_f32", "cmk_topk_1d_f32"):
        getattr(lib, name).restype = i
    lib.cmk_workspace_bytes.argtypes = [i, i, i, i, i, i]
    lib.cmk_workspace_bytes.restype = sz
    lib.cmk_last_error.argtypes = []
    lib.cmk_last_error.restype = ctypes.c_char_p
    lib.cmk_abi_version.argtypes = []
    lib.cmk_abi_version.restype = i
    got = lib.cmk_abi_version()
    if got != ABI_VERSION:
        raise ImportError("libcmk.so has ABI version %d, this package needs %d" % (got, ABI_VERSION))
    _lib = lib
    return lib


def check(status):
    """Raise for a non-zero status of an entry point."""
    if status == 0:
        return
    msg = load().cmk_last_error().decode("utf-8", "replace")
    if status == ERR_UNSUPPORTED:
        raise NotImplementedError(msg)
    if status == ERR_INVALID_ARG:
        raise ValueError(msg)
    raise CmkError(status, msg)
