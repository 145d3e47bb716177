"""Host logic shared by the four operator classes: layout inference from
strides, promotion of 2-D inputs to a batch of one, argument checks and the
translation of a pair of tensors into a ``cmk_gemm_desc``."""
import torch

from . import _lib


def get_mode(A, B):
    """Layout letters of A[l,m,k] and B[l,k,n] as the reference infers them
    from strides (reference bmm.py:56-66): "n" when the last axis is
    contiguous, "t" when the second-to-last is, None otherwise."""
    mode = []
    for T in (A, B):
        if T.stride()[-1] == 1:
            mode.append("n")
        elif T.stride()[-2] == 1:
            mode.append("t")
        else:
            mode.append(None)
    return mode


def promote(A, B):
    """2-D operands become a batch of one (reference bmm.py:78-88)."""
    assert len(A.shape) == len(B.shape)
    if A.dim() == 2 and B.dim() == 2:
        return A[None], B[None], True
    if A.dim() == 3 and B.dim() == 3:
        return A, B, False
    raise ValueError("A and B need to be 2d or 3d")


def check_operands(A, B):
    """The reference's asserts (bmm.py:85-90) except that half precision,
    which its kernels silently misread as float, is rejected."""
    assert A.shape[0] == B.shape[0]
    assert A.shape[2] == B.shape[1]
    assert A.dtype == B.dtype
    if A.dtype != torch.float32:
        raise TypeError("only torch.float32 operands are supported, got %s" % A.dtype)
    assert A.device.type == B.device.type == "cuda"
    assert A.device == B.device


def _operand(T, want_inner, name):
    """Returns (tensor, trans, ld, batch_stride) for one [l, r, c] operand.
    A tensor whose strides fit neither layout is copied to row-major."""
    l, r, c = T.shape
    s0, s1, s2 = T.stride()
    # an axis of extent 1 can carry any stride; treat it as the natural one
    if (s2 == 1 or c == 1) and (s1 >= c or r == 1):
        ld = s1 if r > 1 else max(c, 1)
        return T, 0, max(ld, c, 1), (s0 if l > 1 else 0)
    if (s1 == 1 or r == 1) and (s2 >= r or c == 1):
        ld = s2 if c > 1 else max(r, 1)
        return T, 1, max(ld, r, 1), (s0 if l > 1 else 0)
    Tc = T.contiguous()
    return Tc, 0, max(c, 1), r * c


# An operand that is not 16-byte aligned (base, leading dimension or batch
# stride) cannot use the kernels' direct global-to-LDS loads at all and runs
# about three times slower; between these sizes (elements) a padded copy costs
# far less than that and does not double a footprint that matters.
ALIGN_COPY_MIN = 1 << 16
ALIGN_COPY_MAX = 1 << 28


def _aligned(T, trans, ld, stride):
    """The operand itself when the kernels can fetch it with 16-byte loads (or
    when a copy is not worth it), otherwise a copy whose rows are padded to a
    multiple of four elements; the padding is never read.  An operand that all
    batches share (batch stride 0, e.g. an expanded view) is copied once and
    keeps its stride of 0; the size window is about what is physically there."""
    l, r, c = T.shape
    shared = stride == 0 and l > 1
    physical = r * c if shared else T.numel()
    if (T.data_ptr() % 16 == 0 and ld % 4 == 0 and stride % 4 == 0) or \
            not ALIGN_COPY_MIN <= physical <= ALIGN_COPY_MAX:
        return T, trans, ld, stride
    src = T[:1] if shared else T
    inner, outer = (c, r) if trans == 0 else (r, c)
    ldp = (inner + 3) // 4 * 4
    buf = torch.empty(src.shape[0], outer, ldp, dtype=T.dtype, device=T.device)
    if trans == 0:
        view = buf[..., :c]
        view.copy_(src)
    else:
        view = buf[..., :r].transpose(1, 2)
        view.copy_(src)
    if shared:
        return view.expand(l, r, c), trans, ldp, 0
    return view, trans, ldp, outer * ldp


def make_desc(A, B):
    """Builds the descriptor for C = A @ B with A [l,m,k], B [l,k,n].  The
    returned tensors must stay alive until the launch has been enqueued."""
    l, m, k = A.shape
    _, _, n = B.shape
    A2, tA, lda, sA = _operand(A, k, "A")
    B2, tB, ldb, sB = _operand(B, n, "B")
    if sA < 0 or sB < 0:
        A2, tA, lda, sA = A.contiguous(), 0, max(k, 1), m * k
        B2, tB, ldb, sB = B.contiguous(), 0, max(n, 1), k * n
    A2, tA, lda, sA = _aligned(A2, tA, lda, sA)
    B2, tB, ldb, sB = _aligned(B2, tB, ldb, sB)
    # the descriptor's trans flag for A is about [m,k] storage, for B about [k,n]
    d = _lib.GemmDesc(l, m, n, k, tA, tB, lda, ldb, sA, sB)
    return A2, B2, d


def stream_ptr(device):
    """The HIP stream PyTorch currently uses on `device`, read at every call."""
    return torch.cuda.current_stream(device).cuda_stream


def workspace(op, l, m, n, k, dim, device):
    lib = _lib.load()
    nbytes = lib.cmk_workspace_bytes(op, l, m, n, k, dim)
    if nbytes == 0:
        return None, 0
    return torch.empty(nbytes, dtype=torch.uint8, device=device), nbytes


def normalize_dim(dim, two_dimensional):
    """Maps `dim` to an axis of C[l,m,n]: 1 = over m, 2 = over n.  For 2-D
    inputs the reference adds one (minbmm.py:86-90); negative dims, which the
    reference rejects (minbmm.py:100), count from the end."""
    if dim < 0:
        dim += 3
    elif two_dimensional:
        dim += 1
    assert dim in [1, 2]
    return dim


DISTANCES = {
    "inner": _lib.DIST_INNER,
    "l2": _lib.DIST_L2,
    "euclidean": _lib.DIST_L2,
    "l1": _lib.DIST_L1,
    "manhattan": _lib.DIST_L1,
}


def distance_code(distance):
    """The reference builds a ValueError for an unknown distance but never
    raises it (minbmm.py:19); here it is raised."""
    try:
        return DISTANCES[distance]
    except KeyError:
        raise ValueError("Unrecognized distance type") from None
