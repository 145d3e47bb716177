"""The allocation-free min_bmm entry point (static device scratch) gives the
same bits as the entry point that takes a caller workspace: two calls in a row
through the C ABI, the second on a smaller problem, so that whatever the first
call left in the shared scratch array must not leak into the second."""
import ctypes

import pytest
import torch

from custom_matmul_kernels_amd import _lib
from _cases import seeded

pytestmark = pytest.mark.gpu

STATIC_SCRATCH_BYTES = 4 << 20


def _desc(A, B):
    l, m, k = A.shape
    n = B.shape[2]
    return _lib.GemmDesc(l, m, n, k, 0, 0, k, n, m * k, k * n)


def _run(lib, A, B, dim, static, distance=0):
    """One min_bmm through the C ABI; returns (values, indices)."""
    d = _desc(A, B)
    kept = d.N if dim == 1 else d.M
    values = torch.full([d.L, kept], float("nan"), device=A.device)
    indices = torch.full([d.L, kept], -7, device=A.device, dtype=torch.int64)
    stream = torch.cuda.current_stream(A.device).cuda_stream
    if static:
        _lib.check(lib.cmk_min_bmm_f32_static(A.data_ptr(), B.data_ptr(), values.data_ptr(),
                                              indices.data_ptr(), d, dim, distance, stream))
    else:
        need = lib.cmk_workspace_bytes(_lib.OP_MIN_BMM, d.L, d.M, d.N, d.K, dim)
        ws = torch.empty(max(need, 1), dtype=torch.uint8, device=A.device)
        _lib.check(lib.cmk_min_bmm_f32(A.data_ptr(), B.data_ptr(), values.data_ptr(), indices.data_ptr(),
                                       d, dim, distance, ws.data_ptr(), need, stream))
    torch.cuda.synchronize()
    return values, indices


def test_static_scratch_entry_point_matches_workspace_entry_point(device):
    lib = _lib.load()
    # both shapes split the reduced axis (few strips of kept rows), so both use scratch
    shapes = [(1, 4096, 4096, 64, 2), (2, 300, 1500, 48, 2), (1, 2000, 130, 40, 1)]
    for L, M, N, K, dim in shapes:
        print("static scratch", (L, M, N, K), dim, flush=True)
        assert 0 < lib.cmk_workspace_bytes(_lib.OP_MIN_BMM, L, M, N, K, dim) <= STATIC_SCRATCH_BYTES
        A, B = seeded(L, M, N, K, seed=40 + M)
        Ad, Bd = A.to(device), B.to(device)
        want_v, want_i = _run(lib, Ad, Bd, dim, static=False)
        got_v, got_i = _run(lib, Ad, Bd, dim, static=True)
        assert torch.equal(got_v, want_v) and torch.equal(got_i, want_i)
    # a problem that needs no scratch at all goes through as well
    assert lib.cmk_workspace_bytes(_lib.OP_MIN_BMM, 8, 16384, 256, 32, 2) == 0
    A, B = seeded(8, 16384, 256, 32, seed=3)
    Ad, Bd = A.to(device), B.to(device)
    want = _run(lib, Ad, Bd, 2, static=False)
    got = _run(lib, Ad, Bd, 2, static=True)
    assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])


def test_static_scratch_entry_point_refuses_what_does_not_fit(device):
    lib = _lib.load()
    # 262144 kept rows whose reduction is cut in four: 8 MiB of partials; nothing is launched
    d = _lib.GemmDesc(1, 262144, 65536, 256, 0, 0, 256, 65536, 262144 * 256, 256 * 65536)
    need = lib.cmk_workspace_bytes(_lib.OP_MIN_BMM, d.L, d.M, d.N, d.K, 2)
    assert need > STATIC_SCRATCH_BYTES
    fake = ctypes.c_void_p(0x1000)
    assert lib.cmk_min_bmm_f32_static(fake, fake, fake, fake, d, 2, 0, None) == _lib.ERR_WORKSPACE
    assert b"static" in lib.cmk_last_error()


def test_static_scratch_entry_point_replays_in_a_hip_graph(device):
    """After one call outside a capture (the first call on a device looks up the
    scratch array's address, which is not a stream operation) the entry point is
    kernel launches only: captured once, every replay with new inputs matches the
    eager workspace entry point."""
    lib = _lib.load()
    L, M, N, K, dim = 1, 2048, 4096, 64, 2
    assert 0 < lib.cmk_workspace_bytes(_lib.OP_MIN_BMM, L, M, N, K, dim) <= STATIC_SCRATCH_BYTES
    print("static scratch under graph capture", (L, M, N, K), flush=True)
    A, B = seeded(L, M, N, K, seed=77)
    Ad, Bd = A.to(device), B.to(device)
    d = _desc(Ad, Bd)
    values = torch.empty([L, M], device=device)
    indices = torch.empty([L, M], device=device, dtype=torch.int64)

    def enqueue():
        stream = torch.cuda.current_stream(device).cuda_stream
        _lib.check(lib.cmk_min_bmm_f32_static(Ad.data_ptr(), Bd.data_ptr(), values.data_ptr(),
                                              indices.data_ptr(), d, dim, 0, stream))

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        enqueue()                                       # the warm-up call, outside the capture
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        enqueue()
    gen = torch.Generator().manual_seed(5)
    for step in range(3):
        Ad.copy_(torch.randn(L, M, K, generator=gen))
        Bd.copy_(torch.randn(L, K, N, generator=gen))
        graph.replay()
        torch.cuda.synchronize()
        got_v, got_i = values.clone(), indices.clone()
        want_v, want_i = _run(lib, Ad, Bd, dim, static=False)   # eager, between the replays
        assert torch.equal(got_v, want_v) and torch.equal(got_i, want_i), "replay %d differs" % step
