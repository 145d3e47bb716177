"""Benchmark of the fused batched-matmul path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-others] [--no-cpu]

One step = one pass of the hot path over one synthetic batch that is already
resident in HBM.  The headline workload is the large fused min_bmm
(A[1,65536,256] @ B[1,256,65536], min/argmin over dim=-1, product never
stored).  The JSON line carries, for the headline and for every other
workload: the throughput, the roofline fraction of the dominant kernel, a
parity verdict against the CPU oracle computed in the same run on a sample of
the output (outside the timed region), and - for the five benchmark
configurations - the same semantics timed with PyTorch on the host CPU.

Inputs are drawn on the CPU from torch.Generator().manual_seed(0), A before B
(masks from seed 1), and copied to the device, so that the GPU and the CPU
legs see the same bits.

Timing: W warm-up steps, then exactly K steps between two synchronisations;
`ms_per_step` is the wall clock of that region / K, `kernel_ms` the time
between two events recorded on the launch stream around the same region / K
(the average duration of one launch with the stream kept busy), and
`kernel_ms_median` the median over separately bracketed launches.  The short
workloads listed under `other_workloads` are warmed up for a fixed time first,
so that they are measured at the clocks the long ones reach by themselves.
"""
import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP32_MFMA_TFLOPS = 157.3   # MI355X dense fp32 matrix peak
PEAK_HBM_GBS = 8000.0
PEAK_VALU_TOPS = 39.3           # 256 CUs x 64 lanes x 2.4 GHz: one fp32 vector instruction per lane and cycle
                                # (packed fp32 is switched off in this build)

# HBM-side bytes per launch of the dominant kernel come from the tracked
# rocprofv3 summaries under profiles/ (FETCH_SIZE, WRITE_SIZE: KiB per dispatch):
# the counters cannot be read from inside this process, so the file of a workload
# (profiles/<kernel>_<workload>.txt) is parsed at start-up and every figure names
# the file it was read from.  On this box FETCH_SIZE reads half of the true bytes
# of a plain 1 GiB device copy and WRITE_SIZE all of them
# (profiles/copy_probe_1GiB.txt), so traffic = (2 * FETCH_SIZE + WRITE_SIZE) * 1024.
PROFILES_DIR = os.path.join(ROOT, "profiles")


def profile_of(name):
    """(path relative to the repository, kernel tag) of the summary of workload `name`, or None."""
    try:
        files = sorted(os.listdir(PROFILES_DIR))
    except OSError:
        return None
    tail = "_" + name + ".txt"
    for f in files:
        if f.endswith(tail) and f[:len(f) - len(tail)].endswith("_kernel"):
            return os.path.join("profiles", f), f[:len(f) - len(tail)]
    return None


def measured_traffic(name):
    """(bytes per launch of the dominant kernel, file, {kernel: avg microseconds per launch}) from the
    tracked summary of workload `name`; (None, None, {}) when there is none."""
    found = profile_of(name)
    if not found:
        return None, None, {}
    path, tag = found
    fetch = write = None
    trace = {}
    in_trace = False
    with open(os.path.join(ROOT, path)) as f:
        for line in f:
            t = line.split()
            if line.startswith("Kernel trace"):
                in_trace = True
                continue
            if line.startswith("Counters"):
                in_trace = False
            if in_trace and len(t) >= 6 and "cmk::" in line and t[-1].endswith("%"):
                kernel = line[:line.rindex(t[-5])].strip()     # calls avg min max time%
                trace[kernel] = float(t[-4])
            if "cmk::" + tag not in line:
                continue
            for key in ("FETCH_SIZE", "WRITE_SIZE"):
                if key in t and t[-1].startswith("avg="):
                    v = float(t[-1][4:])
                    if key == "FETCH_SIZE":
                        fetch = v
                    else:
                        write = v
    if fetch is None or write is None:
        return None, path, trace
    return (2 * fetch + write) * 1024, path, trace


SEED = 0
WARM_SECONDS = 0.3              # warm-up of the short workloads


# ----------------------------------------------------------------------------
# workloads
# ----------------------------------------------------------------------------
def make_workloads(torch, cmk, O, dev):
    """name -> dict.  `make()` returns (cpu_args, dev_args); `run(*dev_args)` is
    one step; `parity(cpu_args, dev_args, out)` checks a sample of the output
    against the oracle and returns a description of what it checked; `cpu(...)`
    runs the reference semantics on a slab of the workload on the host."""
    def gen(seed=SEED):
        return torch.Generator().manual_seed(seed)

    def randn_pair(L, M, N, K):
        g = gen()
        A = torch.randn(L, M, K, generator=g)
        B = torch.randn(L, K, N, generator=g)
        return A, B

    def uniform_pair(L, M, N, K):
        g = gen()
        A = torch.rand(L, M, K, generator=g) * 2 - 1
        B = torch.rand(L, K, N, generator=g) * 2 - 1
        return A, B

    def to_dev(*ts):
        return tuple(t.to(dev) for t in ts)

    def spread(n, count):
        """`count` positions spread evenly over range(n)."""
        count = min(n, count)
        return torch.arange(count) * (n // count) + (n // count) // 2 if count else torch.arange(0)

    W = {}

    def min_wl(name, L, M, N, K, dim=2, distance="inner", cpu_rows=None, config=None, screen=True):
        """`screen` False keeps squared l2 on the vector unit whatever the size (the
        operator's own choice is by size; both routes return the same bits)."""
        import custom_matmul_kernels_amd.minbmm as minbmm
        op = cmk.MinBMMCUDA(distance=distance)
        inner = distance == "inner"
        on_matrix_pipe = inner or (distance == "l2" and screen and minbmm.screens_l2(L, M, N, K))

        def run(A, B):
            if distance == "l2" and not screen:
                keep, minbmm.L2_SCREEN_MIN_WORK = minbmm.L2_SCREEN_MIN_WORK, 1 << 62
                try:
                    return op(A, B, dim=dim)
                finally:
                    minbmm.L2_SCREEN_MIN_WORK = keep
            return op(A, B, dim=dim)

        def make():
            A, B = randn_pair(L, M, N, K)
            return (A, B), to_dev(A, B)

        def parity(cpu_args, dev_args, out):
            A, B = cpu_args
            v, i = out
            kept = M if dim == 2 else N
            rows = spread(kept, 256 if inner else 48)
            if dim == 2:
                As, Bs = A[:, rows], B
            else:
                As, Bs = A, B[:, :, rows]
            vs, is_ = v[:, rows].cpu(), i[:, rows].cpu()
            if inner:
                mism = O.check_min(vs, is_, As, Bs, dim)
                return "%d of %d output rows per batch against torch.bmm(A,B).min(dim) on the CPU; " \
                       "%d index differences, all between products closer than the tolerance" % (len(rows), kept, mism)
            cv, ci = O.c_min_bmm(As.numpy(), Bs.numpy(), dim, 1 if distance == "l2" else 2)
            assert torch.equal(vs, torch.from_numpy(cv)) and torch.equal(is_, torch.from_numpy(ci).long())
            return "%d of %d output rows bit-equal to the C oracle's %s accumulation" % (len(rows), kept, distance)

        # flop: what the route executes per product term (matrix pipe: multiply + add of the
        # screening product; vector unit: subtract, multiply, add for l2, subtract, |.|, add for l1 counted as 2)
        per = 2.0 if on_matrix_pipe else (3.0 if distance == "l2" else 2.0)
        w = dict(make=make, run=run, flop=per * L * M * N * K, parity=parity,
                 desc="min_bmm%s fp32 A[%d,%d,%d] @ B[%d,%d,%d], min+argmin over dim=%d" % (
                     "" if inner else " distance=" + distance + (
                         " (screened on the matrix pipe, settled exactly)" if on_matrix_pipe else " (vector unit)"),
                     L, M, K, L, K, N, dim))
        if not on_matrix_pipe:
            w["valu_ops"] = 2.0 * L * M * N * K   # subtract + fused multiply-add, or subtract + add of |.|
        if cpu_rows:
            w.update(cpu=lambda A, B, r0: torch.bmm(A[:, r0:r0 + cpu_rows], B).min(-1), cpu_rows=cpu_rows, rows=M,
                     cpu_flop_per_row=2.0 * L * N * K, cpu_expr="torch.bmm(A,B).min(-1)")
        if config:
            w["config"] = config
        W[name] = w

    def topk_wl(name, L, M, N, K, dim=2, cpu_rows=None, config=None, b_transposed=False, distance="inner"):
        op = cmk.TopkBMMCUDA(distance=distance)
        inner = distance == "inner"

        def make():
            A, B = randn_pair(L, M, N, K)
            Ad, Bd = to_dev(A, B)
            if b_transposed:                         # B stored [n, k]: the "nt" layout of the reference
                Bd = Bd.transpose(1, 2).contiguous().transpose(1, 2)
            return (A, B), (Ad, Bd)

        def parity(cpu_args, dev_args, out):
            A, B = cpu_args
            v, i = out
            kept = M if dim == 2 else N
            rows = spread(kept, 128 if dim == 2 else 8)
            if dim == 2:
                As, Bs = A[:, rows], B
            else:
                As, Bs = A, B[:, :, rows]
            if not inner:
                cv, ci = O.c_topk_bmm(As.numpy(), Bs.numpy(), 128, dim, 1 if distance == "l2" else 2)
                assert torch.equal(v[:, rows].cpu(), torch.from_numpy(cv)), "values differ from the C oracle"
                return "%d of %d output rows: values bit-equal to the C oracle's %s accumulation and selection" % (
                    len(rows), kept, distance)
            mism = O.check_topk(v[:, rows].cpu(), i[:, rows].cpu(), As, Bs, 128, dim)
            return "%d of %d output rows per batch against torch.bmm(A,B).topk(128) on the CPU (values, order, " \
                   "value-at-index, uniqueness); %d index differences, all between products closer than the " \
                   "tolerance" % (len(rows), kept, mism)

        per = 2.0 if inner else (3.0 if distance == "l2" else 2.0)
        w = dict(make=make, run=lambda A, B: op(A, B, k=128, dim=dim), flop=per * L * M * N * K, parity=parity,
                 desc="topk_bmm%s fp32 A[%d,%d,%d] @ B[%d,%d,%d]%s, k=128 over dim=%d" % (
                     "" if inner else " distance=" + distance, L, M, K, L, K, N,
                     " (B stored [n,k])" if b_transposed else "", dim))
        if not inner:
            w["valu_ops"] = 2.0 * L * M * N * K
        if cpu_rows:
            w.update(cpu=lambda A, B, r0: torch.bmm(A[:, r0:r0 + cpu_rows], B).topk(128, dim=-1), cpu_rows=cpu_rows,
                     rows=M, cpu_flop_per_row=2.0 * L * N * K, cpu_expr="torch.bmm(A,B).topk(128,-1)")
        if config:
            w["config"] = config
        W[name] = w

    def bmm_wl(name, L, M, N, K, cpu=False, config=None):
        op = cmk.BMMCUDA()

        def make():
            A, B = uniform_pair(L, M, N, K)
            return (A, B), to_dev(A, B)

        def parity(cpu_args, dev_args, out):
            A, B = cpu_args
            bs = spread(L, 4).tolist()
            rows = spread(M, 256)
            for b in bs:
                want = A[b, rows].double() @ B[b].double()
                O.check_values(out[b, rows].cpu(), want, K, "bmm batch %d" % b)
            return "%d rows of each of %d batches against a float64 product on the CPU" % (len(rows), len(bs))

        w = dict(make=make, run=lambda A, B: op(A, B), flop=2.0 * L * M * N * K, parity=parity,
                 desc="bmm fp32 A[%d,%d,%d] @ B[%d,%d,%d]" % (L, M, K, L, K, N),
                 bytes=4.0 * L * (M * N + M * K + K * N))
        if cpu:
            w.update(cpu=lambda A, B, r0: torch.bmm(A[r0:r0 + 16], B[r0:r0 + 16]), cpu_rows=16, rows=L,
                     cpu_flop_per_row=2.0 * M * N * K, cpu_expr="torch.bmm(A,B)", cpu_unit="batches")
        if config:
            w["config"] = config
        W[name] = w

    def mbmm_wl(name, L, M, N, K, tiles=True, cpu=False, config=None):
        op = cmk.MBMMCUDA(share_mask=False)

        def make():
            A, B = randn_pair(L, M, N, K)
            fm = torch.tril(torch.ones(M, N)).bool()[None].expand(L, -1, -1)
            if tiles:
                keep = torch.rand(L, M // 128, N // 128, generator=gen(SEED + 1)) < 0.5
                fm = fm & keep.repeat_interleave(128, 1).repeat_interleave(128, 2)
            fm = fm.contiguous()
            Ad, Bd = to_dev(A, B)
            bm, tm, em = cmk.derive_masks(fm.to(dev))
            return (A, B, fm), (Ad, Bd, bm, tm, em)

        def parity(cpu_args, dev_args, out):
            A, B, fm = cpu_args
            bs = spread(L, 8).tolist()
            for b in bs:
                want = O.ref_mbmm(A[b:b + 1], B[b:b + 1], fm[b:b + 1])
                O.check_values(out[b:b + 1].cpu(), want, K, "mbmm batch %d" % b)
                assert (out[b].cpu()[~fm[b]] == 0).all(), "masked-out element not zero"
            return "%d of %d batches against torch.bmm + masked_fill on the CPU; masked-out elements exactly 0" % (
                len(bs), L)

        w = dict(make=make, run=lambda A, B, bm, tm, em: op(A, B, bm, tm, em), flop=2.0 * L * M * N * K,
                 parity=parity, mbmm=True,
                 desc="mbmm fp32 A[%d,%d,%d] @ B[%d,%d,%d], %s mask" % (
                     L, M, K, L, K, N, "tril & tile-Bernoulli(0.5)" if tiles else "tril"),
                 bytes=4.0 * L * (M * N + M * K + K * N) + L * M * N + L * (M // 8) * (N // 8))
        if cpu:
            w.update(cpu=lambda A, B, fm, r0: torch.bmm(A[r0:r0 + 16], B[r0:r0 + 16]).masked_fill_(~fm[r0:r0 + 16], 0),
                     cpu_rows=16, rows=L, cpu_flop_per_row=2.0 * M * N * K,
                     cpu_expr="torch.bmm(A,B).masked_fill_(~mask,0)", cpu_unit="batches")
        if config:
            w["config"] = config
        W[name] = w

    def masks_wl(name, L, M, N):
        # byte work: reads the element mask once, writes 1/64 + 1/16384 of it
        def make():
            keep = torch.rand(L, M // 128, N // 128, generator=gen(SEED + 1)) < 0.5
            fm = torch.tril(torch.ones(M, N)).bool()[None] & keep.repeat_interleave(128, 1).repeat_interleave(128, 2)
            return (fm,), (fm.to(dev),)

        def parity(cpu_args, dev_args, out):
            fm, = cpu_args
            bs = spread(L, 4).tolist()
            for b in bs:
                bm, tm, em = O.ref_derive_masks(fm[b:b + 1])
                assert torch.equal(out[0][b:b + 1].cpu(), bm) and torch.equal(out[1][b:b + 1].cpu(), tm)
            return "%d of %d batches bit-equal to the oracle's block and thread masks" % (len(bs), L)

        W[name] = dict(make=make, run=lambda fm: cmk.derive_masks(fm), flop=0.0, dtype="u8", parity=parity,
                       desc="derive_masks of a bool mask [%d,%d,%d] (block + thread masks)" % (L, M, N),
                       bytes=1.0 * L * M * N + L * (M // 8) * (N // 8) + L * (M // 128) * (N // 128))

    def copy_wl(name, nbytes):
        # a plain device copy of known size: the yardstick the HBM counters are scaled by
        def make():
            src = torch.empty(nbytes // 4, dtype=torch.float32, device=dev).normal_()
            return (), (src, torch.empty_like(src))

        W[name] = dict(make=make, run=lambda src, dst: dst.copy_(src), flop=0.0,
                       desc="device copy of %d bytes (reads and writes that many)" % nbytes, bytes=2.0 * nbytes)

    copy_wl("copy_probe", 1 << 30)
    # the five benchmark configurations
    min_wl("min_bmm_large", 1, 65536, 65536, 256, cpu_rows=4096, config=4)
    min_wl("min_bmm_small", 1, 4096, 4096, 64, cpu_rows=4096, config=1)
    bmm_wl("bmm", 128, 1024, 1024, 128, cpu=True, config=2)
    mbmm_wl("mbmm", 128, 1024, 1024, 64, cpu=True, config=3)
    topk_wl("topk_bmm", 1, 1048576, 1024, 256, cpu_rows=65536, config=5)
    # the next rows: mask derivation and the vector-unit distances
    masks_wl("derive_masks", 128, 1024, 1024)
    masks_wl("derive_masks_4GiB", 1024, 2048, 2048)
    min_wl("min_bmm_l2", 1, 16384, 16384, 256, distance="l2")
    min_wl("min_bmm_l2_vector", 1, 16384, 16384, 256, distance="l2", screen=False)
    min_wl("min_bmm_l1", 1, 16384, 16384, 256, distance="l1")
    # the shapes the reference publishes numbers for (its notebooks' printed results and plots, Tesla T4)
    bmm_wl("ref_bmm_8192x512", 1, 8192, 8192, 512)             # colab/test_bmm.ipynb:2163-2164
    bmm_wl("ref_bmm_8192_cube", 1, 8192, 8192, 8192)           # imgs/bmm_A[1,N,N] B[1,N,N].png
    bmm_wl("bmm_long_k", 1, 512, 512, 4096)                    # few tiles, long contraction: k cut into ranges
    min_wl("ref_min_bmm_1024x131072_k64", 1, 1024, 131072, 64)  # colab/test_minbmm.ipynb:2192-2193
    min_wl("ref_min_bmm_16384_k64", 1, 16384, 16384, 64)       # imgs/min_bmm_A[1,N,64] B[1,64,N].png
    min_wl("ref_min_bmm_16384_k256", 1, 16384, 16384, 256)     # imgs/min_bmm_A[1,N,256] B[1,256,N].png
    min_wl("ref_min_bmm_b64_3072_k64", 64, 3072, 3072, 64)     # imgs/min_bmm_A[64,N,64] B[64,64,N].png
    mbmm_wl("ref_mbmm_tril_1024", 128, 1024, 1024, 64, tiles=False)   # imgs/mbmm_A[128,1024,X] B[128,X,1024].png
    mbmm_wl("ref_mbmm_tril_2048", 128, 2048, 2048, 64, tiles=False)   # imgs/mbmm_A[128,X,64] B[128,64,X].png
    topk_wl("ref_topk_bmm_32768_dim1", 1, 32768, 1024, 256, dim=1)   # colab/test_topkbmm.ipynb:2747-2751
    topk_wl("ref_topk_bmm_2e20_k64_dim1", 1, 1048576, 1024, 64, dim=1)     # imgs/topk_bmm_A[1,N,64] ..._loglog.png
    topk_wl("ref_topk_bmm_2e20_k256_dim1", 1, 1048576, 1024, 256, dim=1)   # imgs/topk_bmm_A[1,N,256] ..._loglog.png
    topk_wl("ref_topk_bmm_2e20_k1024_dim1", 1, 1048576, 1024, 1024, dim=1)  # imgs/topk_bmm_A[1,N,1024] ..._loglog.png
    topk_wl("topk_bmm_k64", 1, 1048576, 1024, 64)              # the fused top-k at K = 64, dim=-1
    # other code paths of the top-k kernel: B stored [n,k], a reduced axis of several chunks, a vector-unit distance
    topk_wl("topk_bmm_nt", 1, 262144, 1024, 256, b_transposed=True)
    topk_wl("topk_bmm_multi", 1, 16384, 16384, 256)
    # nearest-neighbour search geometry: few kept rows, a reduced axis of hundreds of chunks
    topk_wl("topk_bmm_long_axis", 1, 4096, 1048576, 256)
    topk_wl("topk_bmm_long_axis_k64", 1, 16384, 131072, 64)
    topk_wl("topk_bmm_l2", 1, 65536, 1024, 64, distance="l2")
    return W


# ----------------------------------------------------------------------------
# timing
# ----------------------------------------------------------------------------
def time_region(torch, fn, steps, warmup):
    """`warmup` untimed steps, then exactly `steps` steps between two
    synchronisations.  Returns (wall seconds of the region, milliseconds between
    two events recorded on the launch stream around the region)."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for _ in range(steps):
        fn()
    end.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    return wall, start.elapsed_time(end)


def median_launch_ms(torch, fn, n):
    """Median over `n` launches, each between two events of its own."""
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(n)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(n)]
    for s in range(n):
        starts[s].record()
        fn()
        ends[s].record()
    torch.cuda.synchronize()
    return statistics.median(starts[s].elapsed_time(ends[s]) for s in range(n))


def warm_for(torch, fn, seconds):
    """Keeps the GPU busy with `fn` for about `seconds`; returns the steps done."""
    done = 0
    t0 = time.perf_counter()
    while True:
        for _ in range(10):
            fn()
        done += 10
        torch.cuda.synchronize()
        if time.perf_counter() - t0 >= seconds:
            return done


def cpu_model():
    """The host CPU's model string, from /proc/cpuinfo."""
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown CPU"


def cpu_baseline(torch, wl, cpu_args, budget_s):
    """The reference semantics with PyTorch on the host cores, on a bounded
    sample (slabs of rows, or of batches, of the same workload)."""
    if "cpu" not in wl:
        return None
    rows, total = wl["cpu_rows"], wl["rows"]
    unit = wl.get("cpu_unit", "rows")
    wl["cpu"](*cpu_args, 0)                           # warm-up slab
    done, t_total, off = 0, 0.0, 0
    while t_total < budget_s and done < 8 * total:
        if off + rows > total:
            off = 0                                   # another pass over the same data
        t0 = time.perf_counter()
        wl["cpu"](*cpu_args, off)
        t_total += time.perf_counter() - t0
        done += rows
        off += rows
    gflops = done * wl["cpu_flop_per_row"] / t_total / 1e9
    return {"value": round(gflops, 2), "unit": "GFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": "%s on %d %s in slabs of %d (%.2f passes over the workload's %d %s), "
                      "%d threads of %d logical CPUs (%s), %.2f s"
                      % (wl["cpu_expr"], done, unit, rows, done / total, total, unit,
                         torch.get_num_threads(), os.cpu_count() or 0, cpu_model(), t_total)}


def parity_of(torch, wl, cpu_args, dev_args):
    """Runs the workload once more and checks a sample of its output against the
    oracle; never inside a timed region."""
    if "parity" not in wl:
        return None
    out = wl["run"](*dev_args)
    torch.cuda.synchronize()
    try:
        what = wl["parity"](cpu_args, dev_args, out)
        return {"ok": True, "checked": what}
    except AssertionError as e:
        return {"ok": False, "error": str(e)[:300]}


def roofline_of(name, wl, kern_ms):
    traffic, source, _ = measured_traffic(name)
    if wl["flop"] == 0:
        ach = wl["bytes"] / (kern_ms * 1e-3) / 1e9
        roof = {"bound": "hbm", "achieved": round(ach, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                "frac": round(ach / PEAK_HBM_GBS, 4)}
    elif "valu_ops" in wl:
        ach = wl["valu_ops"] / (kern_ms * 1e-3) / 1e12
        roof = {"bound": "valu", "achieved": round(ach, 2), "peak": PEAK_VALU_TOPS, "unit": "Tinstr/s (per lane)",
                "frac": round(ach / PEAK_VALU_TOPS, 4)}
    elif wl.get("mbmm"):
        ach = wl["bytes"] / (kern_ms * 1e-3) / 1e9
        roof = {"bound": "hbm", "achieved": round(ach, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                "frac": round(ach / PEAK_HBM_GBS, 4)}
    else:
        ach = wl["flop"] / (kern_ms * 1e-3) / 1e12
        roof = {"bound": "mfma", "achieved": round(ach, 2), "peak": PEAK_FP32_MFMA_TFLOPS, "unit": "TFLOP/s",
                "frac": round(ach / PEAK_FP32_MFMA_TFLOPS, 4)}
    roof["traffic"] = traffic
    if source:
        roof["traffic_source"] = source
    if traffic and wl.get("bytes"):
        roof["traffic_over_algorithmic_bytes"] = round(traffic / wl["bytes"], 2)
    roof["kernel_ms"] = round(kern_ms, 5)
    return roof


def steps_for(torch, fn):
    """Step count of a short workload: about 50 ms of launches, 20 to 2000 steps."""
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(5):
        fn()
    torch.cuda.synchronize()
    per = (time.perf_counter() - t0) / 5
    return int(min(2000, max(20, 0.05 / max(per, 1e-6))))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="min_bmm_large")
    ap.add_argument("--details", default=None, help="also write the full record (one JSON line) to this file")
    ap.add_argument("--no-others", action="store_true", help="skip the short runs of the other workloads")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baselines")
    ap.add_argument("--no-parity", action="store_true", help="skip the parity checks")
    ap.add_argument("--warm-seconds", type=float, default=0.0,
                    help="keep the GPU busy with the workload this long before the warm-up steps")
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus %d is not supported "
              "(every output row depends on one row of A and all of B, so the path "
              "would shard by rows without communication)" % a.gpus, file=sys.stderr)
        sys.exit(2)

    import torch
    import custom_matmul_kernels_amd as cmk
    from oracle import oracle as O                   # the checker of the parity legs and nothing else
    cmk.load()                                       # fails loudly if libcmk.so is missing
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    W = make_workloads(torch, cmk, O, dev)
    wl = W[a.workload]

    cpu_args, dev_args = wl["make"]()
    torch.cuda.synchronize()
    fn = lambda: wl["run"](*dev_args)                # noqa: E731
    if a.warm_seconds > 0:
        warm_for(torch, fn, a.warm_seconds)
    wall, region_ms = time_region(torch, fn, a.steps, a.warmup)
    ms = wall * 1e3 / a.steps
    kern_ms = region_ms / a.steps
    med_ms = median_launch_ms(torch, fn, min(a.steps, 50))
    roof = roofline_of(a.workload, wl, kern_ms)
    roof["kernel_ms_median"] = round(med_ms, 5)
    if wl["flop"] > 0:
        value, unit = wl["flop"] / (ms * 1e-3) / 1e9, "GFLOP/s"
        kind = "fp32 vector unit" if "valu_ops" in wl else "fp32 MFMA"
        metric = "GFLOP/s of %s (2*L*M*N*K / time), %s" % (a.workload, kind)
    else:
        value, unit = wl["bytes"] / (ms * 1e-3) / 1e9, "GB/s"
        metric = "GB/s of %s (algorithmic bytes / time)" % a.workload
    out = {
        "metric": metric, "value": round(value, 1), "unit": unit, "n_gpus": 1, "steps": a.steps,
        "warmup": a.warmup, "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": wl.get("dtype", "f32"),
        "data": "synthetic (CPU generator seed %d, A before B, copied to the device)" % SEED,
        "config": {"workload": wl["desc"], "name": a.workload},
        "roofline": roof,
    }
    if not a.no_parity:
        out["parity"] = parity_of(torch, wl, cpu_args, dev_args)
    if not a.no_cpu:
        out["cpu_baseline"] = cpu_baseline(torch, wl, cpu_args, budget_s=12.0)
    del cpu_args, dev_args
    torch.cuda.empty_cache()

    if not a.no_others:
        others = {}
        for name, w in W.items():
            if name == a.workload or name == "copy_probe":
                continue
            cpu_args, dev_args = w["make"]()
            torch.cuda.synchronize()
            fn = lambda: w["run"](*dev_args)         # noqa: E731
            steps = steps_for(torch, fn)
            warm_for(torch, fn, WARM_SECONDS)
            wall_o, region_o = time_region(torch, fn, steps, 3)
            kern_o = region_o / steps
            med_o = median_launch_ms(torch, fn, min(steps, 50))
            rec = {"workload": w["desc"], "steps": steps, "ms_per_step": round(wall_o * 1e3 / steps, 5),
                   "kernel_ms": round(kern_o, 5), "kernel_ms_median": round(med_o, 5)}
            if "config" in w:
                rec["config"] = w["config"]
            traffic, source, trace = measured_traffic(name)
            strict_ms = max(kern_o, med_o)       # the less favourable of the two live clocks
            if w.get("mbmm"):
                # skipped tiles do no arithmetic: only the executed work is priced against the matrix peak
                kept = int(dev_args[2].sum())
                rec["kept_tiles"] = kept
                executed = 2.0 * 128 * 128 * cpu_args[0].shape[2] * kept
                rec["dense_equivalent_GFLOP/s"] = round(w["flop"] / (kern_o * 1e-3) / 1e9, 1)
                rec["executed_GFLOP/s"] = round(executed / (kern_o * 1e-3) / 1e9, 1)
                rec["executed_frac_fp32_mfma_peak"] = round(executed / (kern_o * 1e-3) / 1e12 / PEAK_FP32_MFMA_TFLOPS, 4)
            elif w["flop"] > 0:
                rec["GFLOP/s"] = round(w["flop"] / (kern_o * 1e-3) / 1e9, 1)
                key = "frac_valu_issue_peak" if "valu_ops" in w else "frac_fp32_mfma_peak"
                work = w["valu_ops"] / PEAK_VALU_TOPS if "valu_ops" in w else w["flop"] / PEAK_FP32_MFMA_TFLOPS
                # priced by the stricter clock; the region average is carried beside it
                rec[key] = round(work / (strict_ms * 1e-3) / 1e12, 4)
                rec[key + "_region_average"] = round(work / (kern_o * 1e-3) / 1e12, 4)
                if len(trace) > 1:
                    # an operation of several launches: the kernels' own durations from the tracked trace
                    rec["trace_us"] = {k: v for k, v in trace.items()}
                    rec[key + "_by_trace"] = round(work / (sum(trace.values()) * 1e-6) / 1e12, 4)
            if "bytes" in w:
                rec["GB/s"] = round(w["bytes"] / (kern_o * 1e-3) / 1e9, 1)
                rec["frac_hbm_peak"] = round(rec["GB/s"] / PEAK_HBM_GBS, 4)
            if traffic:
                rec["traffic"], rec["traffic_source"] = traffic, source
                if w.get("bytes"):
                    rec["traffic_over_algorithmic_bytes"] = round(traffic / w["bytes"], 2)
                    # what actually moved, by the counters, over the live time
                    rec["frac_hbm_peak_by_counter_bytes"] = round(traffic / (kern_o * 1e-3) / 1e9 / PEAK_HBM_GBS, 4)
            if not a.no_parity:
                rec["parity"] = parity_of(torch, w, cpu_args, dev_args)
            if not a.no_cpu and "cpu" in w:
                rec["cpu_baseline"] = cpu_baseline(torch, w, cpu_args, budget_s=4.0)
            others[name] = rec
            del cpu_args, dev_args
            torch.cuda.empty_cache()
        out["other_workloads"] = others
    # The full record goes to stderr (and to the file --details names); the one
    # line on stdout keeps the headline in full and, per other workload, the
    # figures only, so that it stays a few kilobytes.
    full = json.dumps(out)
    print(full, file=sys.stderr)
    if a.details:
        with open(a.details, "w") as f:
            f.write(full + "\n")
    if "other_workloads" in out:
        keep = ("config", "kernel_ms", "kernel_ms_median", "frac_fp32_mfma_peak", "frac_fp32_mfma_peak_region_average",
                "frac_fp32_mfma_peak_by_trace", "executed_frac_fp32_mfma_peak", "frac_hbm_peak",
                "frac_hbm_peak_by_counter_bytes", "frac_valu_issue_peak", "traffic_over_algorithmic_bytes")
        brief = {}
        for name, rec in out["other_workloads"].items():
            b = {k: rec[k] for k in keep if k in rec}
            if rec.get("parity") is not None:
                b["parity_ok"] = rec["parity"]["ok"]
            if rec.get("cpu_baseline"):
                b["cpu_GFLOP/s"] = rec["cpu_baseline"]["value"]
                b["cpu_cores"] = rec["cpu_baseline"]["cores"]
            brief[name] = b
        out["other_workloads"] = brief
        out["other_workloads_note"] = ("shapes, step counts, parity details and CPU samples of these workloads: "
                                       "the same record in full on stderr; kernel_ms = events around the timed "
                                       "region / steps, after 0.3 s of warm-up; fractions are priced by the larger of "
                                       "kernel_ms and kernel_ms_median (the region average is carried beside them); "
                                       "mbmm: only the kept tiles' arithmetic counts")
    print(json.dumps(out))


if __name__ == "__main__":
    main()
