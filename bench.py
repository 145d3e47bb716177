"""Benchmark of the fused batched-matmul path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-others]

One step = one pass of the hot path over one synthetic batch that is already
resident in HBM.  The headline workload is the large fused min_bmm
(A[1,65536,256] @ B[1,256,65536], min/argmin over dim=-1, product never
stored); the JSON line also carries the roofline of its kernel, the same
semantics timed with PyTorch on the host CPU, and short runs of the other
configurations.
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

# HBM-side bytes per launch of the dominant kernel, from rocprofv3 --pmc
# (FETCH_SIZE, WRITE_SIZE: KiB per dispatch).  On this box FETCH_SIZE reads half
# of the true bytes of a plain 1 GiB device copy and WRITE_SIZE all of them, so
# traffic = (2 * FETCH_SIZE + WRITE_SIZE) * 1024.  The counters cannot be read
# from inside this process; the figures are those of the summaries in profiles/.
MEASURED_TRAFFIC_BYTES = {
    "min_bmm_large": (2 * 2.15038e6 + 2048) * 1024,      # profiles/min_kernel_min_bmm_large.txt
    "topk_bmm": (2 * 882558 + 1.71006e6) * 1024,           # profiles/topk_kernel_topk_bmm.txt
    "derive_masks_4GiB": (2 * 2.09726e6 + 66564.6) * 1024,  # profiles/derive_masks_kernel_4GiB.txt
}


def make_workloads(torch, cmk, dev):
    """name -> dict(make=..., run=..., flop=..., desc=..., cpu=...)."""
    def randn(*shape, seed):
        g = torch.Generator(device=dev).manual_seed(seed)
        return torch.randn(*shape, generator=g, device=dev)

    def rand_pm1(*shape, seed):
        g = torch.Generator(device=dev).manual_seed(seed)
        return torch.rand(*shape, generator=g, device=dev) * 2 - 1

    W = {}

    def min_wl(name, M, N, K, cpu_rows):
        op = cmk.MinBMMCUDA()

        def make():
            return randn(1, M, K, seed=0), randn(1, K, N, seed=1)

        def cpu(A, B):   # torch.bmm(A, B).min(-1) on a slab of rows
            return torch.bmm(A[:, :cpu_rows], B).min(-1)

        W[name] = dict(make=make, run=lambda A, B: op(A, B, dim=-1), flop=2.0 * M * N * K,
                       desc="min_bmm fp32 A[1,%d,%d] @ B[1,%d,%d], min+argmin over dim=-1" % (M, K, K, N),
                       cpu=cpu, cpu_rows=cpu_rows, rows=M, cpu_flop_per_row=2.0 * N * K,
                       cpu_expr="torch.bmm(A,B).min(-1)")

    def min_dist_wl(name, distance, M, N, K):
        # (a-b)^2 / |a-b| accumulation on the vector unit: two instructions per (m, n, k) either way
        # (subtract + fused multiply-add for l2, subtract + add-of-absolute-value for l1)
        op = cmk.MinBMMCUDA(distance=distance)

        def make():
            return randn(1, M, K, seed=0), randn(1, K, N, seed=1)

        per = 3.0 if distance == "l2" else 2.0
        W[name] = dict(make=make, run=lambda A, B: op(A, B, dim=-1), flop=per * M * N * K, valu_ops=2.0 * M * N * K,
                       desc="min_bmm distance=%s fp32 A[1,%d,%d] vs B[1,%d,%d], min+argmin over dim=-1 "
                            "(vector unit, %d flop per element pair and k)" % (distance, M, K, K, N, int(per)))

    def topk_wl(name, M, N, K, cpu_rows):
        op = cmk.TopkBMMCUDA()

        def make():
            return randn(1, M, K, seed=0), randn(1, K, N, seed=1)

        def cpu(A, B):
            return torch.bmm(A[:, :cpu_rows], B).topk(128, dim=-1)

        W[name] = dict(make=make, run=lambda A, B: op(A, B, k=128, dim=-1), flop=2.0 * M * N * K,
                       desc="topk_bmm fp32 A[1,%d,%d] @ B[1,%d,%d], k=128 over dim=-1" % (M, K, K, N),
                       cpu=cpu, cpu_rows=cpu_rows, rows=M, cpu_flop_per_row=2.0 * N * K,
                       cpu_expr="torch.bmm(A,B).topk(128,-1)")

    def bmm_wl(name, L, M, N, K):
        op = cmk.BMMCUDA()

        def make():
            return rand_pm1(L, M, K, seed=0), rand_pm1(L, K, N, seed=1)

        W[name] = dict(make=make, run=lambda A, B: op(A, B), flop=2.0 * L * M * N * K,
                       desc="bmm fp32 A[%d,%d,%d] @ B[%d,%d,%d]" % (L, M, K, L, K, N),
                       bytes=4.0 * L * (M * N + M * K + K * N))

    def mbmm_wl(name, L, M, N, K):
        op = cmk.MBMMCUDA(share_mask=False)

        def make():
            A, B = randn(L, M, K, seed=0), randn(L, K, N, seed=1)
            g = torch.Generator().manual_seed(1)
            tiles = torch.rand(L, M // 128, N // 128, generator=g) < 0.5
            keep = tiles.repeat_interleave(128, 1).repeat_interleave(128, 2)
            fm = torch.tril(torch.ones(M, N)).bool()[None] & keep
            bm, tm, em = cmk.derive_masks(fm.to(dev))
            kept_tiles = int(bm.sum())
            return A, B, bm, tm, em, kept_tiles

        W[name] = dict(make=make, run=lambda A, B, bm, tm, em, kt: op(A, B, bm, tm, em),
                       flop=2.0 * L * M * N * K,
                       desc="mbmm fp32 A[%d,%d,%d] @ B[%d,%d,%d], tril & tile-Bernoulli(0.5) mask" % (L, M, K, L, K, N),
                       bytes=4.0 * L * (M * N + M * K + K * N) + L * M * N + L * (M // 8) * (N // 8))

    def masks_wl(name, L, M, N):
        # byte work: reads the element mask once, writes 1/64 + 1/16384 of it
        def make():
            g = torch.Generator().manual_seed(1)
            tiles = (torch.rand(L, M // 128, N // 128, generator=g) < 0.5).to(dev)
            keep = tiles.repeat_interleave(128, 1).repeat_interleave(128, 2)
            return (torch.tril(torch.ones(M, N, device=dev)).bool()[None] & keep,)

        W[name] = dict(make=make, run=lambda fm: cmk.derive_masks(fm), flop=0.0, dtype="u8",
                       desc="derive_masks of a bool mask [%d,%d,%d] (block + thread masks)" % (L, M, N),
                       bytes=1.0 * L * M * N + L * (M // 8) * (N // 8) + L * (M // 128) * (N // 128))

    def copy_wl(name, nbytes):
        # a plain device copy of known size: the yardstick the HBM counters are scaled by
        def make():
            src = torch.empty(nbytes // 4, dtype=torch.float32, device=dev).normal_()
            return src, torch.empty_like(src)

        W[name] = dict(make=make, run=lambda src, dst: dst.copy_(src), flop=0.0,
                       desc="device copy of %d bytes (reads and writes that many)" % nbytes,
                       bytes=2.0 * nbytes)

    copy_wl("copy_probe", 1 << 30)
    min_wl("min_bmm_large", 65536, 65536, 256, cpu_rows=4096)
    min_wl("min_bmm_small", 4096, 4096, 64, cpu_rows=4096)
    topk_wl("topk_bmm", 1048576, 1024, 256, cpu_rows=65536)
    bmm_wl("bmm", 128, 1024, 1024, 128)
    mbmm_wl("mbmm", 128, 1024, 1024, 64)
    masks_wl("derive_masks", 128, 1024, 1024)
    masks_wl("derive_masks_4GiB", 1024, 2048, 2048)
    min_dist_wl("min_bmm_l2", "l2", 16384, 16384, 256)
    min_dist_wl("min_bmm_l1", "l1", 16384, 16384, 256)
    return W


def time_steps(torch, fn, steps, warmup):
    """Wall time of exactly `steps` steps between synchronisations, plus the
    per-launch device time from events recorded on the launch stream."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    t0 = time.perf_counter()
    for s in range(steps):
        starts[s].record()
        fn()
        ends[s].record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    dev_ms = [starts[s].elapsed_time(ends[s]) for s in range(steps)]
    return wall, dev_ms


def cpu_baseline(torch, wl, args_dev, budget_s=12.0):
    """The reference semantics with PyTorch on the host cores, on a bounded
    sample (slabs of rows of the same workload)."""
    if "cpu" not in wl:
        return None
    A, B = args_dev[0].cpu(), args_dev[1].cpu()
    wl["cpu"](A, B)                                  # warm-up slab
    done_rows, t_total = 0, 0.0
    rows = wl["cpu_rows"]
    off = 0
    while t_total < budget_s and done_rows < 8 * wl["rows"]:
        if off + rows > wl["rows"]:
            off = 0                                  # another pass over the same rows
        a = A[:, off:off + rows]
        t0 = time.perf_counter()
        wl["cpu"](a, B)
        t_total += time.perf_counter() - t0
        done_rows += rows
        off += rows
    gflops = done_rows * wl["cpu_flop_per_row"] / t_total / 1e9
    return {"value": round(gflops, 2), "unit": "GFLOP/s", "cores": torch.get_num_threads(),
            "kind": "port",
            "sample": "%s on %d rows in slabs of %d (%.2f passes over the workload's %d rows), "
                      "%d threads of %d logical CPUs (%s), %.2f s"
                      % (wl["cpu_expr"], done_rows, rows, done_rows / wl["rows"], wl["rows"],
                         torch.get_num_threads(), os.cpu_count() or 0, cpu_model(), t_total)}


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


def run_workload(torch, wl, steps, warmup):
    args = wl["make"]()
    torch.cuda.synchronize()
    wall, dev_ms = time_steps(torch, lambda: wl["run"](*args), steps, warmup)
    ms = wall * 1e3 / steps
    kern_ms = statistics.mean(dev_ms)
    return args, ms, kern_ms


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="min_bmm_large")
    ap.add_argument("--no-others", action="store_true", help="skip the short runs of the other configurations")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus %d is not supported "
              "(every output row depends on one row of A and all of B, so the path "
              "would shard by rows without communication)" % a.gpus, file=sys.stderr)
        sys.exit(2)

    import torch
    import custom_matmul_kernels_amd as cmk
    cmk.load()                                       # fails loudly if libcmk.so is missing
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    W = make_workloads(torch, cmk, dev)
    wl = W[a.workload]

    args, ms, kern_ms = run_workload(torch, wl, a.steps, a.warmup)
    gflops = wl["flop"] / (ms * 1e-3) / 1e9
    achieved = wl["flop"] / (kern_ms * 1e-3) / 1e12
    if wl["flop"] == 0:
        ach = wl["bytes"] / (kern_ms * 1e-3) / 1e9
        roof = {"bound": "hbm", "achieved": round(ach, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                "frac": round(ach / PEAK_HBM_GBS, 4), "traffic": MEASURED_TRAFFIC_BYTES.get(a.workload),
                "kernel_ms": round(kern_ms, 4)}
        metric = "GB/s of %s (algorithmic bytes / time)" % a.workload
    elif "valu_ops" in wl:
        ach = wl["valu_ops"] / (kern_ms * 1e-3) / 1e12
        roof = {"bound": "valu", "achieved": round(ach, 2), "peak": PEAK_VALU_TOPS, "unit": "Tinstr/s (per lane)",
                "frac": round(ach / PEAK_VALU_TOPS, 4), "traffic": None, "kernel_ms": round(kern_ms, 4)}
        metric = "GFLOP/s of fused %s (flop as the workload states / time), fp32 vector unit" % a.workload
    else:
        roof = {"bound": "mfma", "achieved": round(achieved, 2), "peak": PEAK_FP32_MFMA_TFLOPS,
                "unit": "TFLOP/s", "frac": round(achieved / PEAK_FP32_MFMA_TFLOPS, 4),
                "traffic": MEASURED_TRAFFIC_BYTES.get(a.workload), "kernel_ms": round(kern_ms, 4)}
        metric = ("GFLOP/s of fused %s (2*M*N*K / time), fp32 MFMA"
                  % a.workload.split("_large")[0].split("_small")[0])
    out = {
        "metric": metric,
        "value": round(gflops, 1) if wl["flop"] > 0 else round(wl["bytes"] / (ms * 1e-3) / 1e9, 1),
        "unit": "GFLOP/s" if wl["flop"] > 0 else "GB/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": wl.get("dtype", "f32"), "data": "synthetic",
        "config": {"workload": wl["desc"], "name": a.workload},
        "roofline": roof,
    }
    if not a.no_cpu:
        out["cpu_baseline"] = cpu_baseline(torch, wl, args)
    del args
    torch.cuda.empty_cache()

    if not a.no_others:
        others = {}
        for name, w in W.items():
            if name == a.workload or name == "copy_probe":
                continue
            steps = 5 if name == "topk_bmm" else 20
            args, ms_o, kern_o = run_workload(torch, w, steps, 3)
            rec = {"workload": w["desc"], "ms_per_step": round(ms_o, 4), "kernel_ms": round(kern_o, 4)}
            if w["flop"] > 0:
                rec["GFLOP/s"] = round(w["flop"] / (kern_o * 1e-3) / 1e9, 1)
            if w["flop"] == 0:
                pass
            elif "valu_ops" in w:
                rec["frac_valu_issue_peak"] = round(w["valu_ops"] / (kern_o * 1e-3) / 1e12 / PEAK_VALU_TOPS, 4)
            else:
                rec["frac_fp32_mfma_peak"] = round(w["flop"] / (kern_o * 1e-3) / 1e12 / PEAK_FP32_MFMA_TFLOPS, 4)
            if "bytes" in w:
                rec["GB/s"] = round(w["bytes"] / (kern_o * 1e-3) / 1e9, 1)
                rec["frac_hbm_peak"] = round(rec["GB/s"] / PEAK_HBM_GBS, 4)
            if name == "mbmm":
                kept = args[5]
                rec["kept_tiles"] = kept
                rec["executed_GFLOP/s"] = round(2.0 * 128 * 128 * 64 * kept / (kern_o * 1e-3) / 1e9, 1)
            if not a.no_cpu and "cpu" in w and name != "min_bmm_small":
                rec["cpu_baseline"] = cpu_baseline(torch, w, args, budget_s=6.0)
            others[name] = rec
            del args
            torch.cuda.empty_cache()
        out["other_workloads"] = others
    print(json.dumps(out))


if __name__ == "__main__":
    main()
