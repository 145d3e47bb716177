"""Size sweeps of the fused operators against their unfused equivalents:
run time and result-memory footprint as functions of N for A[l,N,k] @ B[l,k,N].

This is the measurement the reference's notebooks plot (grid tests of
colab/test_minbmm.ipynb:2236-2335 and colab/test_topkbmm.ipynb:2810-2947, timing
loops of test_min_bmm, colab/test_minbmm.ipynb:2098-2186): for every size, the
library product followed by the reduction (``torch.bmm`` + ``min`` / ``topk`` /
``masked_fill``), this package's plain product followed by the same reduction,
and the fused operator, each warmed up and then timed over ``iters`` calls.

    python -m custom_matmul_kernels_amd.sweep --op min_bmm --l 1 --k 64 \\
        --start 256 --stop 16384 --step 256 --iters 25 --csv min_bmm.csv --plot min_bmm.png

Columns of the CSV: op, l, n, k, variant, ms (per call), tflops (2*l*n*n*k /
time), result_mib (bytes of everything the variant leaves allocated for its
results, the quantity the notebooks' memory plots show: the product C counts for
the unfused variants, not for the fused ones), peak_mib (allocator high-water
mark above the inputs, workspaces included), max_abs_err and index_mismatch of
the fused result against ``torch.bmm`` + reduction.
"""
import argparse
import csv
import sys

import torch

from . import BMMCUDA, MBMMCUDA, MinBMMCUDA, TopkBMMCUDA, derive_masks

OPS = ("min_bmm", "topk_bmm", "bmm", "mbmm")
FIELDS = ("op", "l", "n", "k", "variant", "ms", "tflops", "result_mib", "peak_mib",
          "max_abs_err", "index_mismatch")


def sizes(start, stop, step):
    """start, start+step, ... up to and including stop."""
    if start <= 0 or step <= 0 or stop < start:
        raise ValueError("need 0 < start <= stop and step > 0")
    return list(range(start, stop + 1, step))


def _nbytes(result):
    if isinstance(result, torch.Tensor):
        return result.numel() * result.element_size()
    return sum(_nbytes(r) for r in result)


def _time(fn, iters, warmup):
    """(ms per call, last result, allocator peak in bytes above the level before the timed calls)."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    base = torch.cuda.memory_allocated()
    torch.cuda.reset_peak_memory_stats()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(iters):
        out = fn()
    stop.record()
    torch.cuda.synchronize()
    peak = torch.cuda.max_memory_allocated() - base
    return start.elapsed_time(stop) / iters, out, peak


def variants(op, A, B, k_top, dim, mask):
    """name -> callable, in plotting order: the unfused library path, this
    package's product followed by the library reduction, and the fused operator.
    The unfused variants return the product C with their results so that it
    counts towards their footprint."""
    bmm = BMMCUDA()
    if op == "min_bmm":
        fused = MinBMMCUDA()
        return {
            "torch.bmm + min": lambda: (lambda C: (C, *C.min(dim=dim)))(torch.bmm(A, B)),
            "custom bmm + min": lambda: (lambda C: (C, *C.min(dim=dim)))(bmm(A, B)),
            "custom min_bmm": lambda: fused(A, B, dim=dim),
        }
    if op == "topk_bmm":
        fused = TopkBMMCUDA()
        return {
            "torch.bmm + topk": lambda: (lambda C: (C, *C.topk(k_top, dim=dim)))(torch.bmm(A, B)),
            "custom bmm + topk": lambda: (lambda C: (C, *C.topk(k_top, dim=dim)))(bmm(A, B)),
            "custom topk_bmm": lambda: fused(A, B, k=k_top, dim=dim),
        }
    if op == "bmm":
        return {"torch.bmm": lambda: torch.bmm(A, B), "custom bmm": lambda: bmm(A, B)}
    fused = MBMMCUDA(share_mask=False)
    bm, tm, em = derive_masks(mask)
    drop = ~mask
    return {
        "torch.bmm + masked_fill": lambda: torch.bmm(A, B).masked_fill_(drop, 0),
        "custom mbmm": lambda: fused(A, B, bm, tm, em),
    }


def _compare(op, want, got):
    """(max abs value error, number of differing indices) of the fused result."""
    if op in ("bmm", "mbmm"):
        return float((want - got).abs().max()), 0
    _, wv, wi = want
    gv, gi = got
    return float((wv - gv).abs().max()), int((wi != gi).sum())


def run(op, l, ns, k, iters=25, warmup=3, k_top=128, dim=2, seed=0, out=None):
    """Rows (dicts keyed by FIELDS) for every size and variant."""
    if op not in OPS:
        raise ValueError("op must be one of %s" % (OPS,))
    dev = torch.device("cuda:0")
    rows = []
    for n in ns:
        g = torch.Generator(device=dev).manual_seed(seed)
        A = torch.randn(l, n, k, device=dev, generator=g)
        B = torch.randn(l, k, n, device=dev, generator=g)
        mask = None
        if op == "mbmm":
            mask = torch.tril(torch.ones(n, n, device=dev)).bool()[None].expand(l, -1, -1).contiguous()
        flop = 2.0 * l * n * n * k
        first = None
        for name, fn in variants(op, A, B, min(k_top, n), dim, mask).items():
            ms, res, peak = _time(fn, iters, warmup)
            err, mism = ("", "")
            if first is None:
                first = res
            elif name.startswith("custom") and ("+" not in name):
                err, mism = _compare(op, first, res)
            row = dict(op=op, l=l, n=n, k=k, variant=name, ms=round(ms, 5),
                       tflops=round(flop / (ms * 1e-3) / 1e12, 3),
                       result_mib=round(_nbytes(res) / 2**20, 3), peak_mib=round(peak / 2**20, 3),
                       max_abs_err=err, index_mismatch=mism)
            rows.append(row)
            if out is not None:
                print("  ".join("%s=%s" % (f, row[f]) for f in FIELDS if row[f] != ""), file=out, flush=True)
            del res
        del first, A, B, mask
        torch.cuda.empty_cache()
    return rows


def write_csv(rows, path):
    with open(path, "w", newline="") as f:
        w = csv.DictWriter(f, fieldnames=FIELDS)
        w.writeheader()
        w.writerows(rows)


def write_table(rows, path, command=None):
    """A compact text table: one line per size, per variant its milliseconds per
    call and the MiB its results occupy."""
    names = []
    for r in rows:
        if r["variant"] not in names:
            names.append(r["variant"])
    r0 = rows[0]
    with open(path, "w") as f:
        f.write("%s  A[%d,N,%d] @ B[%d,%d,N]: ms per call | MiB held by the results (the product C counts "
                "for the unfused variants)\n" % (r0["op"], r0["l"], r0["k"], r0["l"], r0["k"]))
        if command:
            f.write("command: %s\n" % command)
        f.write("%8s" % "N" + "".join("  %28s" % n for n in names) + "\n")
        for n in sorted({r["n"] for r in rows}):
            line = "%8d" % n
            for name in names:
                sel = [r for r in rows if r["n"] == n and r["variant"] == name]
                line += "  %14.4f | %11.2f" % (sel[0]["ms"], sel[0]["result_mib"]) if sel else " " * 30
            f.write(line + "\n")


def plot(rows, path, quantity="ms"):
    """One line per variant, N on the x axis (the notebooks' figure)."""
    import matplotlib
    matplotlib.use("Agg")
    import matplotlib.pyplot as plt
    fig, ax = plt.subplots(figsize=(15, 10))
    names = []
    for r in rows:
        if r["variant"] not in names:
            names.append(r["variant"])
    for name in names:
        sel = [r for r in rows if r["variant"] == name]
        ax.plot([r["n"] for r in sel], [r[quantity] for r in sel], label=name)
    r0 = rows[0]
    ax.set_title("%s  A[%d,N,%d] B[%d,%d,N]" % (r0["op"], r0["l"], r0["k"], r0["l"], r0["k"]))
    ax.set_xlabel("N")
    ax.set_ylabel({"ms": "milliseconds", "result_mib": "MiB", "peak_mib": "MiB", "tflops": "TFLOP/s"}[quantity])
    ax.grid(True)
    ax.legend()
    fig.savefig(path)
    plt.close(fig)


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--op", choices=OPS, default="min_bmm")
    ap.add_argument("--l", type=int, default=1)
    ap.add_argument("--k", type=int, default=64)
    ap.add_argument("--start", type=int, default=256)
    ap.add_argument("--stop", type=int, default=16384)
    ap.add_argument("--step", type=int, default=256)
    ap.add_argument("--iters", type=int, default=25)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--topk", type=int, default=128)
    ap.add_argument("--dim", type=int, default=2)
    ap.add_argument("--csv", default=None)
    ap.add_argument("--table", default=None, help="write a compact text table (ms and result MiB per variant)")
    ap.add_argument("--plot", default=None)
    ap.add_argument("--plot-quantity", choices=("ms", "tflops", "result_mib", "peak_mib"), default="ms")
    a = ap.parse_args(argv)
    rows = run(a.op, a.l, sizes(a.start, a.stop, a.step), a.k, a.iters, a.warmup, a.topk, a.dim,
               out=sys.stdout)
    if a.csv:
        write_csv(rows, a.csv)
    if a.table:
        write_table(rows, a.table, "python -m custom_matmul_kernels_amd.sweep " + " ".join(argv if argv is not None else sys.argv[1:]))
    if a.plot:
        plot(rows, a.plot, a.plot_quantity)
    return 0


if __name__ == "__main__":
    sys.exit(main())
