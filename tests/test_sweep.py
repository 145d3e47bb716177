"""The size-sweep harness: host logic without a GPU, one short sweep of every
operator on the GPU."""
import csv

import pytest

from custom_matmul_kernels_amd import sweep


def test_sizes_and_arguments():
    assert sweep.sizes(256, 1024, 256) == [256, 512, 768, 1024]
    assert sweep.sizes(100, 100, 7) == [100]
    for bad in ((0, 10, 1), (10, 5, 1), (1, 5, 0)):
        with pytest.raises(ValueError):
            sweep.sizes(*bad)
    with pytest.raises(ValueError):
        sweep.run("nope", 1, [8], 8)


def test_csv_and_plot_from_rows(tmp_path):
    rows = [dict(op="min_bmm", l=1, n=n, k=64, variant=v, ms=0.1 * n, tflops=1.0, result_mib=2.0,
                 peak_mib=3.0, max_abs_err="", index_mismatch="")
            for n in (256, 512) for v in ("torch.bmm + min", "custom min_bmm")]
    path = tmp_path / "s.csv"
    sweep.write_csv(rows, path)
    back = list(csv.DictReader(open(path)))
    assert [r["variant"] for r in back] == [r["variant"] for r in rows]
    assert tuple(back[0].keys()) == sweep.FIELDS
    pytest.importorskip("matplotlib")
    sweep.plot(rows, tmp_path / "s.png", "ms")
    assert (tmp_path / "s.png").stat().st_size > 0


@pytest.mark.gpu
@pytest.mark.parametrize("op,nvar", [("min_bmm", 3), ("topk_bmm", 3), ("bmm", 2), ("mbmm", 2)])
def test_short_sweep_on_gpu(device, op, nvar):
    print("sweep", op, flush=True)
    ns = [128, 200]
    rows = sweep.run(op, 2, ns, 40, iters=2, warmup=1)
    assert len(rows) == nvar * len(ns)
    for r in rows:
        assert r["ms"] > 0 and r["result_mib"] > 0
    fused = [r for r in rows if r["variant"].startswith("custom") and "+" not in r["variant"]]
    assert len(fused) == len(ns)
    for r in fused:
        # the comparison is against the GPU library product, whose rounding differs:
        # positions whose products are closer than that may swap
        assert r["max_abs_err"] <= 1e-3 * 40 ** 0.5 and r["index_mismatch"] <= 20
    if op in ("min_bmm", "topk_bmm"):
        # the fused operator leaves no product behind: its results are smaller
        for n in ns:
            sel = {r["variant"]: r["result_mib"] for r in rows if r["n"] == n}
            assert sel["custom " + op] < sel["torch.bmm + " + op.split("_")[0]]
