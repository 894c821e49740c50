"""bench.py's contract without a GPU: one GPU only, loud failure without one,
and the bookkeeping that ties profiles/traffic.json to the kernel sources."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)


def _run(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True,
                          timeout=300)


def test_more_than_one_gpu_is_refused_with_a_message():
    p = _run("--gpus", "2")
    assert p.returncode == 2 and "not supported" in p.stderr and p.stdout == ""


def test_no_gpu_is_an_error_not_a_cpu_run():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present: the benchmark would run")
    p = _run("--steps", "1", "--warmup", "0")
    assert p.returncode == 3 and "no CPU fallback" in p.stderr and p.stdout == ""


class _Tuning:
    def __init__(self, values):
        self.values = values

    def get_tuning(self, key):
        return self.values[key]


def test_counter_traffic_is_tied_to_the_kernel_sources(monkeypatch):
    """The bench line carries the HBM bytes of the committed counter runs only for
    the kernel sources, tuning and size they were taken with; the committed table
    must belong to the sources in the tree (re-run the profiles after a kernel change)."""
    import bench
    with open(os.path.join(ROOT, "profiles", "traffic.json")) as fh:
        table = json.load(fh)
    assert table["source_sha256_16"] == bench.source_hash(), \
        "profiles/traffic.json was recorded with other kernel sources: regenerate the counter summaries"
    lib = _Tuning(dict(table["tuning"]))
    got, why = bench.profiled_traffic("cfg2", "steps", "k_add_rows", lib, 1.0)
    assert why is None and got == table["entries"]["cfg2:steps:k_add_rows"]
    assert abs(got / (3 * 8 * (32 << 20) * 2) - 1) < 0.01              # ~ the algorithmic bytes of one launch (= one step)
    # another size, another tuning, an unknown row, other sources: no figure, and the reason
    assert bench.profiled_traffic("cfg2", "steps", "k_add_rows", lib, 0.5)[0] is None
    other = _Tuning(dict(table["tuning"], unroll=8))
    assert bench.profiled_traffic("cfg2", "steps", "k_add_rows", other, 1.0)[0] is None
    assert "no counter run" in bench.profiled_traffic("cfg9", "steps", "k_add_rows", lib, 1.0)[1]
    monkeypatch.setattr(bench, "source_hash", lambda: "0" * 16)
    got, why = bench.profiled_traffic("cfg2", "steps", "k_add_rows", lib, 1.0)
    assert got is None and "other kernel sources" in why


def test_every_profiled_row_is_a_row_of_the_default_run():
    import bench
    with open(os.path.join(ROOT, "profiles", "traffic.json")) as fh:
        entries = json.load(fh)["entries"]
    rows = set(bench.ALL_ROWS) | {("cfg2", "steps")}
    for key in entries:
        workload, mode, kernel = key.split(":")
        assert (workload, mode) in rows, key
        assert kernel.startswith("k_")
