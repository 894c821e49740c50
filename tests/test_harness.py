"""The raw-collectives harness (flags, sweep, --test, CSV) on virtual ranks."""
import csv
import os
import sys

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "sc2025-pccl-reproducer_amd"))


@pytest.mark.parametrize("extra", [["--pccl-recursive-alg"], [], ["--pccl-disable-cpp-backend"],
                                   ["--library", "mpi"], ["--dtype", "bf16", "--pccl-recursive-alg"]])
def test_reduce_scatter_harness(tmp_path, extra):
    from benchmark_raw_collectives import reduce_scatter
    path = reduce_scatter.main(["--num-gpus-per-node", "4", "--machine", "mi355x", "--test", "--world-size", "8",
                                "--sizes", "1", "4", "--data-dir", str(tmp_path)] + extra)
    rows = list(csv.reader(open(path)))
    assert rows[0][:4] == ["gpu_count", "slurm_job_id", "output_size", "unit"] and rows[0][4].startswith("time_")
    assert [r[2] for r in rows[1:]] == ["1", "4"] and all(float(r[4]) > 0 for r in rows[1:])
    assert os.path.basename(path) == "gpus_8_slurm_unknown.csv"


@pytest.mark.parametrize("extra", [["--pccl-recursive-alg"], [], ["--pccl-disable-cpp-backend", "--pccl-recursive-alg"],
                                   ["--library", "mpi"], ["--dtype", "bf16"]])
def test_all_gather_harness(tmp_path, extra):
    from benchmark_raw_collectives import all_gather
    path = all_gather.main(["--num-gpus-per-node", "2", "--machine", "mi355x", "--test", "--world-size", "8",
                            "--sizes", "1", "4", "--data-dir", str(tmp_path)] + extra)
    rows = list(csv.reader(open(path)))
    assert len(rows) == 3 and rows[0][4].startswith("time_")


def test_xccl_is_refused():
    from benchmark_raw_collectives import reduce_scatter
    with pytest.raises(SystemExit, match="not available on virtual ranks"):
        reduce_scatter.main(["--num-gpus-per-node", "4", "--machine", "x", "--library", "xccl"])
