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


def _harness_args(tmp_path, per_node, dump, extra):
    return ["--num-gpus-per-node", str(per_node), "--machine", "mi355x", "--test", "--world-size", "8",
            "--sizes", "1", "2", "--data-dir", str(tmp_path), "--dump", dump] + extra


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("extra,oracle_alg", [
    ([], "ring"), (["--pccl-recursive-alg"], "recursive"),
    (["--pccl-disable-cpp-backend"], "ring"), (["--pccl-disable-cpp-backend", "--pccl-recursive-alg"], "recursive"),
    (["--library", "mpi"], None)])
def test_reduce_scatter_harness_outputs_match_the_oracle(tmp_path, extra, oracle_alg, dtype):
    """What the harness computed for the last size of its sweep, bit for bit:
    --library pccl against the two-level oracle (permute, inner, outer
    reduce_scatter) for both algorithms and both backends, --library mpi (the
    library's Reduce_scatter_block) against the flat ring oracle."""
    import numpy as np
    from benchmark_raw_collectives import reduce_scatter
    from oracle import pccl_oracle as O
    dump = str(tmp_path / "last.npz")
    reduce_scatter.main(_harness_args(tmp_path, 4, dump, ["--dtype", dtype] + extra))
    d = np.load(dump)
    odt = O.F32 if dtype == "fp32" else O.BF16
    ins = [row.view(np.float32) if dtype == "fp32" else row.view(np.uint16) for row in d["inputs"]]
    if oracle_alg is None:
        want = O.ring_reduce_scatter(ins, odt)
    else:
        want = O.reduce_scatter_2d(ins, 4, 2, odt, oracle_alg)
    assert d["outputs"].shape[0] == 8 and d["outputs"].shape[1] * 8 == d["inputs"].shape[1]
    for r in range(8):
        assert np.array_equal(d["outputs"][r].view(np.uint8), np.ascontiguousarray(want[r]).view(np.uint8)), f"rank {r}"


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("extra,oracle_alg", [
    ([], "ring"), (["--pccl-recursive-alg"], "recursive"),
    (["--pccl-disable-cpp-backend"], "ring"), (["--pccl-disable-cpp-backend", "--pccl-recursive-alg"], "recursive"),
    (["--library", "mpi"], None)])
def test_all_gather_harness_outputs_match_the_oracle(tmp_path, extra, oracle_alg, dtype):
    import numpy as np
    from benchmark_raw_collectives import all_gather
    from oracle import pccl_oracle as O
    dump = str(tmp_path / "last.npz")
    all_gather.main(_harness_args(tmp_path, 2, dump, ["--dtype", dtype] + extra))
    d = np.load(dump)
    ins = [np.ascontiguousarray(row).view(np.uint8) for row in d["inputs"]]
    want = O.ring_all_gather(ins) if oracle_alg is None else O.all_gather_2d(ins, 2, 4, oracle_alg)
    for r in range(8):
        assert np.array_equal(np.ascontiguousarray(d["outputs"][r]).view(np.uint8), want[r]), f"rank {r}"


def test_xccl_is_refused():
    from benchmark_raw_collectives import reduce_scatter
    with pytest.raises(SystemExit, match="not available on virtual ranks"):
        reduce_scatter.main(["--num-gpus-per-node", "4", "--machine", "x", "--library", "xccl"])
