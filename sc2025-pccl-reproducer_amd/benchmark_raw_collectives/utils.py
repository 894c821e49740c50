"""Timing and comparison helpers of the raw-collectives harness
(benchmark_raw_collectives/utils.py of the reference), for virtual ranks.

The reference runs one process per GPU; here one Python thread per virtual
rank executes the same per-rank loop and all of them enqueue on one stream.
Timing keeps the reference's convention: 5 warm-up calls, then the mean of 20
timed calls between two device events (benchmark_raw_collectives/utils.py:16-33).
"""
import os

import torch
from torch.profiler import record_function


def world_size_from_env(default: int = 8) -> int:
    """SLURM_NTASKS names the number of ranks in the reference
    (benchmark_raw_collectives/utils.py:8); here it is the number of virtual ranks."""
    return int(os.getenv("SLURM_NTASKS", os.getenv("PCCL_VIRTUAL_RANKS", str(default))))


def time_something(comm, fn, *args, warmup_iters=5, timed_iters=20, **kwargs):
    """Per-rank timing loop.  Every rank calls it; the events are recorded on
    the shared stream between barriers, so every rank gets the same figure."""
    start_event = torch.cuda.Event(enable_timing=True)
    end_event = torch.cuda.Event(enable_timing=True)
    # the ranges a torch profiler run shows, named as the reference names them
    # (benchmark_raw_collectives/utils.py:20,27)
    for i in range(warmup_iters):
        with record_function(f"warmup_{i}"):
            fn(*args, **kwargs)
    comm.Barrier()
    torch.cuda.synchronize()
    if comm.Get_rank() == 0:
        start_event.record()
    comm.Barrier()
    for i in range(timed_iters):
        with record_function(f"iteration_{i}"):
            fn(*args, **kwargs)
    comm.Barrier()
    if comm.Get_rank() == 0:
        end_event.record()
    torch.cuda.synchronize()
    comm.Barrier()
    return start_event.elapsed_time(end_event) / timed_iters if comm.Get_rank() == 0 else None


def allclose(x, y, pct=2.0, rtol=1e-5, atol=1e-8):
    """The reference's acceptance test: isclose(rtol=1e-5) with at most `pct`
    percent of the elements off (benchmark_raw_collectives/utils.py:35-42).
    bfloat16 sums are rounded at every hop, so callers widen the tolerance to
    one bf16 ulp (2^-8 relative) per hop for them."""
    mask = torch.isclose(x, y, rtol=rtol, atol=atol)
    pct_diff = (mask.numel() - mask.sum()) / mask.numel() * 100
    if pct_diff > pct:
        print(x[torch.logical_not(mask)], y[torch.logical_not(mask)])
        print("{:.2f}% of values not close.".format(pct_diff))
        return False
    return True
