#!/usr/bin/env python3
"""all_gather sweep on virtual ranks: the raw-collectives benchmark of the
reference (benchmark_raw_collectives/all_gather.py) on one MI355X.

    python -m benchmark_raw_collectives.all_gather --num-gpus-per-node 4 --machine mi355x \\
           --library pccl --pccl-recursive-alg --test [--world-size 8] [--dtype bf16]

Same flags, size sweep (1 .. 1024 MB of output per rank), timing convention and
CSV layout as the reference, plus bytes / GB/s / share of the HBM peak.
"""
import csv
import os
import sys
from argparse import ArgumentParser

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))

from pccl import ProcessGroups, VirtualWorld, all_gather_2D, kernels, _all_gather  # noqa: E402
from pccl.build_kernels import build as build_pccl  # noqa: E402
from benchmark_raw_collectives.utils import allclose, time_something, world_size_from_env  # noqa: E402

HBM_PEAK_GBPS = 8000.0


def parse_args(argv=None):
    parser = ArgumentParser()
    parser.add_argument("--num-gpus-per-node", type=int, required=True,
                        help="specify number of GPUs/GCDs per node")
    parser.add_argument("--machine", type=str, required=True,
                        help="specify the machine you are running on. Will be used to create folders")
    parser.add_argument("--library", type=str, choices=["pccl", "mpi", "xccl"], default="pccl")
    parser.add_argument("--pccl-disable-cpp-backend", dest="use_pccl_cpp_backend", action="store_false",
                        help="Disable the native backend in PCCL. Will fall back to the per-rank Python algorithms.")
    parser.add_argument("--test", action="store_true", help="test for correctness")
    parser.add_argument("--pccl-recursive-alg", action="store_true",
                        help="Use the recursive doubling algorithm for PCCL.")
    parser.add_argument("--dtype", choices=["fp32", "bf16", "fp16"], default="fp32")
    parser.add_argument("--world-size", type=int, default=None,
                        help="number of virtual ranks (default: $SLURM_NTASKS or 8)")
    parser.add_argument("--sizes", type=int, nargs="*", default=None, help="output sizes per rank in MB")
    parser.add_argument("--data-dir", default="./data")
    parser.add_argument("--dump", default=None, metavar="FILE.npz",
                        help="write the inputs and outputs of every rank for the LAST size of the sweep (raw element "
                             "bits, one row per rank), so that a checker can recompute them")
    return parser.parse_args(argv)


def main(argv=None):
    args = parse_args(argv)
    if args.library == "xccl":
        raise SystemExit("--library xccl runs torch.distributed collectives over real process groups; "
                         "it is not available on virtual ranks")
    if args.use_pccl_cpp_backend:
        build_pccl()
    world_size = args.world_size or world_size_from_env()
    gpu_count = world_size
    slurm_job_id = os.getenv("SLURM_JOB_ID", "unknown")
    sizes = np.array(args.sizes if args.sizes else [1, 2, 4, 8, 16, 32, 64, 128, 256, 512, 1024])
    unit = "MB"
    use_rd = args.pccl_recursive_alg
    dtype = {"fp32": torch.float32, "bf16": torch.bfloat16, "fp16": torch.float16}[args.dtype]
    esize = 4 if args.dtype == "fp32" else 2
    library = args.library
    if library == "pccl":
        library += "_cpp" if args.use_pccl_cpp_backend else "_py"
        library += "_rec" if use_rd else "_ring"

    device = torch.device("cuda", 0)
    world = VirtualWorld(world_size, device)
    data_folder = f"{args.data_dir}/all_gather/{args.machine}"
    os.makedirs(data_folder, exist_ok=True)
    csv_filename = os.path.join(data_folder, f"gpus_{gpu_count}_slurm_{slurm_job_id}.csv")

    with open(csv_filename, "w", newline="") as f:
        writer = csv.writer(f)
        writer.writerow(["gpu_count", "slurm_job_id", "output_size", "unit", f"time_{library}",
                         "bytes", "GBps", "pct_peak"])
        for size in sizes:
            print(f"output size = {size} {unit}")
            output_numel = int(size) * 2 ** 20 // esize
            output_numel -= output_numel % world_size
            input_numel = output_numel // world_size
            gen = torch.Generator(device=device).manual_seed(1234)
            inputs = [torch.randn(input_numel, generator=gen, device=device).to(dtype) for _ in range(world_size)]
            outputs = [torch.empty(output_numel, dtype=dtype, device=device) for _ in range(world_size)]

            def rank_main(comm):
                r = comm.Get_rank()
                if args.library == "pccl":
                    group = ProcessGroups(args.num_gpus_per_node, world_size // args.num_gpus_per_node,
                                          inner_group_backend="mpi", outer_group_backend="mpi", comm=comm)
                    return time_something(comm, all_gather_2D, outputs[r], inputs[r], group=group, use_rd=use_rd,
                                          use_pccl_cpp_backend=args.use_pccl_cpp_backend)
                return time_something(comm, _all_gather, outputs[r], inputs[r], group=comm, use_rd=False)

            time_ms = world.run(rank_main)[0]

            if args.test:
                gold = torch.cat(inputs)
                for r in range(world_size):
                    assert allclose(outputs[r].float(), gold.float())

            # bytes the job moves: one fused pass reads every shard once and writes it into every
            # output; a per-step replay reads and writes every byte of every output (2 * bytes each)
            one_pass = args.library == "mpi" or (args.use_pccl_cpp_backend and
                                                 kernels.mode_code(None) == kernels.MODE_FUSED)
            if one_pass:
                job_bytes = (world_size + 1) * output_numel * esize
            else:
                job_bytes = 2 * output_numel * esize * world_size
            gbps = job_bytes / (time_ms * 1e-3) / 1e9
            print(f"time_{library} = {time_ms:.3f} ms  ({gbps:.0f} GB/s of bytes moved)")
            print("===============================")
            writer.writerow([gpu_count, slurm_job_id, size, unit, time_ms, job_bytes, round(gbps, 1),
                             round(100 * gbps / HBM_PEAK_GBPS, 2)])
            if args.dump and size == sizes[-1]:
                bits = torch.int32 if dtype == torch.float32 else torch.int16
                np.savez(args.dump,
                         inputs=torch.stack([t.view(bits) for t in inputs]).cpu().numpy(),
                         outputs=torch.stack([t.view(bits) for t in outputs]).cpu().numpy())
            del inputs, outputs
        if args.test:
            print("All tests passed! PCCL outputs match the concatenation of the inputs!")
    return csv_filename


if __name__ == "__main__":
    main()
