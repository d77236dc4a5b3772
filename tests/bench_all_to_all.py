"""Eager latency table of AllToAll.dispatch / .combine through the per-rank Python API.

The loopback counterpart of the reference's ``tests/bench_all_to_all.py:31-222`` (same model
shapes, :252-268; same event-timed loop: 10 samples per run, 10 warm-up runs, 20 measured runs,
mean and standard deviation; same one-way payload formulas, :131-139).  All simulated ranks live
in this process, so one "dispatch" below is the sum of every rank's call, launched from the
host without a graph: it measures what a caller of the reference API sees, Python included.
``bench.py`` at the repository root measures the workloads of the benchmark plan in every
launch form (its ``per_rank_api_step_us`` is this path on those workloads).

    python -m tests.bench_all_to_all [--ranks 8] [--dp-size 1] [--in-dtype float8_e4m3fn]
"""

# ruff: noqa: T201
from __future__ import annotations

import argparse
import os
import sys

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "pplx-kernels_amd"))

from tests.all_to_all_utils import DeviceStep, WorkloadSpec, generate  # noqa: E402

MODELS = [(64, 6, 2048), (256, 8, 7168)]  # V2-Lite, R1: experts, experts per token, hidden dim
TOKENS = [1, 4, 8, 16, 32, 64, 128]
SAMPLES, WARMUP_RUNS, MEASURED_RUNS = 10, 10, 20


def bench_one(spec: WorkloadSpec) -> tuple[int, int, torch.Tensor]:
    from pplx_kernels import AllToAll

    groups = generate(spec)
    for g in groups:
        g.n = spec.max_num_tokens  # the reference benches full batches (use_max_tokens=True)
    step = DeviceStep(spec, groups)
    ranks = [
        AllToAll.intranode(
            max_num_tokens=spec.max_num_tokens,
            num_experts=spec.num_experts,
            experts_per_token=spec.experts_per_token,
            rank=r,
            world_size=spec.world_size,
            dp_size=spec.dp_size,
            hidden_dim=spec.hidden_dim,
            hidden_dim_bytes=spec.hidden_dim_bytes,
            hidden_dim_scale_bytes=spec.hidden_dim_scale_bytes,
            group_name=f"bench-{spec.num_experts}-{spec.max_num_tokens}",
        )
        for r in range(spec.world_size)
    ]
    pairs = spec.num_dp_groups * spec.max_num_tokens * spec.experts_per_token
    dispatch_bytes = pairs * (spec.hidden_dim_bytes + spec.hidden_dim_scale_bytes)
    combine_bytes = pairs * spec.hidden_dim * spec.out_dtype.itemsize
    stream = torch.cuda.current_stream()

    def run() -> tuple[float, float]:
        events = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(SAMPLES)]
        for e0, e1, e2 in events:
            e0.record(stream)
            step.dispatch_per_rank(ranks)
            e1.record(stream)
            step.combine_per_rank(ranks)
            e2.record(stream)
        stream.synchronize()
        d = sum(e0.elapsed_time(e1) for e0, e1, _ in events) * 1e3 / SAMPLES
        c = sum(e1.elapsed_time(e2) for _, e1, e2 in events) * 1e3 / SAMPLES
        return d, c

    for _ in range(WARMUP_RUNS):
        run()
    result = torch.tensor([run() for _ in range(MEASURED_RUNS)])
    for a in ranks:
        a.destroy()
    return dispatch_bytes, combine_bytes, result


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--ranks", type=int, default=8, help="simulated EP ranks (all on this GPU)")
    ap.add_argument("--dp-size", type=int, default=1)
    ap.add_argument("--in-dtype", default="float8_e4m3fn", choices=["bfloat16", "float16", "float8_e4m3fn"])
    ap.add_argument("--out-dtype", default="bfloat16", choices=["bfloat16", "float16"])
    ap.add_argument("--quick", action="store_true", help="two token counts per model, fewer runs")
    args = ap.parse_args()
    global TOKENS, WARMUP_RUNS, MEASURED_RUNS
    if args.quick:
        TOKENS, WARMUP_RUNS, MEASURED_RUNS = [1, 128], 2, 4
    if not torch.cuda.is_available():
        sys.exit("bench_all_to_all: no GPU visible")
    in_dtype, out_dtype = getattr(torch, args.in_dtype), getattr(torch, args.out_dtype)
    header = ["E", "E/tok", "tok", "dim", "Dispatch_lat", "Dispatch_bw", "Dispatch_bytes",
              "Combine_lat", "Combine_bw", "Combine_bytes"]  # fmt: skip
    print(f"EP={args.ranks} DP={args.ranks // args.dp_size} (simulated ranks on one GPU, eager per-rank calls)")
    print("\t".join(header))
    for experts, k, hidden in MODELS:
        if args.ranks > experts or experts % args.ranks:
            continue
        for tokens in TOKENS:
            spec = WorkloadSpec(
                f"{experts}x{tokens}", 70, args.ranks, experts, k, hidden, tokens, in_dtype,
                dp_size=args.dp_size, out_dtype=out_dtype, expert_y_dtype=out_dtype, tokens="max",
            )  # fmt: skip
            d_bytes, c_bytes, res = bench_one(spec)
            d, c = res[:, 0], res[:, 1]
            row = [
                f"{experts}", f"{k}", f"{tokens}", f"{hidden}",
                f"{d.mean():4.1f}us ± {d.std():4.1f}us", f"{d_bytes / d.mean() / 1e3:2.3f}GB/s", f"{d_bytes}",
                f"{c.mean():4.1f}us ± {c.std():4.1f}us", f"{c_bytes / c.mean() / 1e3:2.3f}GB/s", f"{c_bytes}",
            ]  # fmt: skip
            print("\t".join(row), flush=True)


if __name__ == "__main__":
    main()
