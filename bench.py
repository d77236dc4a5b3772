"""Benchmark of the MoE dispatch + combine hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload C2] [--only] [--no-cpu]

A *step* is one dispatch + one combine over all simulated ranks of a workload, inputs resident
in HBM.  To keep the working set from living in the 256 MB last-level cache between steps, the
steps rotate over several independent buffer sets, so every timed step touches memory that was
last used several steps ago.

Prints ONE JSON line.  ``value`` is the mean step latency in microseconds on the workload the
metric is quoted on (C2: DeepSeek-V3 shape, 128 tokens/rank, 8 simulated ranks), over exactly
``--steps`` steps in one timed region.  Every workload C1..C5 is measured in the same three
launch forms under fixed keys, on the same rotating buffer sets:

* ``bound_eager_step_us`` (= ``step_us``): eager launches of a step whose arguments were checked
  and packed once (``LoopbackWorld.bind``: two library calls per step);
* ``graph_step_us``: the same step captured into one hipGraph per buffer set and replayed;
* ``per_rank_api_step_us``: the reference's own call path, ``AllToAll.dispatch`` once per
  simulated rank and then ``AllToAll.combine`` once per rank, eagerly, arguments checked on
  every call (what ``tests/bench_all_to_all.py`` of the reference times per rank).

``bound_eager_host_us_per_call`` is what the launching thread spends on one of those library
calls (issued into an empty queue).  Every timed region is exactly ``--steps`` steps between two
synchronisations; in front of it come at least 64 untimed calls (more if ``--warmup`` says so)
and, behind the synchronisation, 200 us of busy host, so that a region of 20 decode steps is not
dominated by a thread that has just woken up (see ``wake_host``).

The decode shape C3 additionally carries ``graph_replay_1000x_us``: ONE captured graph over ONE
buffer set replayed 1000 times, the form its specification names; 12.5 MB replayed back to back
stay in the last-level cache, so that figure is cache-resident and carries no HBM fraction;
``bound_eager_1000x_us`` is the same thousand steps on that one buffer set as eager launches.
``roofline`` is for the dominant kernel of the headline workload (``combine_gather``):
algorithmic bytes per launch divided by its mean duration, measured with HIP events around graph
replays that contain only launches of that kernel; ``traffic`` is read from the rocprofv3 counter
summary under ``profiles/`` when that summary was made with the library that is running.  Every
workload carries a ``cpu_baseline``: the oracle's vectorised torch CPU port of the same step on
the same inputs, on this host's cores.
"""

from __future__ import annotations

import argparse
import json
import os
import re
import statistics
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (os.path.join(ROOT, "pplx-kernels_amd"), ROOT):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBPS = 8000.0  # MI355X published HBM3E peak
LLC_BYTES = 256 << 20
GRAPH_REPLAYS_C3 = 1000


def measured_traffic_bytes(workload: str, kernel: str, build_id: str):
    """(HBM bytes per launch of `kernel`, note) from profiles/hbm_traffic_<workload>.txt (rocprofv3
    --pmc FETCH_SIZE / WRITE_SIZE, scaled by a copy of known size in the same run).  The summary
    names the library it was measured with; bytes are None when it is missing or was made with
    another build.  Counters cannot be read from inside this script."""
    path = os.path.join(ROOT, "profiles", f"hbm_traffic_{workload}.txt")
    try:
        lines = open(path).read().splitlines()
    except OSError:
        return None, f"no counter summary {os.path.relpath(path, ROOT)}"
    measured_with = None
    for line in lines:
        m = re.search(r"library build id:\s*([0-9a-f]+)", line)
        if m:
            measured_with = m.group(1)
    if measured_with != build_id:
        return None, (
            f"{os.path.relpath(path, ROOT)} was measured with library build {measured_with}, "
            f"this run uses {build_id}: counters not carried over"
        )
    for line in lines:
        fields = line.split()
        if fields and fields[0] == kernel and re.fullmatch(r"[0-9.]+", fields[-1]):
            return float(fields[-1]) * 1e6, f"{os.path.relpath(path, ROOT)} (library build {build_id})"
    return None, f"{os.path.relpath(path, ROOT)} has no line for {kernel}"


def build_steps(spec, groups, cap, n_sets):
    from pplx_kernels.workloads import DeviceStep

    steps = []
    gen = torch.Generator(device="cuda").manual_seed(7)
    for _ in range(n_sets):
        st = DeviceStep(spec, groups, cap=cap)
        # N(0,1) expert outputs in the rows that will be read; fill in slabs to bound memory
        for r in range(spec.world_size):
            st.expert_y_all[r].copy_(
                torch.randn(st.expert_y_all[r].shape, generator=gen, device="cuda", dtype=torch.bfloat16)
            )
        steps.append(st)
    return steps


HOST_WAKE_US = 200.0
# Untimed calls in front of every timed region, whatever --warmup says: every buffer set (up to
# eight) is touched several times and the launch path of the host is warm before 20 steps of
# 10 us each are timed.
MIN_WARMUP_CALLS = 64


def wake_host():
    """Keeps the launching thread busy for a moment between the synchronisation in front of a
    timed region and its first launch.  A blocking wait parks the thread, and the launches it
    issues right after waking are two to three times slower than in a running loop; a region of
    20 decode steps (0.2 ms, two launches of host-bound size each) cannot amortise that: without
    this, 20-step regions of C3 read 11.2-18.5 us per step, with it 10.5-10.9, as 200-step
    regions do.  Steps whose kernels outlast the host's part of a launch do not notice."""
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e6 < HOST_WAKE_US:
        pass


def time_graphs(graphs, order, stream, warmup, repeats=1):
    """Mean microseconds per graph launch over `order` (a list of graph indices), HIP events
    on the launch stream."""
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    with torch.cuda.stream(stream):
        for i in range(max(warmup, MIN_WARMUP_CALLS)):
            graphs[order[i % len(order)]].replay(stream)
        stream.synchronize()
        torch.cuda.synchronize()
        wake_host()
        start.record(stream)
        for _ in range(repeats):
            for i in order:
                graphs[i].replay(stream)
        end.record(stream)
        stream.synchronize()
        torch.cuda.synchronize()
    return start.elapsed_time(end) * 1e3 / (len(order) * repeats)


def time_steps(run, order, stream, warmup):
    """Mean microseconds per call of run(i) over `order` (buffer-set indices) in ONE timed region,
    HIP events on the launch stream, which is also the current stream inside run."""
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    with torch.cuda.stream(stream):
        for i in range(max(warmup, MIN_WARMUP_CALLS)):
            run(order[i % len(order)])
        stream.synchronize()
        wake_host()
        start.record(stream)
        for i in order:
            run(i)
        end.record(stream)
        stream.synchronize()
    return start.elapsed_time(end) * 1e3 / len(order)


def host_cost(run, n_sets, stream, calls=16):
    """Host microseconds per call of run(i), issued into an empty queue (the launches are
    asynchronous: this is what the launching thread spends, whatever the kernels take)."""
    best = None
    with torch.cuda.stream(stream):
        for _ in range(5):
            stream.synchronize()
            wake_host()
            t0 = time.perf_counter()
            for i in range(calls):
                run(i % n_sets)
            t = (time.perf_counter() - t0) * 1e6 / calls
            best = t if best is None else min(best, t)
        stream.synchronize()
    return best


def capture(world, stream, body):
    with torch.cuda.stream(stream):
        body()  # eager once: binds tables, warms code objects
        stream.synchronize()
        with world.capture() as cap:
            body()
    return cap.graph


EXTRA_REGIONS = 4  # further timed regions of the same length, for the spread


def measure_workload(name, spec, steps_k, warmup):
    from pplx_kernels.workloads import expert_counts, generate, make_world

    groups = generate(spec)
    counts = expert_counts(groups, spec.num_experts)
    cap = max(int(counts.max()), 1)
    full_cap = spec.max_num_tokens * spec.num_dp_groups
    if spec.num_experts * full_cap * spec.hidden_dim * 3 < (8 << 30):
        cap = full_cap  # small enough: use the reference's own sizing
    # enough buffer sets that a step's data is evicted before it is used again
    probe_bytes = sum(g.n for g in groups) * spec.experts_per_token * spec.hidden_dim * 3
    n_sets = max(2, min(8, int(2.5 * LLC_BYTES / max(probe_bytes, 1)) + 1))
    per_set = spec.num_experts * cap * spec.hidden_dim * (spec.in_dtype.itemsize + 2)
    n_sets = max(1, min(n_sets, int((160 << 30) // max(per_set, 1))))
    steps = build_steps(spec, groups, cap, n_sets)
    disp_b, comb_b = steps[0].algorithmic_bytes()
    world = make_world(spec, group_name=f"bench-{name}")
    stream = torch.cuda.Stream()
    torch.cuda.synchronize()
    order = [i % n_sets for i in range(steps_k)]

    # 1. eager launches of steps packed once (LoopbackWorld.bind): two library calls per step
    bound = [st.bind_world(world) for st in steps]
    bound_us = time_steps(lambda i: (bound[i].dispatch(stream), bound[i].combine(stream)), order, stream, warmup)
    more = [
        time_steps(lambda i: (bound[i].dispatch(stream), bound[i].combine(stream)), order, stream, 0)
        for _ in range(EXTRA_REGIONS)
    ]
    host_us = host_cost(lambda i: (bound[i].dispatch(stream), bound[i].combine(stream)), n_sets, stream) / 2
    d_us = time_steps(lambda i: bound[i].dispatch(stream), order, stream, warmup)
    c_us = time_steps(lambda i: bound[i].combine(stream), order, stream, warmup)

    # 2. the reference's call path: one AllToAll.dispatch per simulated rank, then one
    # AllToAll.combine per rank (src/pplx_kernels/all_to_all.py:27-81), eagerly, on the same sets
    ranks = world.ranks
    per_rank_us = time_steps(
        lambda i: (steps[i].dispatch_per_rank(ranks), steps[i].combine_per_rank(ranks)), order, stream, warmup
    )

    # 3. the same step as a captured hipGraph, one per buffer set
    def both(st):
        return lambda: (st.dispatch_world(world), st.combine_world(world))

    graphs = [capture(world, stream, both(st)) for st in steps]
    graph_us = time_graphs(graphs, order, stream, warmup)
    replay_1000 = eager_1000 = None
    if name == "C3":
        # the form the decode shape is specified in: ONE graph, replayed 1000 times back to back ...
        replay_1000 = time_graphs([graphs[0]], [0], stream, warmup, GRAPH_REPLAYS_C3)
        # ... and the same 1000 steps on that one buffer set as eager launches of the bound step
        eager_1000 = time_steps(
            lambda i: (bound[0].dispatch(stream), bound[0].combine(stream)), [0] * GRAPH_REPLAYS_C3, stream, warmup
        )
    for g in graphs:
        g.destroy()
    del bound

    pairs = int(sum(g.n for g in groups) * spec.experts_per_token)
    spread = [bound_us] + more
    out = {
        "workload": spec.name,
        "tokens": int(sum(g.n for g in groups)),
        "pairs": pairs,
        "rows_per_expert_capacity": cap,
        "buffer_sets": n_sets,
        "steps_timed": len(order),
        "launch_form": "bound_eager",
        "step_us": bound_us,
        "step_us_regions": {
            "n": len(spread),
            "mean": statistics.mean(spread),
            "std": statistics.pstdev(spread),
            "min": min(spread),
            "note": f"{len(spread)} timed regions of {len(order)} steps each; step_us is the first",
        },
        "bound_eager_step_us": bound_us,
        "bound_eager_host_us_per_call": host_us,
        "graph_step_us": graph_us,
        "per_rank_api_step_us": per_rank_us,
        "per_rank_api_calls_per_step": 2 * spec.world_size,
        "dispatch_us": d_us,
        "combine_us": c_us,
        "dispatch_bytes": disp_b,
        "combine_bytes": comb_b,
        "step_hbm_frac": (disp_b + comb_b) / bound_us / 1e3 / HBM_PEAK_GBPS,
        "dispatch_hbm_frac": disp_b / d_us / 1e3 / HBM_PEAK_GBPS,
        "combine_hbm_frac": comb_b / c_us / 1e3 / HBM_PEAK_GBPS,
        "step_GBps": (disp_b + comb_b) / bound_us / 1e3,
        # the reference bench's one-way payload figures (tests/bench_all_to_all.py:131-139):
        # pairs x bytes per dispatched token, pairs x bytes per combined row
        "dispatch_payload_GBps": pairs * (spec.hidden_dim_bytes + spec.hidden_dim_scale_bytes) / d_us / 1e3,
        "combine_payload_GBps": pairs * spec.hidden_dim * spec.out_dtype.itemsize / c_us / 1e3,
    }
    if replay_1000 is not None:
        out["graph_replay_1000x_us"] = replay_1000
        out["bound_eager_1000x_us"] = eager_1000
        out["graph_replay_1000x_note"] = (
            f"one hipGraph over one buffer set replayed {GRAPH_REPLAYS_C3} times back to back: the "
            f"{(disp_b + comb_b) / 1e6:.1f} MB of a step stay in the 256 MB last-level cache, so this is a "
            "cache-resident latency and no HBM fraction is derived from it"
        )
    assert world.faults() == 0, "device-side fault bits set during the benchmark"
    world.destroy()
    return out, groups, steps


def combine_kernel_roofline(name, spec, steps, comb_b, steps_k):
    """Roofline of the dominant kernel: graphs holding back-to-back combine_gather launches only,
    rotating buffer sets; mean launch duration by HIP events on the launch stream."""
    from pplx_kernels.workloads import make_world

    world = make_world(spec, group_name="bench-roofline")
    stream = torch.cuda.Stream()
    n_sets = len(steps)
    launches_per_graph = 8

    def many_combines(st):
        def body():
            for _ in range(launches_per_graph):
                st.combine_world(world)

        return body

    with torch.cuda.stream(stream):
        for st in steps:
            st.dispatch_world(world)  # slot map of this world
        stream.synchronize()
    # combine reads the world's slot map, identical for every buffer set (same routing)
    k_graphs = [capture(world, stream, many_combines(st)) for st in steps]
    reps = max(1, steps_k // (n_sets * launches_per_graph))
    per_graph_us = time_graphs(k_graphs, list(range(n_sets)), stream, 2, reps)
    kernel_us = per_graph_us / launches_per_graph
    for g in k_graphs:
        g.destroy()
    world.destroy()
    from pplx_kernels import ops

    traffic, traffic_source = measured_traffic_bytes(
        name, "combine_gather", ops.load_library().pplx_a2a_build_id().decode()
    )
    return {
        "kernel": "combine_gather<bf16,bf16>",
        "bound": "hbm",
        "achieved": comb_b / kernel_us / 1e3,
        "peak": HBM_PEAK_GBPS,
        "unit": "GB/s",
        "frac": comb_b / kernel_us / 1e3 / HBM_PEAK_GBPS,
        "traffic": traffic,
        "traffic_source": traffic_source,
        "bytes_per_launch": comb_b,
        "avg_launch_us": kernel_us,
        "launches_timed": reps * n_sets * launches_per_graph,
    }


def cpu_baseline(spec, groups, budget_s=12.0):
    """The oracle's vectorised torch CPU port of one full step (stable argsort on the expert id,
    index_select / index_copy_ for dispatch; index_select + fp32 weighted sum for combine; it
    restates the routing of the reference's tests/test_all_to_all.py:113-120,277-286), on all host
    cores, on the inputs the GPU leg ran.  expert_y holds as many rows per expert as the busiest
    expert receives, so that the 8192-token prefill fits host memory."""
    from oracle import a2a_oracle as orc
    from pplx_kernels.workloads import expert_counts

    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    M, E, K, H = spec.max_num_tokens, spec.num_experts, spec.experts_per_token, spec.hidden_dim
    cap = max(int(expert_counts(groups, E).max()), 1)
    groups_t = [(g.x, g.x_scale, g.indices.to(torch.int64), g.n) for g in groups]
    weights_t = [g.weights for g in groups]
    # N(0,1) rows; one [cap, H] slab replicated per expert keeps the set-up short
    slab = torch.randn(cap, H, generator=torch.Generator().manual_seed(1)).to(spec.expert_y_dtype)
    expert_y = slab.unsqueeze(0).expand(E, cap, H).contiguous()
    times = []
    t_all = time.perf_counter()
    while len(times) < 3 or (time.perf_counter() - t_all < budget_s / 2 and len(times) < 15):
        t0 = time.perf_counter()
        _, _, _, slot_flat = orc.torch_dispatch(groups_t, M, E, K, cap)
        orc.torch_combine(groups_t, weights_t, slot_flat, expert_y, spec.out_dtype)
        times.append(time.perf_counter() - t0)
        if time.perf_counter() - t_all > budget_s:
            break
    return {
        "value": statistics.median(times) * 1e6,
        "unit": "us",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"{len(times)} full steps of the same workload (all {sum(g.n for g in groups)} tokens, "
        f"{cap} rows per expert), median; torch CPU stable-argsort scatter + fp32 gather-sum "
        "(oracle.a2a_oracle.torch_*)",
    }


def cpu_literal_loops(spec):
    """One step in the literal per-token loops of the reference's test
    (tests/test_all_to_all.py:113-120, 281-285), single core; only sensible for the smallest
    workload (the loops are O(pairs) interpreter iterations)."""
    import numpy as np

    from oracle import a2a_oracle as orc
    from pplx_kernels.workloads import generate

    dtype_code = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}
    og = [
        orc.GroupData(
            g.x.contiguous().view(torch.uint8).reshape(g.x.shape[0], -1).numpy(),
            None if g.x_scale is None else g.x_scale.numpy(),
            g.indices.numpy().astype(np.uint32),
            g.weights.numpy(),
            g.n,
        )
        for g in generate(spec)
    ]
    M, E, K, H = spec.max_num_tokens, spec.num_experts, spec.experts_per_token, spec.hidden_dim
    cap = M * spec.num_dp_groups
    rng = np.random.default_rng(1)
    y_dt, out_dt = dtype_code[spec.expert_y_dtype], dtype_code[spec.out_dtype]
    expert_y = orc.from_float32(rng.standard_normal((E, cap, H), dtype=np.float32), y_dt)
    t0 = time.perf_counter()
    res = orc.loop_dispatch(og, M, E, K, cap)
    orc.loop_combine(og, M, E, K, H, expert_y, y_dt, out_dt, res.slot_map)
    return {"value": (time.perf_counter() - t0) * 1e6, "unit": "us", "cores": 1, "kind": "port",
            "sample": "one full step, python loops over tokens and picks (oracle.a2a_oracle.loop_*)"}  # fmt: skip


def counter_probe(spec, launches=3):
    """For `rocprofv3 --pmc FETCH_SIZE` / `--pmc WRITE_SIZE` runs: a few eager dispatch and
    combine launches of the workload plus a plain elementwise copy of known size (1 GiB read,
    1 GiB written) whose counter reading calibrates the unit."""
    from pplx_kernels.workloads import DeviceStep, expert_counts, generate, make_world

    groups = generate(spec)
    cap = max(int(expert_counts(groups, spec.num_experts).max()), 1)
    step = DeviceStep(spec, groups, cap=cap)
    step.expert_y_all.normal_()
    world = make_world(spec, group_name="probe")
    a = torch.ones(1 << 28, dtype=torch.int32, device="cuda")
    b = torch.empty_like(a)
    torch.cuda.synchronize()
    for _ in range(launches):
        torch.mul(a, 3, out=b)  # calibration: reads 2^30 bytes, writes 2^30 bytes
        step.dispatch_world(world)
        step.combine_world(world)
        torch.cuda.synchronize()
    d, c = step.algorithmic_bytes()
    from pplx_kernels import ops

    print(json.dumps({"probe": spec.name, "dispatch_bytes": d, "combine_bytes": c, "copy_bytes_each_way": 1 << 30,
                      "library_build_id": ops.load_library().pplx_a2a_build_id().decode()}))  # fmt: skip
    world.destroy()


TIMELINE_PHASES = (
    "workgroup entered", "rank table in LDS", "earlier picks counted", "own picks marked, row loads issued",
    "barrier passed", "slots and destinations resolved", "row arrived", "stores issued", "stores complete",
)  # fmt: skip


def fused_dispatch_timeline(spec, launches=6):
    """Per-workgroup phase times of the one-launch dispatch, from a library built with
    `make -C pplx-kernels_amd/csrc -B TIMELINE=1`: thread 0 of every workgroup stamps the GPU's
    100 MHz clock at its phase boundaries.  Each launch is made cold (a 768 MB fill in front evicts
    the caches); the last three are summarised as ns after the first workgroup's entry."""
    import ctypes

    import numpy as np

    from pplx_kernels import ops
    from pplx_kernels.workloads import DeviceStep, generate, make_world

    lib = ops.load_library()
    if not hasattr(lib, "pplx_a2a_debug_timeline"):
        sys.exit("bench.py --timeline needs a library built with `make -C pplx-kernels_amd/csrc -B TIMELINE=1`")
    lib.pplx_a2a_debug_timeline.argtypes = [ctypes.c_void_p, ctypes.c_int]
    step = DeviceStep(spec, generate(spec))
    world = make_world(spec, group_name="timeline")
    evict = torch.empty(768 << 20, dtype=torch.uint8, device="cuda")
    print(f"dispatch_fused phase times, workload {spec.name}, library build {lib.pplx_a2a_build_id().decode()} + TIMELINE")
    for it in range(launches):
        evict.fill_(it)
        torch.cuda.synchronize()
        step.dispatch_world(world)
        torch.cuda.synchronize()
        buf = (ctypes.c_ulonglong * 16384)()
        assert lib.pplx_a2a_debug_timeline(buf, 16384) == 0
        a = np.frombuffer(buf, dtype=np.uint64).reshape(1024, 16).astype(np.int64)
        a = a[: int((a[:, 0] > 0).sum())]
        rel = (a[:, :9] - a[:, 0].min()) * 10
        if it < launches - 3:
            continue
        print(f"launch {it}: {len(a)} workgroups, last store complete {rel[:, 8].max()} ns after the first entry")
        print(f"  {'phase':<38s} {'min':>7s} {'median':>7s} {'p90':>7s} {'max':>7s}  ns")
        for i, label in enumerate(TIMELINE_PHASES):
            col = rel[:, i]
            print(f"  {label:<38s} {col.min():7d} {int(np.median(col)):7d} {int(np.percentile(col, 90)):7d} {col.max():7d}")
    world.destroy()


def steps_for(name, steps_k):
    """Timed steps per workload: the large prefills take milliseconds per step."""
    if name == "C5":
        return max(10, steps_k // 10)
    if name == "C4":
        return max(20, steps_k // 4)
    return steps_k


COMPACT_FIELDS = (
    "workload", "tokens", "pairs", "buffer_sets", "steps_timed", "launch_form", "step_us", "step_us_regions",
    "bound_eager_step_us", "bound_eager_host_us_per_call", "graph_step_us", "per_rank_api_step_us", "per_rank_api_calls_per_step", "dispatch_us",
    "combine_us", "step_hbm_frac", "dispatch_hbm_frac", "combine_hbm_frac", "graph_replay_1000x_us", "bound_eager_1000x_us",
    "graph_replay_1000x_note",
)  # fmt: skip


def compact(res):
    return {k: res[k] for k in COMPACT_FIELDS if k in res}


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="C2", help="the headline workload (value, roofline, cpu_baseline)")
    ap.add_argument("--only", action="store_true", help="measure the headline workload alone (profiling runs)")
    ap.add_argument("--all", action="store_true", help="accepted for compatibility: every workload is measured by default")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--counter-probe", action="store_true", help="few eager launches + a calibration copy, for rocprofv3 --pmc")
    ap.add_argument("--timeline", action="store_true", help="phase times of the one-launch dispatch (needs a TIMELINE=1 build)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print(
            "bench.py: this build is a single-GPU loopback (all simulated EP ranks share one HBM); "
            "run it with --gpus 1",
            file=sys.stderr,
        )
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(2)
    torch.cuda.set_device(0)
    from pplx_kernels import ops
    from pplx_kernels.workloads import baseline_configs

    ops.load_library()  # fail loudly here if the HIP library is missing
    specs = baseline_configs()
    spec = specs[args.workload]
    if args.counter_probe:
        counter_probe(spec)
        return
    if args.timeline:
        fused_dispatch_timeline(spec)
        return
    main_res, groups, steps = measure_workload(args.workload, spec, steps_for(args.workload, args.steps), args.warmup)
    roofline = combine_kernel_roofline(args.workload, spec, steps, main_res["combine_bytes"], args.steps)
    del steps
    torch.cuda.empty_cache()

    workloads = {args.workload: compact(main_res)}
    if not args.no_cpu:
        workloads[args.workload]["cpu_baseline"] = cpu_baseline(spec, groups)
    del groups
    if not args.only:
        # the 8192-token prefill (the >= 60 % target) first, then the rest
        for name in ("C5", "C4", "C3", "C1"):
            if name == args.workload:
                continue
            res, grp, st = measure_workload(name, specs[name], steps_for(name, args.steps), min(args.warmup, 5))
            del st
            torch.cuda.empty_cache()
            workloads[name] = compact(res)
            if not args.no_cpu:
                workloads[name]["cpu_baseline"] = cpu_baseline(specs[name], grp)
                if name == "C1":
                    workloads[name]["cpu_literal_loops"] = cpu_literal_loops(specs[name])
            del grp

    form = (
        "eager launches of a bound step (LoopbackWorld.bind: pplx_a2a_world_dispatch + _combine on arguments "
        "packed once)"
    )
    result = {
        "metric": "dispatch+combine latency (us) and achieved HBM GB/s, DSv3 shape 128 tok/rank, 1 GPU",
        "value": main_res["step_us"],
        "unit": "us",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": main_res["step_us"] / 1e3,
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "fp8_e4m3 rows + f32 block scales moved as bytes; combine bf16 in, f32 accumulate, bf16 out",
        "data": "synthetic",
        "config": {
            "workload": spec.name,
            "simulated_ranks": spec.world_size,
            "num_experts": spec.num_experts,
            "experts_per_token": spec.experts_per_token,
            "hidden_dim": spec.hidden_dim,
            "tokens_per_rank": spec.max_num_tokens,
            "in_dtype": str(spec.in_dtype).replace("torch.", ""),
            "out_dtype": str(spec.out_dtype).replace("torch.", ""),
            "timed": f"{form}, rotating buffer sets; the same step as a hipGraph replay takes "
            f"{main_res['graph_step_us']:.1f} us, through the reference's per-rank API "
            f"(AllToAll.dispatch / .combine, {main_res['per_rank_api_calls_per_step']} calls) "
            f"{main_res['per_rank_api_step_us']:.1f} us",
        },
        "roofline": roofline,
        "workloads": workloads,
        "detail": main_res,
    }
    if not args.no_cpu:
        result["cpu_baseline"] = workloads[args.workload]["cpu_baseline"]
    print(json.dumps(result))


if __name__ == "__main__":
    main()
