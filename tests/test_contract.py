"""GPU tests of the call contract around the kernels: inputs the reference tolerates or asserts
on (repeated expert ids, too many tokens), ranks that call on different streams, the explicit
reservation of split-mode staging, and the C++ benchmark's phase sequence."""

from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np
import pytest
import torch

from tests.all_to_all_utils import (
    FP8,
    DeviceStep,
    WorkloadSpec,
    check_combine_against_oracle,
    check_dispatch_against_oracle,
    expert_counts,
    generate,
    make_world,
)

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

FAULT_ROW_DROPPED, FAULT_BAD_EXPERT, FAULT_BAD_SLOT, FAULT_DUPLICATE, FAULT_TOO_MANY = 1, 2, 4, 8, 16


def _spec(**kw) -> WorkloadSpec:
    base = dict(
        name="contract", config_id=60, world_size=4, num_experts=16, experts_per_token=4,
        hidden_dim=256, max_num_tokens=24, in_dtype=torch.bfloat16, tokens="uniform",
    )  # fmt: skip
    base.update(kw)
    return WorkloadSpec(**base)


def _make_ranks(spec, name):
    from pplx_kernels import AllToAll

    return [
        AllToAll.intranode(
            spec.max_num_tokens, spec.num_experts, spec.experts_per_token, r, spec.world_size, spec.dp_size,
            spec.hidden_dim, spec.hidden_dim_bytes, spec.hidden_dim_scale_bytes, group_name=name,
        )  # fmt: skip
        for r in range(spec.world_size)
    ]


def _dispatch_kw(step, r):
    return dict(
        out_expert_num_tokens=step.expert_num_tokens[r], out_expert_x=step.expert_x[r],
        out_expert_x_scale=step.expert_x_scale[r], dp_x=step.dp_x[r], dp_x_scale=step.dp_x_scale[r],
        indices=step.indices[r], bound_m=step.bound_m[r],
    )  # fmt: skip


def _combine_kw(step, r):
    return dict(
        out_tokens=step.out_tokens[r], indices=step.indices[r], weights=step.weights[r],
        expert_y=step.expert_y[r], bound_m=step.bound_m[r],
    )  # fmt: skip


# ---------------------------------------------------------------------------
# A repeated expert id inside one token
# ---------------------------------------------------------------------------
def _check_with_repeats_dropped(step, after_combine: bool):
    """Literal expectation for a step whose tokens may repeat an expert: walking groups, tokens
    and picks in order, a pick takes the next row of its expert unless the token already named
    that expert (tests/test_all_to_all.py:113-120 appends a token to an expert's list once).  A
    pick that names no expert takes no row either, and rows beyond the capacity are not there."""
    spec, groups = step.spec, step.groups
    E, K, H = spec.num_experts, spec.experts_per_token, spec.hidden_dim
    rows_of = [[] for _ in range(E)]
    slot_of = {}
    for g, grp in enumerate(groups):
        for t in range(grp.n):
            seen = set()
            for k in range(K):
                e = int(grp.indices[t, k])
                if e in seen or e >= E:
                    slot_of[(g, t, k)] = None
                    continue
                seen.add(e)
                slot_of[(g, t, k)] = (e, len(rows_of[e]))
                rows_of[e].append((g, t))
    torch.cuda.synchronize()
    counts = step.expert_num_tokens_all.cpu().numpy().reshape(E)
    np.testing.assert_array_equal(counts, [len(r) for r in rows_of])
    got_x = step.expert_x_all.view(torch.uint8).reshape(E, step.cap, -1).cpu().numpy()
    got_s = step.expert_x_scale_all.reshape(E, step.cap, -1).cpu().numpy() if spec.scale_dim else None
    for e in range(E):
        for s_, (g, t) in enumerate(rows_of[e][: step.cap]):
            want = groups[g].x[t].contiguous().view(torch.uint8).numpy()
            np.testing.assert_array_equal(got_x[e, s_], want)
            if got_s is not None:
                np.testing.assert_array_equal(got_s[e, s_].view(np.uint32), groups[g].x_scale[t].numpy().view(np.uint32))
    if not after_combine:
        return
    y = step.expert_y_all.reshape(E, step.cap, H).float().cpu().numpy()
    for r in range(spec.world_size):
        g = r // spec.dp_size
        got = step.out_tokens[r].float().cpu().numpy()
        for t in range(groups[g].n):
            acc = np.zeros(H, dtype=np.float32)
            for k in range(K):
                where = slot_of[(g, t, k)]
                if where is not None:
                    acc = acc + np.float32(groups[g].weights[t, k].item()) * y[where[0], where[1]]
            np.testing.assert_allclose(got[t], acc, rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize(
    "kw",
    [
        dict(name="dup-one-launch"),
        dict(name="dup-fp8", in_dtype=FP8, hidden_dim=512, experts_per_token=8, num_experts=32),
        dict(name="dup-odd-k", experts_per_token=3),
        dict(name="dup-top12", experts_per_token=12, num_experts=32),
        # more than 3072 virtual tokens: routing tiles + scatter
        dict(name="dup-tiles", max_num_tokens=4200, experts_per_token=2),
        # tiles of eight chunks, groups that start in the middle of a tile
        dict(name="dup-wide-tiles", max_num_tokens=20000, experts_per_token=8, num_experts=32, in_dtype=FP8, hidden_dim=512),
    ],
    ids=lambda kw: kw["name"],
)
def test_repeated_expert_is_dropped_and_reported(kw):
    """The repeat takes no row, is not counted and adds nothing in combine; every other pick is
    placed as usual; fault bit 3 reports it and every kernel exits normally."""
    spec = _spec(**kw)
    groups = generate(spec)
    for g in groups:
        g.n = min(g.n, 150)
    K = spec.experts_per_token
    # group 1, token 2: the last pick repeats the first; group 2, token 0: pick 1 repeats pick 0;
    # group 0, last live token: every pick names the same expert
    groups[1].n = max(groups[1].n, 3)
    groups[2].n = max(groups[2].n, 1)
    groups[0].n = max(groups[0].n, 1)
    groups[1].indices[2, K - 1] = groups[1].indices[2, 0]
    groups[2].indices[0, 1] = groups[2].indices[0, 0]
    groups[0].indices[groups[0].n - 1, :] = 5
    cap = max(int(expert_counts(groups, spec.num_experts).max()), 1)
    step = DeviceStep(spec, groups, cap=cap)
    world = make_world(spec, group_name=kw["name"])
    step.dispatch_world(world)
    torch.cuda.synchronize()
    assert world.faults() == FAULT_DUPLICATE
    _check_with_repeats_dropped(step, after_combine=False)
    assert int(step.expert_num_tokens_all.sum()) == K * sum(g.n for g in groups) - 2 - (K - 1)

    step.expert_y_all.normal_()
    step.combine_world(world)
    assert world.faults() == 0
    _check_with_repeats_dropped(step, after_combine=True)
    world.destroy()


def test_faults_of_a_step_of_several_routing_tiles():
    """A pick that names no expert and an expert with more rows than its buffer holds, in the
    dispatch form whose scatter works the slots out itself: both are reported, the counts give
    the full demand and every row that fits is in place."""
    spec = _spec(name="tiles-faults", max_num_tokens=4200, experts_per_token=4)
    groups = generate(spec)
    for g in groups:
        g.n = min(max(g.n, 8), 200)
    groups[1].indices[3, 1] = 999
    counts = np.zeros(spec.num_experts, dtype=np.int64)
    for g in groups:
        ids = g.indices[: g.n].numpy().reshape(-1)
        counts += np.bincount(ids[ids < spec.num_experts], minlength=spec.num_experts)
    step = DeviceStep(spec, groups, cap=int(counts.max()) - 2)
    world = make_world(spec, group_name="tiles-faults")
    step.dispatch_world(world)
    torch.cuda.synchronize()
    assert world.faults() == FAULT_ROW_DROPPED | FAULT_BAD_EXPERT
    np.testing.assert_array_equal(step.expert_num_tokens_all.cpu().numpy().reshape(-1), counts)
    _check_with_repeats_dropped(step, after_combine=False)
    world.destroy()


def test_repeated_expert_in_split_mode():
    spec = _spec(name="dup-split", in_dtype=FP8, hidden_dim=512)
    groups = generate(spec)
    K = spec.experts_per_token
    groups[0].n = max(groups[0].n, 2)
    groups[0].indices[1, 2] = groups[0].indices[1, 0]
    step = DeviceStep(spec, groups)
    ranks = _make_ranks(spec, "dup-split")
    R = spec.world_size
    for r in range(R):
        ranks[r].dispatch(**_dispatch_kw(step, r), do_send=True, do_recv=False)
    for r in range(R):
        ranks[r].dispatch(**_dispatch_kw(step, r), do_send=False, do_recv=True)
    _check_with_repeats_dropped(step, after_combine=False)
    assert int(step.expert_num_tokens_all.sum()) == K * sum(g.n for g in groups) - 1
    step.expert_y_all.normal_()
    for r in range(R):
        ranks[r].combine(**_combine_kw(step, r), do_send=True, do_recv=False)
    for r in range(R):
        ranks[r].combine(**_combine_kw(step, r), do_send=False, do_recv=True)
    _check_with_repeats_dropped(step, after_combine=True)
    for a in ranks:
        a.destroy()


# ---------------------------------------------------------------------------
# Token counts beyond max_num_tokens (the reference asserts, intranode_dispatch.cu:65)
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("big", [False, True], ids=["one-launch", "tiles"])
def test_bound_m_beyond_the_limit_is_clamped_and_reported(big):
    spec = _spec(name=f"toomany-{big}", tokens="max", max_num_tokens=4200 if big else 24, experts_per_token=2)
    groups = generate(spec)
    if big:
        for g in groups:
            g.n = 100
    step = DeviceStep(spec, groups, cap=max(int(expert_counts(groups, spec.num_experts).max()), 1))
    world = make_world(spec, group_name=spec.name)
    step.dispatch_world(world)
    assert world.faults() == 0
    expected_counts = step.expert_num_tokens_all.clone()
    # the same rows, but the device scalar now asks for more tokens than there are
    if not big:
        step.bound_m[2].fill_(spec.max_num_tokens + 5)
        step.dispatch_world(world)
        assert world.faults() == FAULT_TOO_MANY
        assert torch.equal(step.expert_num_tokens_all, expected_counts)
        check_dispatch_against_oracle(step)
    else:
        step.bound_m[2].fill_(spec.max_num_tokens + 5)
        step.dispatch_world(world)
        assert world.faults() & FAULT_TOO_MANY
    world.destroy()


def test_more_rows_than_max_num_tokens_without_bound_m_is_an_error():
    spec = _spec(name="toomany-rows", tokens="max")
    step = DeviceStep(spec, generate(spec), with_bound_m=False)
    ranks = _make_ranks(spec, "toomany-rows")
    kw = _dispatch_kw(step, 0)
    m = spec.max_num_tokens
    kw["dp_x"] = torch.cat([kw["dp_x"], kw["dp_x"][:1]])
    kw["indices"] = torch.cat([kw["indices"].to(torch.int32), kw["indices"].to(torch.int32)[:1]]).to(torch.uint32)
    assert kw["dp_x"].shape[0] == m + 1
    with pytest.raises(RuntimeError, match="exceed max_num_tokens"):
        ranks[0].dispatch(**kw)
    for a in ranks:
        a.destroy()


def test_dp_group_members_must_agree_on_the_row_count():
    spec = _spec(name="dp-rows", dp_size=2, tokens="max")
    step = DeviceStep(spec, generate(spec))
    ranks = _make_ranks(spec, "dp-rows")
    for r in range(spec.world_size):
        kw = _dispatch_kw(step, r)
        if r == 1:  # second member of group 0 passes fewer rows than the first
            kw["dp_x"] = kw["dp_x"][:-2]
            kw["indices"] = kw["indices"].to(torch.int32)[:-2].to(torch.uint32)
        if r < spec.world_size - 1:
            ranks[r].dispatch(**kw)
        else:
            with pytest.raises(RuntimeError, match="share a DP group"):
                ranks[r].dispatch(**kw)
    for a in ranks:
        a.destroy()


# ---------------------------------------------------------------------------
# Ranks that call on different streams
# (csrc/bindings/all_to_all_ops.cpp:163,194: every rank runs on its own current stream)
# ---------------------------------------------------------------------------
def test_ranks_on_different_streams_are_ordered():
    """Each rank prepares its inputs on its own stream (a long fill, then the real data) and
    calls dispatch there without synchronising; combine likewise; the results are read on yet
    another rank's stream.  No stream or device synchronisation happens in between."""
    spec = _spec(name="streams", in_dtype=FP8, hidden_dim=1024, max_num_tokens=64, num_experts=32, experts_per_token=8)
    groups = generate(spec)
    step = DeviceStep(spec, groups)
    ranks = _make_ranks(spec, "streams")
    R = spec.world_size
    streams = [torch.cuda.Stream() for _ in range(R)]
    true_x = [x.clone() for x in step.dp_x]
    ballast = torch.empty(64 << 20, dtype=torch.uint8, device="cuda")
    torch.cuda.synchronize()
    for round_ in range(2):
        for r in range(R):
            step.dp_x[r].view(torch.uint8).fill_(0x55)
        step.expert_x_all.view(torch.uint8).fill_(0)
        torch.cuda.synchronize()
        for r in range(R):
            with torch.cuda.stream(streams[r]):
                for _ in range(4):
                    ballast.fill_(r)  # keeps the stream busy ahead of the real inputs
                step.dp_x[r].copy_(true_x[r])
                ranks[r].dispatch(**_dispatch_kw(step, r))
        # read back on the stream of rank 0, which did not launch the kernels
        with torch.cuda.stream(streams[0]):
            got_counts = step.expert_num_tokens_all.clone()
            got_x = step.expert_x_all.clone()
        streams[0].synchronize()
        torch.cuda.synchronize()
        expected = check_dispatch_against_oracle(step)
        assert torch.equal(got_counts, step.expert_num_tokens_all)
        assert torch.equal(got_x.view(torch.uint8), step.expert_x_all.view(torch.uint8))

        y = torch.randn(step.expert_y_all.shape, device="cuda").to(step.expert_y_all.dtype)
        step.expert_y_all.zero_()
        for t in step.out_tokens:
            t.fill_(float("nan"))
        torch.cuda.synchronize()
        for r in range(R):
            with torch.cuda.stream(streams[r]):
                for _ in range(4):
                    ballast.fill_(r)
                if r == 1:
                    step.expert_y_all.copy_(y)  # every rank's expert_y arrives on rank 1's stream
                ranks[r].combine(**_combine_kw(step, r))
        with torch.cuda.stream(streams[2]):
            got_out = [t.clone() for t in step.out_tokens]
        streams[2].synchronize()
        torch.cuda.synchronize()
        check_combine_against_oracle(step, expected.slot_map)
        for a, b in zip(got_out, step.out_tokens):
            assert torch.equal(a.view(torch.int16), b.view(torch.int16))
    for a in ranks:
        a.destroy()


# ---------------------------------------------------------------------------
# Split-mode staging is reserved, never allocated by a dispatch / combine call
# ---------------------------------------------------------------------------
def test_split_calls_need_reserved_staging():
    from pplx_kernels import ops

    lib = ops.load_library()
    spec = _spec(name="reserve", tokens="max")
    step = DeviceStep(spec, generate(spec))
    ranks = _make_ranks(spec, "reserve")
    world = ops.world_of(ranks[0]._ptr)
    args = ops.pack_dispatch_args(spec.experts_per_token, *[_dispatch_kw(step, 0)[k] for k in (
        "out_expert_num_tokens", "out_expert_x", "out_expert_x_scale", "dp_x", "dp_x_scale", "indices", "bound_m")])  # fmt: skip
    stream = torch.cuda.current_stream().cuda_stream
    # straight through the C ABI, without the binding's own reservation
    assert lib.pplx_a2a_dispatch(ranks[0]._ptr, ctypes.byref(args), ops.SPLIT_SEND, stream) == 2
    assert b"pplx_a2a_world_reserve_split" in lib.pplx_a2a_last_error()
    assert lib.pplx_a2a_world_reserve_split(world.ptr, 3) == 1
    assert lib.pplx_a2a_world_reserve_split(world.ptr, 0) == 0
    assert lib.pplx_a2a_dispatch(ranks[0]._ptr, ctypes.byref(args), ops.SPLIT_SEND, stream) == 0
    cargs = ops.pack_combine_args(*[_combine_kw(step, 0)[k] for k in ("out_tokens", "indices", "weights", "expert_y", "bound_m")])
    # combine staging was not reserved (0 bytes per element): refused, then reserved
    assert lib.pplx_a2a_combine(ranks[0]._ptr, ctypes.byref(cargs), ops.SPLIT_SEND, stream) == 2
    assert lib.pplx_a2a_world_reserve_split(world.ptr, 2) == 0
    # finish the dispatch step through the Python surface
    for r in range(1, spec.world_size):
        ranks[r].dispatch(**_dispatch_kw(step, r), do_send=True, do_recv=False)
    for r in range(spec.world_size):
        ranks[r].dispatch(**_dispatch_kw(step, r), do_send=False, do_recv=True)
    check_dispatch_against_oracle(step)
    for a in ranks:
        a.destroy()


def test_first_split_step_is_capturable_once_reserved():
    """With staging reserved up front, the very first split calls of a world can be recorded
    into a graph: nothing in them allocates or synchronises."""
    from pplx_kernels import ops

    spec = _spec(name="split-capture", in_dtype=FP8, hidden_dim=512)
    groups = generate(spec)
    step = DeviceStep(spec, groups)
    ranks = _make_ranks(spec, "split-capture")
    world = ops.world_of(ranks[0]._ptr)
    ops.reserve_split(world, 2)
    lib = ops.load_library()
    R = spec.world_size
    stream = torch.cuda.Stream()
    gen = torch.Generator(device="cuda").manual_seed(3)
    step.expert_y_all.copy_(torch.randn(step.expert_y_all.shape, generator=gen, device="cuda"))
    torch.cuda.synchronize()
    graph = ctypes.c_void_p()
    with torch.cuda.stream(stream):
        ops.check_status(lib.pplx_a2a_graph_begin_capture(stream.cuda_stream))
        for r in range(R):
            ranks[r].dispatch(**_dispatch_kw(step, r), do_send=True, do_recv=False)
        for r in range(R):
            ranks[r].dispatch(**_dispatch_kw(step, r), do_send=False, do_recv=True)
        for r in range(R):
            ranks[r].combine(**_combine_kw(step, r), do_send=True, do_recv=False)
        for r in range(R):
            ranks[r].combine(**_combine_kw(step, r), do_send=False, do_recv=True)
        ops.check_status(lib.pplx_a2a_graph_end_capture(stream.cuda_stream, ctypes.byref(graph)))
    for replay in range(3):
        step.expert_x_all.view(torch.uint8).fill_(0)
        for t in step.out_tokens:
            t.fill_(float("nan"))
        torch.cuda.synchronize()
        ops.check_status(lib.pplx_a2a_graph_launch(graph, stream.cuda_stream))
        stream.synchronize()
        expected = check_dispatch_against_oracle(step)
        check_combine_against_oracle(step, expected.slot_map)
    # Nothing that has been reserved ever moves (the combined rows are staged in the dtype of
    # out_tokens, whatever expert_y holds): a later reservation for f32 expert_y and an f32 split
    # combine leave the staging where the graph expects it, and the graph replays as before.
    assert lib.pplx_a2a_world_reserve_split(world.ptr, 4) == 0
    with torch.cuda.stream(stream):
        for do_send in (True, False):
            for r in range(R):
                ranks[r].combine(
                    **{**_combine_kw(step, r), "expert_y": step.expert_y[r].float()}, do_send=do_send, do_recv=not do_send
                )  # fmt: skip
    stream.synchronize()
    check_combine_against_oracle(step, expected.slot_map)
    for t in step.out_tokens:
        t.fill_(float("nan"))
    torch.cuda.synchronize()
    ops.check_status(lib.pplx_a2a_graph_launch(graph, stream.cuda_stream))
    stream.synchronize()
    check_combine_against_oracle(step, check_dispatch_against_oracle(step).slot_map)
    ops.check_status(lib.pplx_a2a_graph_destroy(graph))
    for a in ranks:
        a.destroy()


def test_a_rank_replaced_in_the_middle_of_a_split_phase():
    """A handle destroyed after its SEND call, before the phase is complete, takes that call with
    it: the handle that replaces it sends again and the step comes out whole."""
    from pplx_kernels import AllToAll

    spec = _spec(name="split-replace", in_dtype=FP8, hidden_dim=512)
    step = DeviceStep(spec, generate(spec))
    ranks = _make_ranks(spec, "split-replace")
    R = spec.world_size
    ranks[1].dispatch(**_dispatch_kw(step, 1), do_send=True, do_recv=False)
    ranks[1].destroy()
    ranks[1] = AllToAll.intranode(
        spec.max_num_tokens, spec.num_experts, spec.experts_per_token, 1, spec.world_size, spec.dp_size,
        spec.hidden_dim, spec.hidden_dim_bytes, spec.hidden_dim_scale_bytes, group_name="split-replace",
    )  # fmt: skip
    for r in range(R):
        ranks[r].dispatch(**_dispatch_kw(step, r), do_send=True, do_recv=False)
    for r in range(R):
        ranks[r].dispatch(**_dispatch_kw(step, r), do_send=False, do_recv=True)
    check_dispatch_against_oracle(step)
    for a in ranks:
        a.destroy()


# ---------------------------------------------------------------------------
# Many routing tiles (the prefix over tiles takes several trips)
# ---------------------------------------------------------------------------
def test_more_than_256_routing_tiles():
    spec = _spec(
        name="many-tiles", world_size=64, num_experts=64, experts_per_token=2, hidden_dim=16,
        max_num_tokens=4200, tokens="uniform",
    )  # fmt: skip
    groups = generate(spec)
    for i, g in enumerate(groups):
        g.n = (i * 37) % 90
    cap = max(int(expert_counts(groups, spec.num_experts).max()), 1)
    step = DeviceStep(spec, groups, cap=cap)
    world = make_world(spec, group_name="many-tiles")
    step.dispatch_world(world)
    expected = check_dispatch_against_oracle(step)
    step.expert_y_all.normal_()
    step.combine_world(world)
    assert world.faults() == 0
    check_combine_against_oracle(step, expected.slot_map, use_numpy=True)
    world.destroy()


# ---------------------------------------------------------------------------
# The C++ benchmark's phase sequence (send, gap, recv) runs to the end
# ---------------------------------------------------------------------------
def test_cpp_benchmark_runs_the_reference_sequence():
    exe = os.path.join(ROOT, "pplx-kernels_amd", "bin", "bench_a2a")
    assert os.path.exists(exe), "build it with `make -C pplx-kernels_amd/csrc`"
    proc = subprocess.run([exe, "8", "2", "quick"], capture_output=True, text=True, timeout=300)
    print(proc.stdout[-3000:], proc.stderr[-2000:])
    assert proc.returncode == 0, proc.stdout[-2000:] + proc.stderr[-2000:]
    assert "send+recv against one call" in proc.stdout
    assert "overlap," in proc.stdout
    assert np.isfinite(float(proc.stdout.split("send+recv against one call: dispatch ")[1].split("x")[0]))


def test_cpp_memory_yardstick_runs():
    """The plain streaming kernels that the achieved rates are read against: every line reports
    a rate below the published peak and above a tenth of it."""
    exe = os.path.join(ROOT, "pplx-kernels_amd", "bin", "bench_hbm")
    assert os.path.exists(exe), "build it with `make -C pplx-kernels_amd/csrc`"
    proc = subprocess.run([exe, "3"], capture_output=True, text=True, timeout=300)
    print(proc.stdout[-3000:], proc.stderr[-2000:])
    assert proc.returncode == 0, proc.stdout[-2000:] + proc.stderr[-2000:]
    rates = [float(line.split("TB/s")[0].split()[-1]) for line in proc.stdout.splitlines() if "TB/s " in line]
    assert len(rates) == 21
    assert all(0.8 < r < 8.0 for r in rates), rates


def test_cpp_launch_floor_runs():
    """The launch-cost yardstick (empty kernels, eager and as graph replays) that the latency of
    the decode-sized steps is read against: four lines of eight finite figures."""
    exe = os.path.join(ROOT, "pplx-kernels_amd", "bin", "bench_launch")
    assert os.path.exists(exe), "build it with `make -C pplx-kernels_amd/csrc`"
    proc = subprocess.run([exe, "300"], capture_output=True, text=True, timeout=300)
    print(proc.stdout[-3000:], proc.stderr[-2000:])
    assert proc.returncode == 0, proc.stdout[-2000:] + proc.stderr[-2000:]
    rows = [line.split()[-8:] for line in proc.stdout.splitlines() if "of arguments" in line]
    assert len(rows) == 4
    assert all(0.05 < float(x) < 1000.0 for row in rows for x in row), rows


def test_per_rank_api_benchmark_prints_its_table():
    """tests/bench_all_to_all.py (the eager per-rank latency table, counterpart of the reference's
    tests/bench_all_to_all.py) runs to the end for a small rank count."""
    import sys

    proc = subprocess.run(
        [sys.executable, "-m", "tests.bench_all_to_all", "--ranks", "4", "--quick"],
        capture_output=True, text=True, timeout=300, cwd=ROOT,
    )  # fmt: skip
    assert proc.returncode == 0, proc.stdout[-2000:] + proc.stderr[-2000:]
    lines = [line for line in proc.stdout.splitlines() if line[:1].isdigit()]
    assert len(lines) >= 4 and all("GB/s" in line for line in lines), proc.stdout[-2000:]
