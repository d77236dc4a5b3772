"""GPU test of ``pplx_a2a_static_step``, the entry point that allocates nothing: its outputs
must equal those of ``pplx_a2a_world_dispatch`` / ``pplx_a2a_world_combine`` bit for bit (the
kernels are the same; only the scratch memory differs: a fixed array inside the library instead
of a world's allocations), on calls in a row that share the array, the later ones smaller."""

from __future__ import annotations

import ctypes

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


def _spec(**kw) -> WorkloadSpec:
    base = dict(
        name="static", config_id=70, world_size=8, num_experts=64, experts_per_token=8,
        hidden_dim=1024, max_num_tokens=96, in_dtype=FP8, tokens="uniform",
    )  # fmt: skip
    base.update(kw)
    return WorkloadSpec(**base)


def _pack(ops, spec, step):
    R = spec.world_size
    d_args = (ops.DispatchArgs * R)()
    c_args = (ops.CombineArgs * R)()
    for r in range(R):
        ops.pack_dispatch_args(
            spec.experts_per_token, step.expert_num_tokens[r], step.expert_x[r], step.expert_x_scale[r],
            step.dp_x[r], step.dp_x_scale[r], step.indices[r], step.bound_m[r], out=d_args[r],
        )  # fmt: skip
        ops.pack_combine_args(
            step.out_tokens[r], step.indices[r], step.weights[r], step.expert_y[r], step.bound_m[r], out=c_args[r]
        )
    return d_args, c_args


def _config(ops, spec):
    return ops.Config(
        spec.max_num_tokens, spec.num_experts, spec.experts_per_token, spec.world_size, spec.dp_size,
        spec.hidden_dim, spec.hidden_dim_bytes, spec.hidden_dim_scale_bytes,
    )  # fmt: skip


def _zeroed_step(spec, groups, cap):
    step = DeviceStep(spec, groups, cap=cap)
    step.expert_x_all.view(torch.uint8).zero_()
    if step.expert_x_scale_all is not None:
        step.expert_x_scale_all.zero_()
    return step


def _compare(spec, groups, fault_word, cap=None, one_call=False):
    """Runs the step through a world and through the static entry point; everything written
    must be identical."""
    from pplx_kernels import ops

    lib = ops.load_library()
    ref = _zeroed_step(spec, groups, cap)
    got = _zeroed_step(spec, groups, cap)
    gen = torch.Generator(device="cuda").manual_seed(spec.max_num_tokens)
    y = torch.randn(ref.expert_y_all.shape, generator=gen, device="cuda").to(ref.expert_y_all.dtype)
    ref.expert_y_all.copy_(y)
    got.expert_y_all.copy_(y)

    world = make_world(spec, group_name=f"static-ref-{spec.name}")
    ref.dispatch_world(world)
    ref.combine_world(world)
    assert world.faults() == 0
    world.destroy()

    cfg = _config(ops, spec)
    d_args, c_args = _pack(ops, spec, got)
    stream = torch.cuda.current_stream().cuda_stream
    fault_word.zero_()
    # (a first call outside the measurement: the runtime itself may grow its launch buffers the
    # first time a kernel variant runs)
    ops.check_status(lib.pplx_a2a_static_step(ctypes.byref(cfg), 0, d_args, c_args, None, stream))
    torch.cuda.synchronize()
    for t, n in zip(got.out_tokens, (groups[r // spec.dp_size].n for r in range(spec.world_size))):
        t[:n].zero_()
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    if one_call:
        ops.check_status(lib.pplx_a2a_static_step(ctypes.byref(cfg), 0, d_args, c_args, fault_word.data_ptr(), stream))
    else:
        ops.check_status(lib.pplx_a2a_static_step(ctypes.byref(cfg), 0, d_args, None, fault_word.data_ptr(), stream))
        ops.check_status(lib.pplx_a2a_static_step(ctypes.byref(cfg), 0, None, c_args, None, stream))
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before, "the static step changed the device's free memory"
    assert int(fault_word.item()) == 0

    assert torch.equal(got.expert_num_tokens_all, ref.expert_num_tokens_all)
    assert int(ref.expert_num_tokens_all.sum()) == spec.experts_per_token * sum(g.n for g in groups)
    assert torch.equal(got.expert_x_all.view(torch.uint8), ref.expert_x_all.view(torch.uint8))
    if spec.scale_dim:
        assert torch.equal(got.expert_x_scale_all.view(torch.int32), ref.expert_x_scale_all.view(torch.int32))
    for r in range(spec.world_size):
        n = groups[r // spec.dp_size].n
        a, b = got.out_tokens[r][:n], ref.out_tokens[r][:n]
        assert not torch.isnan(b.float()).any()
        assert torch.equal(a.view(torch.int16), b.view(torch.int16)), f"combine differs on rank {r}"
        assert torch.isnan(got.out_tokens[r][n:].float()).all()
    # ... and, like the world path, equal to the CPU oracle
    expected = check_dispatch_against_oracle(got)
    check_combine_against_oracle(got, expected.slot_map, use_numpy=True)


def test_static_step_matches_the_world_path_on_calls_in_a_row():
    fault_word = torch.zeros(1, dtype=torch.int32, device="cuda")
    # 1. DSv3-like rows with block scales, dispatch and combine as two calls
    spec = _spec(name="a")
    _compare(spec, generate(spec), fault_word)
    # 2. right after it a smaller step of another geometry (the array still holds call 1's slot
    #    map), dispatch and combine in one call
    small = _spec(name="b", world_size=4, num_experts=16, experts_per_token=3, hidden_dim=256,
                  max_num_tokens=24, in_dtype=torch.bfloat16)  # fmt: skip
    _compare(small, generate(small), fault_word, one_call=True)
    # 3. the first geometry again with fewer tokens
    groups = generate(spec, seed=5)
    for g in groups:
        g.n = g.n // 3
    _compare(spec, groups, fault_word)
    # 4. more than 3072 virtual tokens: the routing tiles' counts live in the array too
    tiled = _spec(name="c", world_size=4, num_experts=16, experts_per_token=2, hidden_dim=128,
                  max_num_tokens=4200, in_dtype=torch.bfloat16, dp_size=2)  # fmt: skip
    groups = generate(tiled)
    for g in groups:
        g.n = min(g.n, 700)
    _compare(tiled, groups, fault_word, cap=max(int(expert_counts(groups, tiled.num_experts).max()), 1))
    # 5. and a small one once more
    _compare(small, generate(small, seed=9), fault_word)


def test_static_step_reports_faults_and_refuses_what_does_not_fit():
    from pplx_kernels import ops

    lib = ops.load_library()
    spec = _spec(name="limits", world_size=4, num_experts=16, experts_per_token=4, hidden_dim=256,
                 max_num_tokens=24, in_dtype=torch.bfloat16)  # fmt: skip
    groups = generate(spec)
    groups[1].n = max(groups[1].n, 2)
    groups[1].indices[1, 3] = groups[1].indices[1, 0]  # a repeated expert id: fault bit 3
    step = _zeroed_step(spec, groups, None)
    d_args, c_args = _pack(ops, spec, step)
    fault_word = torch.zeros(1, dtype=torch.int32, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    cfg = _config(ops, spec)
    ops.check_status(lib.pplx_a2a_static_step(ctypes.byref(cfg), 0, d_args, None, fault_word.data_ptr(), stream))
    torch.cuda.synchronize()
    assert int(fault_word.item()) == 8
    assert int(step.expert_num_tokens_all.sum()) == spec.experts_per_token * sum(g.n for g in groups) - 1

    # a slot map beyond the array: 8 groups x 32768 tokens x 8 picks x 4 bytes = 8 MiB
    big = ops.Config(32768, 256, 8, 8, 1, 7168, 7168, 224)
    assert lib.pplx_a2a_static_step(ctypes.byref(big), 0, d_args, None, None, stream) == 1
    assert b"static array" in lib.pplx_a2a_last_error()
    wide = ops.Config(4, 128, 2, 128, 1, 64, 128, 0)
    assert lib.pplx_a2a_static_step(ctypes.byref(wide), 0, d_args, None, None, stream) == 4
    assert lib.pplx_a2a_static_step(ctypes.byref(cfg), 0, None, None, None, stream) == 1
    assert lib.pplx_a2a_static_step(None, 0, d_args, None, None, stream) == 1


def test_static_step_replays_from_a_graph():
    """One of the callers the entry point is for: a step recorded into a hipGraph without any
    world.  The first call on a device looks up the library's scratch array and is made eagerly;
    the recorded one is replayed with new inputs and compared with the world path each time."""
    from pplx_kernels import ops

    lib = ops.load_library()
    spec = _spec(name="graph", world_size=4, num_experts=32, experts_per_token=8, hidden_dim=512,
                 max_num_tokens=40)  # fmt: skip
    groups = generate(spec)
    got = _zeroed_step(spec, groups, None)
    ref = _zeroed_step(spec, groups, None)
    cfg = _config(ops, spec)
    d_args, c_args = _pack(ops, spec, got)
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        ops.check_status(lib.pplx_a2a_static_step(ctypes.byref(cfg), 0, d_args, c_args, None, stream.cuda_stream))
        stream.synchronize()
        graph = ctypes.c_void_p()
        ops.check_status(lib.pplx_a2a_graph_begin_capture(stream.cuda_stream))
        ops.check_status(lib.pplx_a2a_static_step(ctypes.byref(cfg), 0, d_args, c_args, None, stream.cuda_stream))
        ops.check_status(lib.pplx_a2a_graph_end_capture(stream.cuda_stream, ctypes.byref(graph)))
    world = make_world(spec, group_name="static-graph-ref")
    for replay in range(3):
        fresh = generate(spec, seed=20 + replay)
        for step in (got, ref):
            for r in range(spec.world_size):
                g = fresh[r // spec.dp_size]
                step.dp_x[r].copy_(g.x)
                step.dp_x_scale[r].copy_(g.x_scale)
                step.indices[r].copy_(g.indices.to(torch.uint32))
                step.weights[r].copy_(g.weights)
                step.bound_m[r].fill_(g.n)
                step.out_tokens[r].fill_(float("nan"))
            step.expert_x_all.view(torch.uint8).zero_()
            step.expert_x_scale_all.zero_()
            step.expert_y_all.copy_(torch.randn(step.expert_y_all.shape, generator=torch.Generator(device="cuda").manual_seed(replay), device="cuda"))
        torch.cuda.synchronize()
        ref.dispatch_world(world)
        ref.combine_world(world)
        ops.check_status(lib.pplx_a2a_graph_launch(graph, stream.cuda_stream))
        stream.synchronize()
        torch.cuda.synchronize()
        assert torch.equal(got.expert_num_tokens_all, ref.expert_num_tokens_all)
        assert int(ref.expert_num_tokens_all.sum()) == spec.experts_per_token * sum(g.n for g in fresh)
        assert torch.equal(got.expert_x_all.view(torch.uint8), ref.expert_x_all.view(torch.uint8))
        assert torch.equal(got.expert_x_scale_all.view(torch.int32), ref.expert_x_scale_all.view(torch.int32))
        for r in range(spec.world_size):
            n = fresh[r // spec.dp_size].n
            assert torch.equal(got.out_tokens[r][:n].view(torch.int16), ref.out_tokens[r][:n].view(torch.int16))
    ops.check_status(lib.pplx_a2a_graph_destroy(graph))
    assert world.faults() == 0
    world.destroy()


_FIRST_CALL_UNDER_CAPTURE = r"""
import ctypes, sys
import torch
sys.path[:0] = [{pkg!r}, {root!r}]
from pplx_kernels import ops
from tests.all_to_all_utils import DeviceStep, WorkloadSpec, generate
from tests.test_zz_no_alloc import _config, _pack, _spec

lib = ops.load_library()
spec = _spec(name="first", world_size=4, num_experts=16, experts_per_token=4, hidden_dim=256,
             max_num_tokens=24, in_dtype=torch.bfloat16)
step = DeviceStep(spec, generate(spec))
cfg = _config(ops, spec)
d_args, c_args = _pack(ops, spec, step)
stream = torch.cuda.Stream()
torch.cuda.synchronize()
graph = ctypes.c_void_p()
with torch.cuda.stream(stream):
    ops.check_status(lib.pplx_a2a_graph_begin_capture(stream.cuda_stream))
    st = lib.pplx_a2a_static_step(ctypes.byref(cfg), 0, d_args, c_args, None, stream.cuda_stream)
    msg = lib.pplx_a2a_last_error().decode()
    ops.check_status(lib.pplx_a2a_graph_end_capture(stream.cuda_stream, ctypes.byref(graph)))
    ops.check_status(lib.pplx_a2a_graph_destroy(graph))
    assert st == 2 and "cannot be captured" in msg, (st, msg)
    ops.check_status(lib.pplx_a2a_static_step(ctypes.byref(cfg), 0, d_args, c_args, None, stream.cuda_stream))
    stream.synchronize()
    ops.check_status(lib.pplx_a2a_graph_begin_capture(stream.cuda_stream))
    st = lib.pplx_a2a_static_step(ctypes.byref(cfg), 0, d_args, c_args, None, stream.cuda_stream)
    ops.check_status(lib.pplx_a2a_graph_end_capture(stream.cuda_stream, ctypes.byref(graph)))
    assert st == 0, lib.pplx_a2a_last_error()
    ops.check_status(lib.pplx_a2a_graph_launch(graph, stream.cuda_stream))
    stream.synchronize()
    ops.check_status(lib.pplx_a2a_graph_destroy(graph))
print("first-call-ok")
"""


def test_first_static_step_of_a_process_cannot_be_captured():
    """The first call on a device sets the library up (address of the scratch array, the
    device's LDS size): under stream capture it is refused with a status code, and works once
    one eager call has been made.  Needs a process in which nothing has touched the library
    yet, hence the child process."""
    import os
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    code = _FIRST_CALL_UNDER_CAPTURE.format(pkg=os.path.join(root, "pplx-kernels_amd"), root=root)
    proc = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0 and "first-call-ok" in proc.stdout, proc.stdout[-2000:] + proc.stderr[-3000:]
