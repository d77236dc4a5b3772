"""``LoopbackWorld``: all simulated ranks of one world behind one object.

The per-rank ``AllToAll`` API costs one Python -> C call per rank and step.  A caller that
owns every rank anyway (a single-GPU MoE layer, a benchmark, a captured decode step) can
hand all ranks' tensors over at once; the library then makes one pass over them
(``pplx_a2a_world_dispatch`` / ``pplx_a2a_world_combine``).  The kernels, the results and
the argument checks are the same as for ``world_size`` per-rank calls.

``capture()`` records whatever the body enqueues on the current stream into a hipGraph
through the library's own capture entry points, so a step can be replayed without any
host-side argument handling (the reference's "CUDA graph support", ``README.md:5``).
"""

from __future__ import annotations

import contextlib
import ctypes
from collections.abc import Sequence

import torch

from . import ops
from .all_to_all import AllToAll


class Graph:
    """An instantiated hipGraph of a recorded step."""

    def __init__(self, ptr: int) -> None:
        self._ptr = ptr

    def replay(self, stream: torch.cuda.Stream | None = None) -> None:
        assert self._ptr is not None
        s = stream if stream is not None else torch.cuda.current_stream()
        ops.check_status(ops.load_library().pplx_a2a_graph_launch(self._ptr, s.cuda_stream))

    def destroy(self) -> None:
        if self._ptr is not None:
            ptr, self._ptr = self._ptr, None
            ops.check_status(ops.load_library().pplx_a2a_graph_destroy(ptr))

    def __del__(self) -> None:
        try:
            self.destroy()
        except Exception:
            pass


class BoundStep:
    """One step's arguments of all ranks, checked and packed once: ``dispatch()`` and
    ``combine()`` then cost one library call each, with no per-rank work in Python.  The eager
    alternative to :class:`Graph` for a caller whose buffers stay where they are from step to
    step (on this stack a graph replay costs more host time than two eager launches).  The
    tensors are kept alive by the object; their contents may change between calls, their
    addresses, shapes and strides may not."""

    def __init__(self, world: "LoopbackWorld", dispatch_args, combine_args, device, keep: tuple) -> None:
        self._world = world
        self._dispatch_args = dispatch_args
        self._combine_args = combine_args
        self._device = device
        self._keep = keep
        self._lib = ops.load_library()

    def dispatch(self, stream: torch.cuda.Stream | None = None) -> None:
        s = stream if stream is not None else torch.cuda.current_stream(self._device)
        ops.check_status(
            self._lib.pplx_a2a_world_dispatch(self._world._world_ptr, self._dispatch_args, s.cuda_stream)
        )

    def combine(self, stream: torch.cuda.Stream | None = None) -> None:
        s = stream if stream is not None else torch.cuda.current_stream(self._device)
        ops.check_status(
            self._lib.pplx_a2a_world_combine(self._world._world_ptr, self._combine_args, s.cuda_stream)
        )


class LoopbackWorld:
    def __init__(
        self,
        max_num_tokens: int,
        num_experts: int,
        experts_per_token: int,
        world_size: int,
        dp_size: int,
        hidden_dim: int,
        hidden_dim_bytes: int,
        hidden_dim_scale_bytes: int,
        group_name: str = "loopback",
    ) -> None:
        self.world_size = world_size
        self.dp_size = dp_size
        self.experts_per_token = experts_per_token
        self.ranks = [
            AllToAll.intranode(
                max_num_tokens,
                num_experts,
                experts_per_token,
                r,
                world_size,
                dp_size,
                hidden_dim,
                hidden_dim_bytes,
                hidden_dim_scale_bytes,
                group_name,
            )
            for r in range(world_size)
        ]
        self._world_ptr = ops.world_of(self.ranks[0]._ptr).ptr
        self._dispatch_args = (ops.DispatchArgs * world_size)()
        self._combine_args = (ops.CombineArgs * world_size)()

    def dispatch(
        self,
        out_expert_num_tokens: Sequence[torch.Tensor],
        out_expert_x: Sequence[torch.Tensor],
        out_expert_x_scale: Sequence[torch.Tensor | None],
        dp_x: Sequence[torch.Tensor],
        dp_x_scale: Sequence[torch.Tensor | None],
        indices: Sequence[torch.Tensor],
        bound_m: Sequence[torch.Tensor | None],
    ) -> None:
        """Entry ``r`` of every sequence is rank ``r``'s argument of ``AllToAll.dispatch``."""
        for r in range(self.world_size):
            ops.pack_dispatch_args(
                self.experts_per_token,
                out_expert_num_tokens[r],
                out_expert_x[r],
                out_expert_x_scale[r],
                dp_x[r],
                dp_x_scale[r],
                indices[r],
                bound_m[r],
                out=self._dispatch_args[r],
            )
        stream = torch.cuda.current_stream(indices[0].device).cuda_stream
        ops.check_status(
            ops.load_library().pplx_a2a_world_dispatch(self._world_ptr, self._dispatch_args, stream)
        )

    def combine(
        self,
        out_tokens: Sequence[torch.Tensor],
        indices: Sequence[torch.Tensor],
        weights: Sequence[torch.Tensor],
        expert_y: Sequence[torch.Tensor],
        bound_m: Sequence[torch.Tensor | None],
    ) -> None:
        """Entry ``r`` of every sequence is rank ``r``'s argument of ``AllToAll.combine``."""
        for r in range(self.world_size):
            ops.pack_combine_args(
                out_tokens[r],
                indices[r],
                weights[r],
                expert_y[r],
                bound_m[r],
                out=self._combine_args[r],
            )
        stream = torch.cuda.current_stream(indices[0].device).cuda_stream
        ops.check_status(
            ops.load_library().pplx_a2a_world_combine(self._world_ptr, self._combine_args, stream)
        )

    def bind(
        self,
        out_expert_num_tokens: Sequence[torch.Tensor],
        out_expert_x: Sequence[torch.Tensor],
        out_expert_x_scale: Sequence[torch.Tensor | None],
        dp_x: Sequence[torch.Tensor],
        dp_x_scale: Sequence[torch.Tensor | None],
        indices: Sequence[torch.Tensor],
        bound_m: Sequence[torch.Tensor | None],
        out_tokens: Sequence[torch.Tensor],
        weights: Sequence[torch.Tensor],
        expert_y: Sequence[torch.Tensor],
    ) -> BoundStep:
        """Checks and packs the arguments of :meth:`dispatch` and :meth:`combine` once and
        returns a :class:`BoundStep` that launches them as often as wanted."""
        d_args = (ops.DispatchArgs * self.world_size)()
        c_args = (ops.CombineArgs * self.world_size)()
        for r in range(self.world_size):
            ops.pack_dispatch_args(
                self.experts_per_token, out_expert_num_tokens[r], out_expert_x[r], out_expert_x_scale[r],
                dp_x[r], dp_x_scale[r], indices[r], bound_m[r], out=d_args[r],
            )  # fmt: skip
            ops.pack_combine_args(out_tokens[r], indices[r], weights[r], expert_y[r], bound_m[r], out=c_args[r])
        keep = tuple(
            list(seq)
            for seq in (out_expert_num_tokens, out_expert_x, out_expert_x_scale, dp_x, dp_x_scale, indices,
                        bound_m, out_tokens, weights, expert_y)
        )  # fmt: skip
        return BoundStep(self, d_args, c_args, indices[0].device, keep)

    def faults(self) -> int:
        """Sticky device-side fault bits since the last call (synchronises the stream):
        1 = a routed row did not fit ``out_expert_x.size(1)``, 2 = an expert index was out of
        range, 4 = combine met a slot beyond ``expert_y.size(1)``, 8 = an expert id repeated
        inside one token was dropped, 16 = a ``bound_m`` beyond ``max_num_tokens`` was clamped."""
        bits = ctypes.c_uint32()
        stream = torch.cuda.current_stream().cuda_stream
        ops.check_status(
            ops.load_library().pplx_a2a_world_faults(self._world_ptr, stream, ctypes.byref(bits))
        )
        return bits.value

    @contextlib.contextmanager
    def capture(self):
        """Records the body's launches on the current stream; yields a holder whose
        ``graph`` attribute is the instantiated :class:`Graph` after the block."""
        lib = ops.load_library()
        stream = torch.cuda.current_stream().cuda_stream
        if stream == 0:
            raise RuntimeError(
                "pplx_kernels: the default stream cannot be captured; enter "
                "`with torch.cuda.stream(torch.cuda.Stream()):` first"
            )

        class _Holder:
            graph: Graph | None = None

        holder = _Holder()
        ops.check_status(lib.pplx_a2a_graph_begin_capture(stream))
        try:
            yield holder
        finally:
            ptr = ctypes.c_void_p()
            ops.check_status(lib.pplx_a2a_graph_end_capture(stream, ctypes.byref(ptr)))
            holder.graph = Graph(ptr.value)

    def destroy(self) -> None:
        for r in self.ranks:
            r.destroy()
        self.ranks = []
