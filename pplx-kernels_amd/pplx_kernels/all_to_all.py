"""``AllToAll``: the per-rank MoE dispatch / combine object, API-compatible with the
reference's ``src/pplx_kernels/all_to_all.py:11-164``.

One ``AllToAll`` is one *simulated* expert-parallel rank.  All ranks created with the same
``group_name`` share a loopback world in one GPU's HBM; a step is collective over that world
exactly as in the reference, where every rank's process calls ``dispatch`` and ``combine``:

    for r in range(world_size):
        ata[r].dispatch(...)       # kernels are enqueued when the last rank has called
    for r in range(world_size):
        ata[r].combine(...)

Keyword names and positional order follow the reference so that existing callers
(``tests/test_all_to_all.py:180-190,264-270``) run unchanged.  Two deliberate widenings:
a world with a single DP group is accepted (the reference asserts
``world_size // dp_size > 1``, ``all_to_all.py:102-103``), and ``dispatch`` tolerates a
``weights=`` keyword, which it does not need.
"""

from __future__ import annotations

import sys
from collections.abc import Callable
from typing import Any

import torch

from . import ops
from .ops import _C, _ops

# (bound once: a step of R simulated ranks makes 2 R of these calls)
_is_compiling = torch.compiler.is_compiling
_eager_dispatch = _C.dispatch
_eager_combine = _C.combine


class AllToAll:
    def __init__(
        self,
        ptr: Any,
        combine_fn: Callable,
        dispatch_fn: Callable,
        has_scales: bool,
    ) -> None:
        self._ptr = ptr
        self._combine_fn = combine_fn
        self._dispatch_fn = dispatch_fn
        self._has_scales = has_scales

    def __del__(self) -> None:
        if sys.is_finalizing():  # the exit hook of pplx_kernels.ops has released everything
            return
        try:
            self.destroy()
        except Exception:
            pass

    # -- reference API ------------------------------------------------------
    def dispatch(
        self,
        out_expert_num_tokens: torch.Tensor,
        out_expert_x: torch.Tensor,
        out_expert_x_scale: torch.Tensor | None,
        dp_x: torch.Tensor,
        dp_x_scale: torch.Tensor | None,
        indices: torch.Tensor,
        bound_m: torch.Tensor | None,
        do_send: bool = True,
        do_recv: bool = True,
        *,
        weights: torch.Tensor | None = None,
    ) -> None:
        """Scatters ``dp_x[t]`` (and ``dp_x_scale[t]``) to the ``K`` experts in ``indices[t]``
        for ``t < bound_m``; this rank's ``out_expert_x[e_local, :count]`` receives the rows
        routed to its experts from every DP group, ordered by (group, token), and
        ``out_expert_num_tokens[e_local]`` their number.  ``weights`` is accepted and unused.
        """
        assert self._ptr is not None
        del weights
        if self._has_scales:
            assert out_expert_x_scale is not None
            assert dp_x_scale is not None
        else:
            assert out_expert_x_scale is None
            assert dp_x_scale is None
        # Under torch.compile the call goes through the registered op (what the reference always
        # does, src/pplx_kernels/all_to_all.py:47-59) so that it traces; an eager call enters the
        # op's implementation directly, without the dispatcher's boxing of ten arguments.
        fn = self._dispatch_fn if _is_compiling() else _eager_dispatch
        fn(
            self._ptr,
            out_expert_num_tokens,
            out_expert_x,
            out_expert_x_scale,
            dp_x,
            dp_x_scale,
            indices,
            bound_m,
            do_send,
            do_recv,
        )

    def combine(
        self,
        out_tokens: torch.Tensor,
        indices: torch.Tensor,
        weights: torch.Tensor,
        expert_y: torch.Tensor,
        bound_m: torch.Tensor | None,
        do_send: bool = True,
        do_recv: bool = True,
    ) -> None:
        """``out_tokens[t] = sum_k weights[t, k] * expert_y[slot of (t, k)]`` for
        ``t < bound_m``, fp32 accumulation in pick order; later rows are left as they are."""
        assert self._ptr is not None
        fn = self._combine_fn if _is_compiling() else _eager_combine
        fn(
            self._ptr,
            out_tokens,
            indices,
            weights,
            expert_y,
            bound_m,
            do_send,
            do_recv,
        )

    def destroy(self) -> None:
        if self._ptr is not None:
            ptr, self._ptr = self._ptr, None
            if ops.is_live(ptr):
                _ops.all_to_all_destroy(ptr)

    # -- constructors -------------------------------------------------------
    @classmethod
    def intranode(
        cls,
        max_num_tokens: int,
        num_experts: int,
        experts_per_token: int,
        rank: int,
        world_size: int,
        dp_size: int,
        hidden_dim: int,
        hidden_dim_bytes: int,
        hidden_dim_scale_bytes: int,
        group_name: str = "default",
    ) -> "AllToAll":
        assert world_size % dp_size == 0
        assert world_size // dp_size >= 1
        ptr = _ops.all_to_all_intranode_create(
            max_num_tokens,
            num_experts,
            experts_per_token,
            rank,
            world_size,
            dp_size,
            hidden_dim,
            hidden_dim_bytes,
            hidden_dim_scale_bytes,
            group_name,
        )
        assert ptr != 0
        return cls(
            ptr,
            _ops.all_to_all_intranode_combine,
            _ops.all_to_all_intranode_dispatch,
            hidden_dim_scale_bytes > 0,
        )

    @classmethod
    def internode(
        cls,
        max_num_tokens: int,
        num_experts: int,
        experts_per_token: int,
        rank: int,
        world_size: int,
        dp_size: int,
        hidden_dim: int,
        hidden_dim_bytes: int,
        hidden_dim_scale_bytes: int,
    ) -> "AllToAll":
        """Same kernels as ``intranode``: inside one HBM there is no second transport."""
        assert world_size % dp_size == 0
        assert world_size // dp_size >= 1
        ptr = _ops.all_to_all_internode_create(
            max_num_tokens,
            num_experts,
            experts_per_token,
            rank,
            world_size,
            dp_size,
            hidden_dim,
            hidden_dim_bytes,
            hidden_dim_scale_bytes,
        )
        assert ptr != 0
        return cls(
            ptr,
            _ops.all_to_all_internode_combine,
            _ops.all_to_all_internode_dispatch,
            hidden_dim_scale_bytes > 0,
        )
