"""Workload generators and device-side drivers shared by the tests and ``bench.py``.

``MoEConfig`` / ``RankTestData`` restate the data model of the reference's
``tests/all_to_all_utils.py:6-56`` (same fields and distributions: ``num_tokens ~ U{1..M-1}``,
indices = first K of a random permutation, weights ~ U[0,1), fp8 activations from
``(U-0.5)*400`` with random scales, otherwise N(0,1)).  The benchmark workloads and the
device-side driver (``WorkloadSpec``, ``DeviceStep`` ...) live in ``pplx_kernels.workloads`` and
are re-exported here; this module adds the comparisons with the CPU oracle.
"""

from __future__ import annotations

import dataclasses
import os
import sys

import numpy as np
import torch

_ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for _p in (os.path.join(_ROOT, "pplx-kernels_amd"), _ROOT):
    if _p not in sys.path:
        sys.path.insert(0, _p)

from pplx_kernels.workloads import (  # noqa: E402,F401  (re-exported for the tests)
    FP8,
    FP8_MAX,
    DeviceStep,
    GroupInputs,
    WorkloadSpec,
    baseline_configs,
    expert_counts,
    generate,
    generate_group,
    make_world,
    quantize_fp8_blockwise,
    sample_routing,
)


@dataclasses.dataclass
class MoEConfig:
    num_experts: int
    experts_per_token: int
    hidden_dim: int
    max_num_tokens: int
    in_dtype: torch.dtype = torch.bfloat16
    out_dtype: torch.dtype = torch.bfloat16
    block_size: int = 128

    @property
    def scale_dim(self) -> int:
        if self.in_dtype.itemsize != 1:
            return 0
        return (self.hidden_dim + self.block_size - 1) // self.block_size


class RankTestData:
    """One DP group's inputs, drawn like the reference's RankTestData."""

    def __init__(self, cfg: MoEConfig, rng: torch.Generator, use_max_tokens: bool) -> None:
        m = cfg.max_num_tokens
        self.num_tokens = m if use_max_tokens else int(torch.randint(1, m, [1], generator=rng).item())
        n, k = self.num_tokens, cfg.experts_per_token
        perms = [torch.randperm(cfg.num_experts, generator=rng)[:k] for _ in range(n)]
        self.indices = torch.stack(perms).to(torch.int32) if n else torch.empty(0, k, dtype=torch.int32)
        self.weights = torch.rand(n, k, dtype=torch.float32, generator=rng)
        self.x_scale: torch.Tensor | None = None
        if cfg.in_dtype.itemsize == 1:
            u = torch.rand(n, cfg.hidden_dim, dtype=torch.float32, generator=rng)
            self.x = ((u - 0.5) * 400).to(cfg.in_dtype)
            self.x_scale = torch.rand(n, cfg.scale_dim, dtype=torch.float32, generator=rng)
        else:
            self.x = torch.randn(n, cfg.hidden_dim, dtype=cfg.in_dtype, generator=rng)


# The reference's two test geometries (tests/test_all_to_all.py:26-38).
small_moe = MoEConfig(num_experts=8, experts_per_token=3, hidden_dim=512, max_num_tokens=10)
medium_moe = MoEConfig(num_experts=64, experts_per_token=4, hidden_dim=1024, max_num_tokens=20)


def to_oracle_groups(groups: list[GroupInputs]):
    from oracle.a2a_oracle import GroupData

    out = []
    for g in groups:
        xb = g.x.contiguous().view(torch.uint8).reshape(g.x.shape[0], -1).numpy()
        xs = None if g.x_scale is None else g.x_scale.numpy()
        out.append(GroupData(xb, xs, g.indices.numpy().astype(np.uint32), g.weights.numpy(), g.n))
    return out


def torch_bits(t: torch.Tensor) -> np.ndarray:
    """bf16 / f16 tensor -> uint16 bit patterns; f32 -> float32 array."""
    t = t.detach().cpu().contiguous()
    if t.dtype == torch.float32:
        return t.numpy()
    return t.view(torch.int16).numpy().view(np.uint16)


ORACLE_DTYPE = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}


# ---------------------------------------------------------------------------
# Comparison of a device step with the CPU oracle
# ---------------------------------------------------------------------------
def check_dispatch_against_oracle(step: DeviceStep, expected=None):
    """Bit-exact comparison of counts, rows and scale bits (rows beyond an expert's count
    are unconstrained).  Returns the oracle's DispatchResult."""
    from oracle import a2a_oracle as orc

    s = step.spec
    E, K, M = s.num_experts, s.experts_per_token, s.max_num_tokens
    if expected is None:
        expected = orc.c_dispatch(to_oracle_groups(step.groups), M, E, K, step.cap)
    torch.cuda.synchronize()
    counts = step.expert_num_tokens_all.cpu().numpy().reshape(E)
    np.testing.assert_array_equal(counts, expected.counts)
    live = np.arange(step.cap)[None, :] < expected.counts[:, None]
    got_x = step.expert_x_all.view(torch.uint8).reshape(E, step.cap, -1).cpu().numpy()
    np.testing.assert_array_equal(got_x[live], expected.expert_x[live])
    if s.scale_dim:
        got_s = step.expert_x_scale_all.reshape(E, step.cap, -1).cpu().numpy()
        np.testing.assert_array_equal(got_s[live].view(np.uint32), expected.expert_x_scale[live].view(np.uint32))
    return expected


COMBINE_RTOL = 1e-2  # bf16 tolerance of the fp32-accumulated reference
COMBINE_ATOL = 1e-2


def check_combine_against_oracle(step: DeviceStep, slot_map: np.ndarray, use_numpy: bool = False):
    """out_tokens[:n] within rtol 1e-2 / atol 1e-2 of the fp32-accumulated oracle; rows >= n
    still hold the NaN they were filled with."""
    from oracle import a2a_oracle as orc

    s = step.spec
    E, K, M, H = s.num_experts, s.experts_per_token, s.max_num_tokens, s.hidden_dim
    torch.cuda.synchronize()
    y = torch_bits(step.expert_y_all.reshape(E, step.cap, H))
    in_dt, out_dt = ORACLE_DTYPE[s.expert_y_dtype], ORACLE_DTYPE[s.out_dtype]
    fn = orc.np_combine if use_numpy else orc.c_combine
    want = fn(to_oracle_groups(step.groups), M, E, K, H, y, in_dt, out_dt, slot_map)
    for r in range(s.world_size):
        g = step.groups[r // s.dp_size]
        got = step.out_tokens[r].cpu()
        w = orc.to_float32(want[r // s.dp_size], out_dt)
        np.testing.assert_allclose(
            got[: g.n].float().numpy(), w, rtol=COMBINE_RTOL, atol=COMBINE_ATOL,
            err_msg=f"combine mismatch on rank {r}",
        )  # fmt: skip
        assert torch.isnan(got[g.n :]).all(), f"rank {r}: rows >= bound_m were written"
    return want
