"""Synthetic workloads of the MoE dispatch / combine path and a device-side driver for them.

``WorkloadSpec`` describes a step (simulated ranks, experts, top-k, row shape, routing skew,
token counts); ``baseline_configs()`` returns the five benchmark workloads C1..C5; ``generate``
draws one DP group's inputs on the CPU from a seeded generator (fp8 block quantisation with an
fp32 absmax scale per 128 columns, uniform or Zipf-skewed routing without replacement, softmax
weights); ``DeviceStep`` holds all ranks' device tensors of one step and runs it through a
``LoopbackWorld`` or through per-rank ``AllToAll`` objects.  Used by ``bench.py`` and by the tests.
"""

from __future__ import annotations

import dataclasses

import numpy as np
import torch

FP8 = torch.float8_e4m3fn
FP8_MAX = 448.0


@dataclasses.dataclass
class WorkloadSpec:
    name: str
    config_id: int
    world_size: int
    num_experts: int
    experts_per_token: int
    hidden_dim: int
    max_num_tokens: int
    in_dtype: torch.dtype
    out_dtype: torch.dtype = torch.bfloat16
    expert_y_dtype: torch.dtype = torch.bfloat16
    dp_size: int = 1
    tokens: str = "max"  # "max": bound_m = M on every rank; "uniform": bound_m ~ U{1..M}
    routing: str = "uniform"  # "uniform" | "zipf:<s>" | "mix:<s>" (half uniform, half Zipf)
    block_size: int = 128

    @property
    def num_dp_groups(self) -> int:
        return self.world_size // self.dp_size

    @property
    def num_local_experts(self) -> int:
        return self.num_experts // self.world_size

    @property
    def hidden_dim_bytes(self) -> int:
        return self.hidden_dim * self.in_dtype.itemsize

    @property
    def scale_dim(self) -> int:
        if self.in_dtype.itemsize != 1:
            return 0
        return (self.hidden_dim + self.block_size - 1) // self.block_size

    @property
    def hidden_dim_scale_bytes(self) -> int:
        return self.scale_dim * 4


def baseline_configs() -> dict[str, WorkloadSpec]:
    """The five workloads of the benchmark plan, C1..C5."""
    return {
        "C1": WorkloadSpec("C1 smallest round-trip", 1, 1, 16, 2, 1024, 32, torch.bfloat16),
        "C2": WorkloadSpec("C2 DSv3 128 tok/rank x 8 ranks", 2, 8, 256, 8, 7168, 128, FP8),
        "C3": WorkloadSpec("C3 decode 1 tok/rank x 64 ranks", 3, 64, 256, 8, 7168, 1, FP8),
        "C4": WorkloadSpec(
            "C4 Mixtral bf16 prefill 4096 tok/rank x 8 ranks", 4, 8, 8, 2, 4096, 4096, torch.bfloat16,
            routing="zipf:1.2",
        ),  # fmt: skip
        "C5": WorkloadSpec(
            "C5 large prefill <=8192 tok/rank x 8 ranks", 5, 8, 256, 8, 7168, 8192, FP8,
            tokens="uniform", routing="mix:1.0",
        ),  # fmt: skip
    }


@dataclasses.dataclass
class GroupInputs:
    """CPU tensors of one DP group."""

    x: torch.Tensor  # [m, H] in_dtype
    x_scale: torch.Tensor | None  # [m, S] f32
    indices: torch.Tensor  # [m, K] int32
    weights: torch.Tensor  # [m, K] f32
    n: int  # bound_m


def quantize_fp8_blockwise(x: torch.Tensor, block: int = 128) -> tuple[torch.Tensor, torch.Tensor]:
    """bf16/f32 [n, H] -> (fp8 e4m3fn [n, H], f32 scales [n, ceil(H/block)]) with
    scale = absmax(block) / 448."""
    n, h = x.shape
    nb = (h + block - 1) // block
    pad = nb * block - h
    xf = torch.nn.functional.pad(x.float(), (0, pad)).view(n, nb, block)
    scale = xf.abs().amax(dim=2) / FP8_MAX
    scale = torch.where(scale == 0, torch.ones_like(scale), scale)
    q = (xf / scale[:, :, None]).view(n, nb * block)[:, :h].to(FP8)
    return q.contiguous(), scale.contiguous()


def sample_routing(n: int, E: int, K: int, routing: str, rng: torch.Generator) -> torch.Tensor:
    """[n, K] int32 expert ids, distinct per row."""
    if n == 0:
        return torch.empty(0, K, dtype=torch.int32)
    if routing == "uniform":
        return torch.rand(n, E, generator=rng).argsort(dim=1)[:, :K].to(torch.int32)
    kind, s = routing.split(":")
    pmf = 1.0 / torch.arange(1, E + 1, dtype=torch.float64) ** float(s)
    pmf = pmf / pmf.sum()
    perm = torch.randperm(E, generator=rng)  # which expert is the hot one varies with the seed
    logp = torch.empty(E, dtype=torch.float64)
    logp[perm] = pmf.log()
    # Gumbel top-k = sampling without replacement from the pmf.
    u = torch.rand(n, E, generator=rng, dtype=torch.float64).clamp_min(1e-300)
    zipf = (logp[None, :] - torch.log(-torch.log(u))).topk(K, dim=1).indices.to(torch.int32)
    if kind == "zipf":
        return zipf
    uni = torch.rand(n, E, generator=rng).argsort(dim=1)[:, :K].to(torch.int32)
    pick_zipf = torch.rand(n, generator=rng) < 0.5
    return torch.where(pick_zipf[:, None], zipf, uni)


def generate_group(spec: WorkloadSpec, group: int, seed: int | None = None, n: int | None = None) -> GroupInputs:
    rng = torch.Generator()
    rng.manual_seed(1000 * spec.config_id + group if seed is None else seed)
    M = spec.max_num_tokens
    if n is None:
        n = M if spec.tokens == "max" else int(torch.randint(1, M + 1, [1], generator=rng).item())
    indices = sample_routing(M, spec.num_experts, spec.experts_per_token, spec.routing, rng)
    weights = torch.softmax(torch.randn(M, spec.experts_per_token, generator=rng), dim=1)
    x = torch.randn(M, spec.hidden_dim, generator=rng).to(torch.bfloat16)
    x_scale = None
    if spec.in_dtype == FP8:
        x, x_scale = quantize_fp8_blockwise(x, spec.block_size)
    else:
        x = x.to(spec.in_dtype)
    return GroupInputs(x, x_scale, indices, weights.contiguous(), n)


def generate(spec: WorkloadSpec, seed: int | None = None) -> list[GroupInputs]:
    return [
        generate_group(spec, g, None if seed is None else seed * 1000 + g)
        for g in range(spec.num_dp_groups)
    ]


def expert_counts(groups: list[GroupInputs], E: int) -> np.ndarray:
    flat = np.concatenate([g.indices[: g.n].reshape(-1).numpy() for g in groups])
    return np.bincount(flat, minlength=E)


# ---------------------------------------------------------------------------
# Device-side state of one step
# ---------------------------------------------------------------------------
class DeviceStep:
    """All ranks' device tensors for one dispatch + combine step of a workload."""

    def __init__(
        self,
        spec: WorkloadSpec,
        groups: list[GroupInputs],
        cap: int | None = None,
        device: str = "cuda:0",
        with_bound_m: bool = True,
        alloc_expert_y: bool = True,
    ) -> None:
        self.spec = spec
        self.groups = groups
        R, dp, L = spec.world_size, spec.dp_size, spec.num_local_experts
        self.cap = cap if cap is not None else spec.max_num_tokens * spec.num_dp_groups
        dev = torch.device(device)
        S = spec.scale_dim
        self.dp_x, self.dp_x_scale, self.indices, self.weights, self.bound_m = [], [], [], [], []
        for r in range(R):
            g = groups[r // dp]
            self.dp_x.append(g.x.to(dev))
            self.dp_x_scale.append(g.x_scale.to(dev) if S else None)
            self.indices.append(g.indices.to(dev).to(torch.uint32))
            self.weights.append(g.weights.to(dev))
            self.bound_m.append(
                torch.tensor([g.n], dtype=torch.uint32, device=dev) if with_bound_m else None
            )
        # One allocation for all ranks' expert-major buffers: [R, L, cap, ...].
        self.expert_num_tokens_all = torch.full((R, L), -1, dtype=torch.int32, device=dev)
        self.expert_x_all = torch.empty((R, L, self.cap, spec.hidden_dim), dtype=spec.in_dtype, device=dev)
        self.expert_x_scale_all = (
            torch.empty((R, L, self.cap, S), dtype=torch.float32, device=dev) if S else None
        )
        self.expert_num_tokens = [self.expert_num_tokens_all[r] for r in range(R)]
        self.expert_x = [self.expert_x_all[r] for r in range(R)]
        self.expert_x_scale = [self.expert_x_scale_all[r] if S else None for r in range(R)]
        self.expert_y_all = None
        self.expert_y = None
        if alloc_expert_y:
            self.expert_y_all = torch.empty(
                (R, L, self.cap, spec.hidden_dim), dtype=spec.expert_y_dtype, device=dev
            )
            self.expert_y = [self.expert_y_all[r] for r in range(R)]
        self.out_tokens = [
            torch.full((spec.max_num_tokens, spec.hidden_dim), float("nan"), dtype=spec.out_dtype, device=dev)
            for _ in range(R)
        ]

    # -- the two ways to run a step ----------------------------------------
    def dispatch_world(self, world) -> None:
        world.dispatch(
            self.expert_num_tokens, self.expert_x, self.expert_x_scale,
            self.dp_x, self.dp_x_scale, self.indices, self.bound_m,
        )  # fmt: skip

    def combine_world(self, world) -> None:
        world.combine(self.out_tokens, self.indices, self.weights, self.expert_y, self.bound_m)

    def bind_world(self, world):
        return world.bind(
            self.expert_num_tokens, self.expert_x, self.expert_x_scale, self.dp_x, self.dp_x_scale,
            self.indices, self.bound_m, self.out_tokens, self.weights, self.expert_y,
        )  # fmt: skip

    def dispatch_per_rank(self, ranks) -> None:
        for r, ata in enumerate(ranks):
            ata.dispatch(
                out_expert_num_tokens=self.expert_num_tokens[r],
                out_expert_x=self.expert_x[r],
                out_expert_x_scale=self.expert_x_scale[r],
                dp_x=self.dp_x[r],
                dp_x_scale=self.dp_x_scale[r],
                indices=self.indices[r],
                bound_m=self.bound_m[r],
            )

    def combine_per_rank(self, ranks) -> None:
        for r, ata in enumerate(ranks):
            ata.combine(
                out_tokens=self.out_tokens[r],
                indices=self.indices[r],
                weights=self.weights[r],
                expert_y=self.expert_y[r],
                bound_m=self.bound_m[r],
            )

    # -- byte accounting ------------------------------------------------------
    def algorithmic_bytes(self) -> tuple[int, int]:
        """(dispatch_bytes, combine_bytes) of a single-hop implementation:
        dispatch = T*tokB + P*4 + P*tokB + E*4,
        combine  = P*H*sizeof(y) + P*8 + T*H*sizeof(out), with T tokens, P = T*K pairs."""
        s = self.spec
        T = sum(g.n for g in self.groups)
        P = T * s.experts_per_token
        tok_b = s.hidden_dim_bytes + s.hidden_dim_scale_bytes
        dispatch = T * tok_b + P * 4 + P * tok_b + s.num_experts * 4
        combine = (
            P * s.hidden_dim * s.expert_y_dtype.itemsize
            + P * 8
            + T * s.dp_size * s.hidden_dim * s.out_dtype.itemsize
        )
        return dispatch, combine


def make_world(spec: WorkloadSpec, group_name: str = "loopback"):
    from .loopback import LoopbackWorld

    return LoopbackWorld(
        spec.max_num_tokens,
        spec.num_experts,
        spec.experts_per_token,
        spec.world_size,
        spec.dp_size,
        spec.hidden_dim,
        spec.hidden_dim_bytes,
        spec.hidden_dim_scale_bytes,
        group_name,
    )


