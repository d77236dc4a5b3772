"""Writes the committed golden vectors ``tests/golden/*.npz``.

The reference stores no golden vectors for this path (its tests regenerate random data and
check properties), so these are made here: inputs are drawn with the reference's recipe
(seed 123, ``tests/test_all_to_all.py:106-110``) and the expected outputs come from the
literal loops of the reference's own torch check, written out below with plain Python
indexing and numpy float32 scalars -- deliberately sharing no code with ``oracle/``:

* routing: ``expert_token_from[e].append((dp_rank, token))`` in dp_rank, token order
  (``tests/test_all_to_all.py:113-120``)
* combine: ``sum_k w[t,k] * float(expert_y[e_k][slot])`` in fp32, k ascending
  (``csrc/all_to_all/intranode_combine.cu:141-168``), with ``expert_y = expert_x * 1.5`` in
  the output dtype as in the reference round trip (``tests/test_all_to_all.py:249-250``).

Run from the repository root:  python tests/golden/make_golden.py
"""

from __future__ import annotations

import dataclasses
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from tests.all_to_all_utils import MoEConfig, RankTestData  # noqa: E402


def bf16_bits(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def make_case(name: str, cfg: MoEConfig, num_groups: int, world_size: int) -> None:
    rng = torch.Generator()
    rng.manual_seed(123)
    ranks = [RankTestData(cfg, rng, use_max_tokens=False) for _ in range(num_groups)]
    E, K, H, M = cfg.num_experts, cfg.experts_per_token, cfg.hidden_dim, cfg.max_num_tokens
    S = cfg.scale_dim
    cap = M * num_groups
    esz = cfg.in_dtype.itemsize

    expert_token_from: list[list[tuple[int, int]]] = [[] for _ in range(E)]
    for i_rank, rd in enumerate(ranks):
        for token_idx in range(rd.num_tokens):
            for expert_idx in rd.indices[token_idx].tolist():
                expert_token_from[expert_idx].append((i_rank, token_idx))

    counts = np.array([len(v) for v in expert_token_from], dtype=np.int32)
    x_bytes = [rd.x.contiguous().view(torch.uint8).reshape(rd.num_tokens, H * esz).numpy() for rd in ranks]
    expert_x = np.zeros((E, cap, H * esz), dtype=np.uint8)
    expert_xs = np.zeros((E, cap, S), dtype=np.float32)
    slot_map = np.full((num_groups, M, K), 0xFFFFFFFF, dtype=np.uint32)
    for e in range(E):
        for s, (r, t) in enumerate(expert_token_from[e]):
            expert_x[e, s] = x_bytes[r][t]
            if S:
                expert_xs[e, s] = ranks[r].x_scale[t].numpy()
            k = ranks[r].indices[t].tolist().index(e)
            slot_map[r, t, k] = s

    # expert_y = expert_x.to(out_dtype) * 1.5, computed by torch in the output dtype.
    ex_t = torch.from_numpy(expert_x).view(cfg.in_dtype).reshape(E, cap, H)
    expert_y = ex_t.to(cfg.out_dtype) * 1.5
    y32 = expert_y.to(torch.float32).numpy()
    outs = {}
    for r, rd in enumerate(ranks):
        acc = np.zeros((rd.num_tokens, H), dtype=np.float32)
        for t in range(rd.num_tokens):
            for j in range(H):
                total = np.float32(0.0)
                for k in range(K):
                    e = int(rd.indices[t, k])
                    w = np.float32(rd.weights[t, k].item())
                    prod = np.float32(w * y32[e, slot_map[r, t, k], j])
                    total = np.float32(total + prod)
                acc[t, j] = total
        outs[f"out_{r}"] = bf16_bits(torch.from_numpy(acc).to(cfg.out_dtype))

    arrays = dict(
        meta=np.array([E, K, H, M, num_groups, world_size, esz, S, cap], dtype=np.int64),
        counts=counts,
        expert_x=expert_x,
        expert_x_scale=expert_xs,
        slot_map=slot_map,
        expert_y_bits=bf16_bits(expert_y),
    )
    for r, rd in enumerate(ranks):
        arrays[f"n_{r}"] = np.array([rd.num_tokens], dtype=np.int64)
        arrays[f"x_{r}"] = x_bytes[r]
        arrays[f"indices_{r}"] = rd.indices.numpy().astype(np.uint32)
        arrays[f"weights_{r}"] = rd.weights.numpy()
        if S:
            arrays[f"x_scale_{r}"] = rd.x_scale.numpy()
    arrays.update(outs)
    path = os.path.join(HERE, f"{name}.npz")
    np.savez_compressed(path, **arrays)
    print(f"wrote {path}: tokens per group {[rd.num_tokens for rd in ranks]}, counts {counts.tolist()}")


def main() -> None:
    base = MoEConfig(num_experts=8, experts_per_token=3, hidden_dim=64, max_num_tokens=10)
    make_case("small_bf16", base, num_groups=2, world_size=4)
    fp8 = dataclasses.replace(base, hidden_dim=512, in_dtype=torch.float8_e4m3fn)
    make_case("small_fp8", fp8, num_groups=2, world_size=4)
    f16 = dataclasses.replace(base, in_dtype=torch.float16, out_dtype=torch.float16, max_num_tokens=6)
    make_case("small_f16", f16, num_groups=4, world_size=4)


if __name__ == "__main__":
    main()
