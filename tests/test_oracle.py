"""Pins the CPU oracle (``oracle/``) before anything is compared against it.

The reference holds no golden vectors for dispatch / combine (its tests are generative,
``tests/test_all_to_all.py:196-286``), so the oracle is pinned by: the committed vectors of
``tests/golden`` (made by literal loops that share no code with the oracle), three
independent restatements agreeing bit for bit, closed forms, the reference's own test
properties, and special cases that reduce to a copy or to a library routine.
"""

from __future__ import annotations

import dataclasses
import glob
import os

import numpy as np
import pytest
import torch

from oracle import a2a_oracle as orc
from tests.all_to_all_utils import (
    FP8,
    ORACLE_DTYPE,
    MoEConfig,
    RankTestData,
    WorkloadSpec,
    baseline_configs,
    generate,
    medium_moe,
    small_moe,
    to_oracle_groups,
    torch_bits,
)

GOLDEN = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "*.npz")))


def load_golden(path):
    z = np.load(path, allow_pickle=False)
    E, K, H, M, G, R, esz, S, cap = (int(v) for v in z["meta"])
    groups = []
    for g in range(G):
        n = int(z[f"n_{g}"][0])
        groups.append(
            orc.GroupData(
                z[f"x_{g}"], z[f"x_scale_{g}"] if S else None, z[f"indices_{g}"], z[f"weights_{g}"], n
            )
        )
    return z, dict(E=E, K=K, H=H, M=M, G=G, R=R, esz=esz, S=S, cap=cap), groups


def assert_dispatch_equal(a: orc.DispatchResult, b: orc.DispatchResult):
    np.testing.assert_array_equal(a.counts, b.counts)
    np.testing.assert_array_equal(a.expert_x, b.expert_x)
    np.testing.assert_array_equal(a.slot_map, b.slot_map)
    if a.expert_x_scale is not None or b.expert_x_scale is not None:
        np.testing.assert_array_equal(a.expert_x_scale.view(np.uint32), b.expert_x_scale.view(np.uint32))


@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p) for p in GOLDEN])
@pytest.mark.parametrize("impl", ["c", "np", "loop"])
def test_dispatch_matches_golden(path, impl):
    z, m, groups = load_golden(path)
    fn = {"c": orc.c_dispatch, "np": orc.np_dispatch, "loop": orc.loop_dispatch}[impl]
    res = fn(groups, m["M"], m["E"], m["K"], m["cap"])
    np.testing.assert_array_equal(res.counts, z["counts"])
    np.testing.assert_array_equal(res.expert_x, z["expert_x"])
    np.testing.assert_array_equal(res.slot_map, z["slot_map"])
    if m["S"]:
        np.testing.assert_array_equal(res.expert_x_scale.view(np.uint32), z["expert_x_scale"].view(np.uint32))


@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p) for p in GOLDEN])
@pytest.mark.parametrize("impl", ["c", "np", "loop"])
def test_combine_matches_golden(path, impl):
    z, m, groups = load_golden(path)
    name = os.path.basename(path)
    dt = orc.F16 if name.startswith("small_f16") else orc.BF16
    fn = {"c": orc.c_combine, "np": orc.np_combine, "loop": orc.loop_combine}[impl]
    outs = fn(groups, m["M"], m["E"], m["K"], m["H"], z["expert_y_bits"], dt, dt, z["slot_map"])
    for g, out in enumerate(outs):
        np.testing.assert_array_equal(out, z[f"out_{g}"])


def test_golden_detects_plausible_mistakes():
    """A swapped group order, a reversed token order or a wrong owner of a row must fail
    the golden comparison -- otherwise the vectors would pin nothing."""
    z, m, groups = load_golden([p for p in GOLDEN if "small_fp8" in p][0])
    good = orc.c_dispatch(groups, m["M"], m["E"], m["K"], m["cap"])
    np.testing.assert_array_equal(good.expert_x, z["expert_x"])
    swapped = orc.c_dispatch(groups[::-1], m["M"], m["E"], m["K"], m["cap"])
    assert not np.array_equal(swapped.expert_x, z["expert_x"])
    rev = [
        dataclasses.replace(
            g,
            x=g.x[: g.n][::-1].copy(),
            x_scale=g.x_scale[: g.n][::-1].copy(),
            indices=g.indices[: g.n][::-1].copy(),
        )
        for g in groups
    ]
    reversed_tokens = orc.c_dispatch(rev, m["M"], m["E"], m["K"], m["cap"])
    np.testing.assert_array_equal(reversed_tokens.counts, z["counts"])  # counts are order-free
    assert not np.array_equal(reversed_tokens.expert_x, z["expert_x"])
    # combine: pairing weight k with another pick's row, or reading through a wrong slot
    # map, fails the golden outputs
    dt = orc.BF16
    args = (m["M"], m["E"], m["K"], m["H"], z["expert_y_bits"], dt, dt)
    base = orc.c_combine(groups, *args, z["slot_map"])
    assert all(np.array_equal(a, z[f"out_{g}"]) for g, a in enumerate(base))
    wrong_w = [dataclasses.replace(g, weights=np.roll(g.weights, 1, axis=1) * 2.0) for g in groups]
    other = orc.c_combine(wrong_w, *args, z["slot_map"])
    assert any(not np.array_equal(a, z[f"out_{g}"]) for g, a in enumerate(other))
    wrong_slots = np.where(z["slot_map"] == 0xFFFFFFFF, z["slot_map"], (z["slot_map"] + 1) % 2)
    other = orc.c_combine(groups, *args, wrong_slots)
    assert any(not np.array_equal(a, z[f"out_{g}"]) for g, a in enumerate(other))


def reference_style_groups(cfg: MoEConfig, num_groups: int, seed: int):
    rng = torch.Generator()
    rng.manual_seed(seed)
    data = [RankTestData(cfg, rng, use_max_tokens=False) for _ in range(num_groups)]
    groups = []
    for rd in data:
        xb = rd.x.contiguous().view(torch.uint8).reshape(rd.num_tokens, -1).numpy()
        xs = None if rd.x_scale is None else rd.x_scale.numpy()
        groups.append(
            orc.GroupData(xb, xs, rd.indices.numpy().astype(np.uint32), rd.weights.numpy(), rd.num_tokens)
        )
    return data, groups


@pytest.mark.parametrize("in_dtype", [torch.bfloat16, FP8, torch.float16])
@pytest.mark.parametrize("cfg,num_groups", [(small_moe, 2), (medium_moe, 4)])
def test_three_restatements_agree_on_reference_geometries(cfg, num_groups, in_dtype):
    """small_moe (world 4, dp 2) and medium_moe of tests/test_all_to_all.py:26-38,313-355."""
    cfg = dataclasses.replace(cfg, in_dtype=in_dtype)
    _, groups = reference_style_groups(cfg, num_groups, seed=123)
    M, E, K = cfg.max_num_tokens, cfg.num_experts, cfg.experts_per_token
    cap = M * num_groups
    c = orc.c_dispatch(groups, M, E, K, cap)
    assert_dispatch_equal(c, orc.np_dispatch(groups, M, E, K, cap))
    assert_dispatch_equal(c, orc.loop_dispatch(groups, M, E, K, cap))


@pytest.mark.parametrize("seed", range(6))
def test_dispatch_closed_forms_and_reference_properties(seed):
    rs = np.random.RandomState(seed)
    E = int(rs.choice([4, 8, 24, 64]))
    K = int(rs.randint(1, min(E, 6) + 1))
    G = int(rs.randint(1, 5))
    M = int(rs.randint(1, 40))
    spec = WorkloadSpec("t", 90 + seed, G, E * G, K, 32, M, torch.bfloat16, tokens="uniform")
    E = spec.num_experts
    gi = generate(spec, seed=seed)
    groups = to_oracle_groups(gi)
    cap = M * G
    res = orc.c_dispatch(groups, M, E, K, cap)
    # counts: closed form and invariant
    flat = np.concatenate([g.indices[: g.n].ravel() for g in groups])
    np.testing.assert_array_equal(res.counts, np.bincount(flat, minlength=E))
    assert res.counts.sum() == K * sum(g.n for g in groups)
    # the reference's own check: per expert, the received rows are the routed rows as a set
    # (tests/test_all_to_all.py:212-246)
    for e in range(E):
        got = {bytes(res.expert_x[e, s]) for s in range(res.counts[e])}
        want = {bytes(g.x[t]) for g in groups for t in range(g.n) if e in g.indices[t]}
        assert got == want
    # slot map is a bijection onto [0, count) per expert, increasing in (group, token)
    for e in range(E):
        slots = [
            int(res.slot_map[gi_, t, k])
            for gi_, g in enumerate(groups)
            for t in range(g.n)
            for k in range(K)
            if g.indices[t, k] == e
        ]
        assert slots == list(range(res.counts[e]))
    # rows of tokens t >= n are never routed
    for gi_, g in enumerate(groups):
        assert (res.slot_map[gi_, g.n :] == 0xFFFFFFFF).all()
    assert_dispatch_equal(res, orc.np_dispatch(groups, M, E, K, cap))


def _combine_inputs(seed, E=8, K=3, H=64, M=12, G=2, y_dtype=torch.bfloat16):
    spec = WorkloadSpec("t", 70 + seed, G, E, K, H, M, torch.bfloat16, tokens="uniform")
    groups = to_oracle_groups(generate(spec, seed=seed))
    cap = M * G
    d = orc.c_dispatch(groups, M, E, K, cap)
    gen = torch.Generator().manual_seed(seed)
    y = torch.randn(E, cap, H, generator=gen).to(y_dtype)
    return spec, groups, d, y


@pytest.mark.parametrize("y_dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float16])
def test_combine_restatements_agree(y_dtype, out_dtype):
    spec, groups, d, y = _combine_inputs(3, y_dtype=y_dtype)
    args = (
        groups, spec.max_num_tokens, spec.num_experts, spec.experts_per_token, spec.hidden_dim,
        torch_bits(y), ORACLE_DTYPE[y_dtype], ORACLE_DTYPE[out_dtype], d.slot_map,
    )  # fmt: skip
    c = orc.c_combine(*args)
    for a, b, l in zip(c, orc.np_combine(*args), orc.loop_combine(*args)):
        np.testing.assert_array_equal(a, b)
        np.testing.assert_array_equal(a, l)


def test_combine_one_hot_weights_is_a_row_copy():
    spec, groups, d, y = _combine_inputs(5)
    K = spec.experts_per_token
    for pick in range(K):
        one_hot = [dataclasses.replace(g, weights=np.eye(K, dtype=np.float32)[[pick] * g.weights.shape[0]]) for g in groups]
        outs = orc.c_combine(
            one_hot, spec.max_num_tokens, spec.num_experts, K, spec.hidden_dim,
            torch_bits(y), orc.BF16, orc.BF16, d.slot_map,
        )  # fmt: skip
        yb = torch_bits(y)
        for gi, g in enumerate(groups):
            for t in range(g.n):
                e = g.indices[t, pick]
                np.testing.assert_array_equal(outs[gi][t], yb[e, d.slot_map[gi, t, pick]])


def test_combine_k1_is_a_scaled_copy_and_equal_rows_scale_by_weight_sum():
    # K = 1: out = bf16(w * y) -- one multiply, checked against torch's own arithmetic
    spec, groups, d, y = _combine_inputs(7, K=1)
    outs = orc.c_combine(
        groups, spec.max_num_tokens, spec.num_experts, 1, spec.hidden_dim,
        torch_bits(y), orc.BF16, orc.BF16, d.slot_map,
    )  # fmt: skip
    for gi, g in enumerate(groups):
        for t in range(g.n):
            row = y[int(g.indices[t, 0]), int(d.slot_map[gi, t, 0])].float()
            want = (row * float(g.weights[t, 0])).to(torch.bfloat16)
            np.testing.assert_array_equal(outs[gi][t], torch_bits(want))
    # every expert row identical and exactly representable weights: out = row * sum(w), exact
    spec, groups, d, _ = _combine_inputs(8, K=4)
    row = (torch.arange(spec.hidden_dim) % 7 - 3).to(torch.bfloat16)
    y = row.expand(spec.num_experts, spec.max_num_tokens * spec.num_dp_groups, spec.hidden_dim).contiguous()
    pow2 = [dataclasses.replace(g, weights=np.full_like(g.weights, 0.25)) for g in groups]
    outs = orc.c_combine(
        pow2, spec.max_num_tokens, spec.num_experts, 4, spec.hidden_dim,
        torch_bits(y), orc.BF16, orc.BF16, d.slot_map,
    )  # fmt: skip
    for gi, g in enumerate(groups):
        for t in range(g.n):
            np.testing.assert_array_equal(outs[gi][t], torch_bits(row))


@pytest.mark.parametrize("in_dtype", [torch.bfloat16, FP8, torch.float16])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float16])
def test_reference_round_trip_identity(in_dtype, out_dtype):
    """expert_y = expert_x.to(out) * 1.5, then y[:n] ~ sum_k x.to(out) * 1.5 * w accumulated
    in the output dtype, under torch.testing.assert_close defaults
    (tests/test_all_to_all.py:249-250,277-286)."""
    cfg = dataclasses.replace(small_moe, in_dtype=in_dtype, out_dtype=out_dtype)
    G = 2
    data, groups = reference_style_groups(cfg, G, seed=123)
    M, E, K, H = cfg.max_num_tokens, cfg.num_experts, cfg.experts_per_token, cfg.hidden_dim
    cap = M * G
    d = orc.c_dispatch(groups, M, E, K, cap)
    expert_x = torch.from_numpy(d.expert_x).view(in_dtype).reshape(E, cap, H)
    expert_y = expert_x.to(out_dtype) * 1.5
    code = ORACLE_DTYPE[out_dtype]
    outs = orc.c_combine(groups, M, E, K, H, torch_bits(expert_y), code, code, d.slot_map)
    for rd, out in zip(data, outs):
        y = torch.from_numpy(out.view(np.int16)).view(out_dtype)
        ref_y = torch.zeros(rd.num_tokens, H, dtype=out_dtype)
        for i_token in range(rd.num_tokens):
            for i_expert in range(K):
                weight = float(rd.weights[i_token, i_expert].item())
                ref_y[i_token] += rd.x[i_token].to(out_dtype) * 1.5 * weight
        torch.testing.assert_close(y, ref_y)


def test_float_conversions_match_libraries():
    lib = orc._c()
    rs = np.random.RandomState(0)
    bits = rs.randint(0, 2**32, size=20000, dtype=np.uint64).astype(np.uint32)
    special = np.array(
        [0, 0x80000000, 0x7F800000, 0xFF800000, 0x7FC00000, 0x7F7FFFFF, 0x00000001, 0x3F808000,
         0x3F818000, 0x3F808001, 0x477FE000, 0x477FF000, 0x33000000, 0x33000001, 0x387FC000,
         0x38800000, 0x3880E000, 0x33800000, 0x477FEFFF],
        dtype=np.uint32,
    )  # fmt: skip
    vals = np.concatenate([bits, special]).view(np.float32)
    with np.errstate(over="ignore", invalid="ignore"):
        want_f16 = vals.astype(np.float16).view(np.uint16)
    want_bf16 = torch.from_numpy(vals.copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    for v, wf, wb in zip(vals, want_f16, want_bf16):
        gf, gb = lib.oracle_float_to_f16(float(v)), lib.oracle_float_to_bf16(float(v))
        if np.isnan(v):
            assert (gf & 0x7C00) == 0x7C00 and (gf & 0x3FF) != 0
            assert (gb & 0x7F80) == 0x7F80 and (gb & 0x7F) != 0
        else:
            assert gf == wf, hex(v.view(np.uint32))
            assert gb == wb, hex(v.view(np.uint32))
    all16 = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    want = all16.view(np.float16).astype(np.float32)
    got = np.array([lib.oracle_f16_to_float(int(h)) for h in all16], dtype=np.float32)
    finite = ~np.isnan(want)
    np.testing.assert_array_equal(got[finite].view(np.uint32), want[finite].view(np.uint32))
    assert np.isnan(got[~finite]).all()


def test_bound_m_excludes_later_rows():
    spec = WorkloadSpec("t", 60, 2, 8, 2, 32, 9, torch.bfloat16)
    gi = generate(spec, seed=1)
    gi[0].n, gi[1].n = 4, 0
    groups = to_oracle_groups(gi)
    res = orc.c_dispatch(groups, 9, 8, 2, 18)
    assert res.counts.sum() == 2 * 4
    assert (res.slot_map[0, 4:] == 0xFFFFFFFF).all() and (res.slot_map[1] == 0xFFFFFFFF).all()
    assert_dispatch_equal(res, orc.np_dispatch(groups, 9, 8, 2, 18))


def test_torch_cpu_port_matches_c_oracle():
    """The timed CPU baseline (vectorised torch) computes what the C oracle computes."""
    spec = dataclasses.replace(baseline_configs()["C2"], max_num_tokens=16, hidden_dim=512)
    gi = generate(spec, seed=4)
    groups = to_oracle_groups(gi)
    M, E, K, H = spec.max_num_tokens, spec.num_experts, spec.experts_per_token, spec.hidden_dim
    cap = M * spec.num_dp_groups
    c = orc.c_dispatch(groups, M, E, K, cap)
    groups_t = [(g.x, g.x_scale, g.indices.to(torch.int64), g.n) for g in gi]
    counts, ex, exs, slot_flat = orc.torch_dispatch(groups_t, M, E, K, cap)
    np.testing.assert_array_equal(counts.numpy(), c.counts)
    for e in range(E):
        n = c.counts[e]
        np.testing.assert_array_equal(ex.view(torch.uint8)[e, :n].numpy(), c.expert_x[e, :n])
        np.testing.assert_array_equal(exs[e, :n].numpy().view(np.uint32), c.expert_x_scale[e, :n].view(np.uint32))
    y = torch.randn(E, cap, H, generator=torch.Generator().manual_seed(0)).to(torch.bfloat16)
    out = orc.torch_combine(groups_t, [g.weights for g in gi], slot_flat, y, torch.bfloat16)
    want = orc.c_combine(groups, M, E, K, H, torch_bits(y), orc.BF16, orc.BF16, c.slot_map)
    got = torch_bits(out)
    off = 0
    for g, w in zip(gi, want):
        # addcmul_ may fuse the multiply-add: compare as values, far inside bf16 tolerance
        a = orc.to_float32(got[off : off + g.n], orc.BF16)
        np.testing.assert_allclose(a, orc.to_float32(w, orc.BF16), rtol=8e-3, atol=1e-3)
        off += g.n
