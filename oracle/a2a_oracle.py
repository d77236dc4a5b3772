"""CPU oracle for the MoE dispatch / combine path.

TEST INFRASTRUCTURE ONLY: the product (the ``pplx_kernels`` package and its
``libpplx_kernels.so``) never imports this module.  It is the checker used by
``tests/``, ``__graft_entry__.smoke()`` and ``bench.py``'s ``cpu_baseline`` leg.

Three independent restatements of the reference's semantics live here so that
they can pin each other:

* ``c_dispatch`` / ``c_combine``      the plain-C loops of ``a2a_oracle.c``
* ``np_dispatch`` / ``np_combine``    closed forms (bincount, stable argsort, gather)
* ``loop_dispatch`` / ``loop_combine``  the literal Python loops of the reference's own
  torch check (reference ``tests/test_all_to_all.py:113-120`` and ``:277-286``), for
  tiny inputs only

plus ``torch_dispatch`` / ``torch_combine``, a vectorised multi-threaded torch CPU
port used as the timed CPU baseline.

Data model: one ``GroupData`` per DP group (the ranks of a group hold identical
tokens, reference ``csrc/all_to_all/all_to_all.cpp:22``).  All simulated ranks'
expert-major outputs are one array indexed by GLOBAL expert, ``[E, cap, ...]``;
rank ``r`` owns experts ``r*L .. r*L+L-1``
(reference ``csrc/all_to_all/intranode_dispatch.cu:133-134``).
"""

from __future__ import annotations

import ctypes
import dataclasses
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liba2a_oracle.so")

F32, BF16, F16 = 0, 1, 2
_NP_OF = {F32: np.float32, BF16: np.uint16, F16: np.uint16}


@dataclasses.dataclass
class GroupData:
    """Inputs of one DP group for one step."""

    x: np.ndarray  # uint8 [m, Hb]: the activation rows as raw bytes
    x_scale: np.ndarray | None  # float32 [m, S] or None
    indices: np.ndarray  # uint32 [m, K], distinct experts per row
    weights: np.ndarray  # float32 [m, K]
    n: int  # tokens present: bound_m if given else m (intranode_dispatch.cu:64)


@dataclasses.dataclass
class DispatchResult:
    counts: np.ndarray  # int32 [E]
    expert_x: np.ndarray  # uint8 [E, cap, Hb]; rows >= counts[e] are zero
    expert_x_scale: np.ndarray | None  # float32 [E, cap, S]
    slot_map: np.ndarray  # uint32 [G, M, K]; 0xffffffff where t >= n


def build(force: bool = False) -> str:
    """Compiles a2a_oracle.c next to this file (gcc) and returns the .so path."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B", "-s"])
    return _LIB_PATH


_lib = None


def _c():
    global _lib
    if _lib is None:
        lib = ctypes.CDLL(build())
        u32, i32, u64, i64 = ctypes.c_uint32, ctypes.c_int32, ctypes.c_uint64, ctypes.c_int64
        vp = ctypes.c_void_p
        lib.oracle_dispatch.restype = ctypes.c_int
        lib.oracle_dispatch.argtypes = [u32, u32, u32, u32, u64, u32, vp, vp, vp, vp, vp, vp, vp, vp, i64, vp]
        lib.oracle_combine.restype = ctypes.c_int
        lib.oracle_combine.argtypes = [u32, u32, u32, u32, u32, i32, i32, vp, i64, vp, vp, vp, vp, vp]
        lib.oracle_float_to_bf16.restype = ctypes.c_uint16
        lib.oracle_float_to_bf16.argtypes = [ctypes.c_float]
        lib.oracle_float_to_f16.restype = ctypes.c_uint16
        lib.oracle_float_to_f16.argtypes = [ctypes.c_float]
        lib.oracle_f16_to_float.restype = ctypes.c_float
        lib.oracle_f16_to_float.argtypes = [ctypes.c_uint16]
        lib.oracle_bf16_to_float.restype = ctypes.c_float
        lib.oracle_bf16_to_float.argtypes = [ctypes.c_uint16]
        _lib = lib
    return _lib


def _ptr_array(arrays):
    arr = (ctypes.c_void_p * len(arrays))()
    for i, a in enumerate(arrays):
        arr[i] = a.ctypes.data if a is not None else None
    return arr


def _check_groups(groups, M, K):
    for g in groups:
        assert g.x.dtype == np.uint8 and g.x.ndim == 2
        assert g.indices.dtype == np.uint32 and g.indices.shape[1] == K
        assert g.n <= g.indices.shape[0] and g.n <= M


# --------------------------------------------------------------------------- C


def c_dispatch(groups: list[GroupData], M: int, E: int, K: int, cap: int) -> DispatchResult:
    _check_groups(groups, M, K)
    G = len(groups)
    Hb = groups[0].x.shape[1]
    S = 0 if groups[0].x_scale is None else groups[0].x_scale.shape[1]
    xs = [np.ascontiguousarray(g.x) for g in groups]
    scales = [None if S == 0 else np.ascontiguousarray(g.x_scale, dtype=np.float32) for g in groups]
    idx = [np.ascontiguousarray(g.indices) for g in groups]
    strides = np.array([x.strides[0] if x.shape[0] else Hb for x in xs], dtype=np.int64)
    n = np.array([g.n for g in groups], dtype=np.uint32)
    counts = np.zeros(E, dtype=np.int32)
    expert_x = np.zeros((E, cap, Hb), dtype=np.uint8)
    expert_xs = np.zeros((E, cap, S), dtype=np.float32) if S else None
    slot_map = np.full((G, M, K), 0xFFFFFFFF, dtype=np.uint32)
    rc = _c().oracle_dispatch(
        G, M, E, K, Hb, S,
        _ptr_array(xs), strides.ctypes.data, _ptr_array(scales), _ptr_array(idx), n.ctypes.data,
        counts.ctypes.data, expert_x.ctypes.data,
        expert_xs.ctypes.data if S else None, cap, slot_map.ctypes.data,
    )  # fmt: skip
    if rc:
        raise ValueError({1: "expert index out of range", 2: "row does not fit cap"}[rc])
    return DispatchResult(counts, expert_x, expert_xs, slot_map)


def c_combine(
    groups: list[GroupData], M: int, E: int, K: int, H: int,
    expert_y: np.ndarray, in_dtype: int, out_dtype: int, slot_map: np.ndarray,
) -> list[np.ndarray]:  # fmt: skip
    """expert_y: [E, cap, H] as float32 (F32) or uint16 bit patterns (BF16 / F16).
    Returns per group a uint16 [n, H] array of out_dtype bit patterns."""
    G = len(groups)
    assert expert_y.dtype == _NP_OF[in_dtype] and expert_y.shape[0] == E and expert_y.shape[2] == H
    expert_y = np.ascontiguousarray(expert_y)
    idx = [np.ascontiguousarray(g.indices) for g in groups]
    wts = [np.ascontiguousarray(g.weights, dtype=np.float32) for g in groups]
    n = np.array([g.n for g in groups], dtype=np.uint32)
    slot_map = np.ascontiguousarray(slot_map, dtype=np.uint32)
    outs = [np.zeros((g.n, H), dtype=np.uint16) for g in groups]
    rc = _c().oracle_combine(
        G, M, E, K, H, in_dtype, out_dtype, expert_y.ctypes.data, expert_y.shape[1],
        _ptr_array(idx), _ptr_array(wts), n.ctypes.data, slot_map.ctypes.data, _ptr_array(outs),
    )  # fmt: skip
    if rc:
        raise ValueError(f"oracle_combine failed with code {rc}")
    return outs


# ----------------------------------------------------------------- closed forms


def np_dispatch(groups: list[GroupData], M: int, E: int, K: int, cap: int) -> DispatchResult:
    """Stable sort of all (group, token, pick) triples by expert id: the closed form
    of "append in (dp_rank asc, token asc) order" (tests/test_all_to_all.py:113-120)."""
    _check_groups(groups, M, K)
    G = len(groups)
    Hb = groups[0].x.shape[1]
    S = 0 if groups[0].x_scale is None else groups[0].x_scale.shape[1]
    flat_e = np.concatenate([g.indices[: g.n].reshape(-1).astype(np.int64) for g in groups])
    flat_g = np.concatenate([np.full(g.n * K, i, dtype=np.int64) for i, g in enumerate(groups)])
    flat_t = np.concatenate([np.repeat(np.arange(g.n, dtype=np.int64), K) for g in groups])
    flat_k = np.concatenate([np.tile(np.arange(K, dtype=np.int64), g.n) for g in groups])
    if flat_e.size and flat_e.max() >= E:
        raise ValueError("expert index out of range")
    counts = np.bincount(flat_e, minlength=E).astype(np.int32)
    if counts.size and counts.max() > cap:
        raise ValueError("row does not fit cap")
    order = np.argsort(flat_e, kind="stable")
    starts = np.concatenate([[0], np.cumsum(counts)[:-1]])
    e_sorted = flat_e[order]
    slot_sorted = np.arange(order.size) - starts[e_sorted]
    expert_x = np.zeros((E, cap, Hb), dtype=np.uint8)
    expert_xs = np.zeros((E, cap, S), dtype=np.float32) if S else None
    slot_map = np.full((G, M, K), 0xFFFFFFFF, dtype=np.uint32)
    for gi, g in enumerate(groups):
        sel = flat_g[order] == gi
        expert_x[e_sorted[sel], slot_sorted[sel]] = g.x[flat_t[order][sel]]
        if S:
            expert_xs[e_sorted[sel], slot_sorted[sel]] = g.x_scale[flat_t[order][sel]]
    slot_map[flat_g[order], flat_t[order], flat_k[order]] = slot_sorted.astype(np.uint32)
    return DispatchResult(counts, expert_x, expert_xs, slot_map)


def to_float32(a: np.ndarray, dtype: int) -> np.ndarray:
    if dtype == F32:
        return a.astype(np.float32, copy=False)
    if dtype == BF16:
        return (a.astype(np.uint32) << 16).view(np.float32)
    return a.view(np.float16).astype(np.float32)


def from_float32(a: np.ndarray, dtype: int) -> np.ndarray:
    """float32 -> bf16 / f16 bit patterns through library conversions
    (torch for bf16, numpy for f16), both round-to-nearest-even."""
    if dtype == BF16:
        import torch

        return torch.from_numpy(np.ascontiguousarray(a)).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    if dtype == F16:
        return a.astype(np.float16).view(np.uint16)
    raise ValueError("out dtype must be BF16 or F16")


def np_combine(
    groups: list[GroupData], M: int, E: int, K: int, H: int,
    expert_y: np.ndarray, in_dtype: int, out_dtype: int, slot_map: np.ndarray,
) -> list[np.ndarray]:  # fmt: skip
    """sum_k w[t,k] * float(expert_y[e_k, slot(t,k), :]) in fp32, k ascending, separate
    multiply and add (csrc/all_to_all/intranode_combine.cu:141-168), then cast."""
    outs = []
    for gi, g in enumerate(groups):
        acc = np.zeros((g.n, H), dtype=np.float32)
        for k in range(K):
            e = g.indices[: g.n, k].astype(np.int64)
            slot = slot_map[gi, : g.n, k].astype(np.int64)
            rows = to_float32(expert_y[e, slot], in_dtype)
            acc = acc + g.weights[: g.n, k : k + 1].astype(np.float32) * rows
        outs.append(from_float32(acc, out_dtype))
    return outs


# -------------------------------------------------------------- literal loops


def loop_dispatch(groups: list[GroupData], M: int, E: int, K: int, cap: int) -> DispatchResult:
    """The reference test's own enumeration, verbatim in structure
    (tests/test_all_to_all.py:113-120): expert_token_from[e].append((i_rank, token_idx))."""
    G = len(groups)
    Hb = groups[0].x.shape[1]
    S = 0 if groups[0].x_scale is None else groups[0].x_scale.shape[1]
    expert_token_from: list[list[tuple[int, int]]] = [[] for _ in range(E)]
    for i_rank, rd in enumerate(groups):
        for token_idx in range(rd.n):
            for expert_idx in rd.indices[token_idx]:
                expert_token_from[int(expert_idx)].append((i_rank, token_idx))
    counts = np.array([len(lst) for lst in expert_token_from], dtype=np.int32)
    expert_x = np.zeros((E, cap, Hb), dtype=np.uint8)
    expert_xs = np.zeros((E, cap, S), dtype=np.float32) if S else None
    slot_map = np.full((G, M, K), 0xFFFFFFFF, dtype=np.uint32)
    for e, lst in enumerate(expert_token_from):
        for s, (r, t) in enumerate(lst):
            expert_x[e, s] = groups[r].x[t]
            if S:
                expert_xs[e, s] = groups[r].x_scale[t]
            k = int(np.nonzero(groups[r].indices[t] == e)[0][0])
            slot_map[r, t, k] = s
    return DispatchResult(counts, expert_x, expert_xs, slot_map)


def loop_combine(
    groups: list[GroupData], M: int, E: int, K: int, H: int,
    expert_y: np.ndarray, in_dtype: int, out_dtype: int, slot_map: np.ndarray,
) -> list[np.ndarray]:  # fmt: skip
    outs = []
    y32 = to_float32(expert_y, in_dtype)
    for gi, g in enumerate(groups):
        acc = np.zeros((g.n, H), dtype=np.float32)
        for t in range(g.n):
            for k in range(K):
                e = int(g.indices[t, k])
                w = np.float32(g.weights[t, k])
                acc[t] = acc[t] + w * y32[e, int(slot_map[gi, t, k])]
        outs.append(from_float32(acc, out_dtype))
    return outs


# ------------------------------------------------------ torch CPU port (timed)


def torch_dispatch(groups_t, M: int, E: int, K: int, cap: int):
    """Vectorised torch CPU dispatch over all groups.

    groups_t: list of (x [m, H] any dtype, x_scale [m, S] | None, indices int64 [m, K], n).
    Returns (counts int32 [E], expert_x [E, cap, H], expert_x_scale | None, slot_map list).
    Same routing as np_dispatch: stable argsort on the expert id."""
    import torch

    xs = torch.cat([x[:n] for x, _, _, n in groups_t])
    has_scale = groups_t[0][1] is not None
    scales = torch.cat([s[:n] for _, s, _, n in groups_t]) if has_scale else None
    flat_e = torch.cat([i[:n].reshape(-1) for _, _, i, n in groups_t])
    counts = torch.bincount(flat_e, minlength=E)
    order = torch.argsort(flat_e, stable=True)
    e_sorted = flat_e[order]
    starts = torch.cumsum(counts, 0) - counts
    slot_sorted = torch.arange(order.numel()) - starts[e_sorted]
    src_token = order // K  # row in the concatenated token list
    expert_x = torch.empty((E, cap) + tuple(xs.shape[1:]), dtype=xs.dtype)
    flat_rows = e_sorted * cap + slot_sorted
    expert_x.view(E * cap, -1).view(torch.uint8).index_copy_(
        0, flat_rows, xs.view(torch.uint8).reshape(xs.shape[0], -1).index_select(0, src_token)
    )
    expert_xs = None
    if has_scale:
        expert_xs = torch.empty((E, cap, scales.shape[1]), dtype=torch.float32)
        expert_xs.view(E * cap, -1).index_copy_(0, flat_rows, scales.index_select(0, src_token))
    slot_flat = torch.empty_like(slot_sorted)
    slot_flat[order] = slot_sorted
    return counts.to(torch.int32), expert_x, expert_xs, slot_flat.view(-1, K)


def torch_combine(groups_t, weights_t, slot_flat, expert_y, out_dtype):
    """Vectorised torch CPU combine: gather K rows per token, fp32 weighted sum, cast.
    groups_t as for torch_dispatch; weights_t: list of float32 [m, K]; slot_flat from
    torch_dispatch; expert_y [E, cap, H].  Returns the concatenated [T, H] result."""
    import torch

    E, cap, H = expert_y.shape
    K = slot_flat.shape[1]
    e = torch.cat([i[:n] for _, _, i, n in groups_t])
    w = torch.cat([wt[:n] for wt, (_, _, _, n) in zip(weights_t, groups_t)])
    rows = (e * cap + slot_flat).reshape(-1)
    y = expert_y.view(E * cap, H).index_select(0, rows).view(-1, K, H)
    acc = torch.zeros((y.shape[0], H), dtype=torch.float32)
    for k in range(K):
        acc.addcmul_(y[:, k].to(torch.float32), w[:, k : k + 1])
    return acc.to(out_dtype)
