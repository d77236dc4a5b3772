"""Loads ``libpplx_kernels.so`` (the C ABI of ``include/pplx_a2a.h``) and registers the
``torch.ops.pplx_kernels`` operators with the reference's schemas.

Mirrors the reference's binding layer: the loader of ``src/pplx_kernels/ops.py:8-16`` and
the op registration + tensor checks of ``csrc/bindings/all_to_all_ops.cpp:19-24,110-196,
238-311,329-391``.  Differences that follow from the single-GPU loopback:

* the library has no torch types in its interface, so the tensor checks and the stride
  extraction happen here and raw pointers cross a ctypes call;
* ``all_to_all_intranode_create`` resolves ``group_name`` to a process-local *world* that
  owns the state shared by all simulated ranks (the reference resolves a c10d process group
  and exchanges IPC handles, ``csrc/bindings/all_to_all_ops.cpp:79-106``);
* a missing or unloadable library is an ``ImportError`` when an op is first used, never a
  silent fallback.
"""

from __future__ import annotations

import atexit
import ctypes
import os
import threading

import torch

_LIB_NAME = "libpplx_kernels.so"
_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), _LIB_NAME)

SPLIT_NONE, SPLIT_SEND, SPLIT_RECV = 0, 1, 2
DTYPE_CODE = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}

STATUS_NAMES = {
    0: "ok",
    1: "invalid argument",
    2: "invalid state",
    3: "HIP error",
    4: "unsupported",
}

# Every symbol include/pplx_a2a.h declares.
EXPORTED_SYMBOLS = (
    "pplx_a2a_world_create",
    "pplx_a2a_world_destroy",
    "pplx_a2a_create",
    "pplx_a2a_destroy",
    "pplx_a2a_num_experts_per_token",
    "pplx_a2a_rank",
    "pplx_a2a_dispatch",
    "pplx_a2a_combine",
    "pplx_a2a_world_dispatch",
    "pplx_a2a_world_combine",
    "pplx_a2a_static_step",
    "pplx_a2a_world_reserve_split",
    "pplx_a2a_world_faults",
    "pplx_a2a_graph_begin_capture",
    "pplx_a2a_graph_end_capture",
    "pplx_a2a_graph_launch",
    "pplx_a2a_graph_destroy",
    "pplx_a2a_last_error",
    "pplx_a2a_version",
    "pplx_a2a_build_id",
)


class Config(ctypes.Structure):
    """pplx_a2a_config_t"""

    _fields_ = [
        ("max_num_tokens", ctypes.c_uint64),
        ("num_experts", ctypes.c_uint64),
        ("experts_per_token", ctypes.c_uint64),
        ("world_size", ctypes.c_uint32),
        ("dp_size", ctypes.c_uint32),
        ("hidden_dim", ctypes.c_uint64),
        ("hidden_dim_bytes", ctypes.c_uint64),
        ("hidden_dim_scale_bytes", ctypes.c_uint64),
    ]


class DispatchArgs(ctypes.Structure):
    """pplx_a2a_dispatch_args_t"""

    _fields_ = [
        ("out_expert_num_tokens", ctypes.c_void_p),
        ("out_expert_num_tokens_stride", ctypes.c_int64),
        ("out_expert_x", ctypes.c_void_p),
        ("out_expert_x_stride_row", ctypes.c_int64),
        ("out_expert_x_stride_expert", ctypes.c_int64),
        ("out_expert_x_rows", ctypes.c_int64),
        ("out_expert_x_scale", ctypes.c_void_p),
        ("out_expert_x_scale_stride_elem", ctypes.c_int64),
        ("out_expert_x_scale_stride_row", ctypes.c_int64),
        ("out_expert_x_scale_stride_expert", ctypes.c_int64),
        ("dp_x", ctypes.c_void_p),
        ("dp_x_stride_row", ctypes.c_int64),
        ("dp_x_scale", ctypes.c_void_p),
        ("dp_x_scale_stride_elem", ctypes.c_int64),
        ("dp_x_scale_stride_row", ctypes.c_int64),
        ("indices", ctypes.c_void_p),
        ("m", ctypes.c_uint32),
        ("bound_m", ctypes.c_void_p),
    ]


class CombineArgs(ctypes.Structure):
    """pplx_a2a_combine_args_t"""

    _fields_ = [
        ("out_tokens", ctypes.c_void_p),
        ("out_tokens_stride_row", ctypes.c_int64),
        ("out_dtype", ctypes.c_int32),
        ("indices", ctypes.c_void_p),
        ("weights", ctypes.c_void_p),
        ("weights_stride_row", ctypes.c_int64),
        ("expert_y", ctypes.c_void_p),
        ("expert_y_stride_row", ctypes.c_int64),
        ("expert_y_stride_expert", ctypes.c_int64),
        ("expert_y_rows", ctypes.c_int64),
        ("in_dtype", ctypes.c_int32),
        ("m", ctypes.c_uint32),
        ("bound_m", ctypes.c_void_p),
    ]


_lib = None
_lib_lock = threading.Lock()


def load_library() -> ctypes.CDLL:
    """Returns the loaded C-ABI library; raises ImportError if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    with _lib_lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(_LIB_PATH):
            raise ImportError(
                f"{_LIB_PATH} is missing: build it with `make -C pplx-kernels_amd/csrc` "
                "(or __graft_entry__.build()); there is no fallback implementation"
            )
        try:
            lib = ctypes.CDLL(_LIB_PATH)
        except OSError as exc:  # e.g. no HIP runtime on this machine
            raise ImportError(f"cannot load {_LIB_PATH}: {exc}") from exc
        vp, i32, u32 = ctypes.c_void_p, ctypes.c_int, ctypes.c_uint32
        lib.pplx_a2a_world_create.argtypes = [ctypes.POINTER(Config), i32, ctypes.POINTER(vp)]
        lib.pplx_a2a_world_destroy.argtypes = [vp]
        lib.pplx_a2a_create.argtypes = [vp, u32, ctypes.POINTER(vp)]
        lib.pplx_a2a_destroy.argtypes = [vp]
        lib.pplx_a2a_num_experts_per_token.argtypes = [vp]
        lib.pplx_a2a_num_experts_per_token.restype = ctypes.c_uint64
        lib.pplx_a2a_rank.argtypes = [vp]
        lib.pplx_a2a_rank.restype = u32
        lib.pplx_a2a_dispatch.argtypes = [vp, ctypes.POINTER(DispatchArgs), i32, vp]
        lib.pplx_a2a_combine.argtypes = [vp, ctypes.POINTER(CombineArgs), i32, vp]
        lib.pplx_a2a_world_dispatch.argtypes = [vp, ctypes.POINTER(DispatchArgs), vp]
        lib.pplx_a2a_world_combine.argtypes = [vp, ctypes.POINTER(CombineArgs), vp]
        lib.pplx_a2a_static_step.argtypes = [
            ctypes.POINTER(Config), i32, ctypes.POINTER(DispatchArgs), ctypes.POINTER(CombineArgs), vp, vp,
        ]  # fmt: skip
        lib.pplx_a2a_world_reserve_split.argtypes = [vp, u32]
        lib.pplx_a2a_world_faults.argtypes = [vp, vp, ctypes.POINTER(u32)]
        lib.pplx_a2a_graph_begin_capture.argtypes = [vp]
        lib.pplx_a2a_graph_end_capture.argtypes = [vp, ctypes.POINTER(vp)]
        lib.pplx_a2a_graph_launch.argtypes = [vp, vp]
        lib.pplx_a2a_graph_destroy.argtypes = [vp]
        lib.pplx_a2a_last_error.restype = ctypes.c_char_p
        lib.pplx_a2a_version.restype = ctypes.c_char_p
        lib.pplx_a2a_build_id.restype = ctypes.c_char_p
        for name in EXPORTED_SYMBOLS:
            getattr(lib, name)  # AttributeError here means a stale or foreign library
        _lib = lib
    return _lib


def check_status(status: int) -> None:
    """Turns a non-zero pplx_a2a_status into the exception the reference would raise
    (TORCH_CHECK -> RuntimeError, csrc/bindings/all_to_all_ops.cpp:19-24)."""
    if status == 0:
        return
    msg = load_library().pplx_a2a_last_error().decode()
    raise RuntimeError(f"pplx_kernels: {STATUS_NAMES.get(status, status)}: {msg}")


# ---------------------------------------------------------------------------
# Worlds: group_name -> the owner of all simulated ranks' shared state.
# ---------------------------------------------------------------------------
class _World:
    def __init__(self, key, cfg_tuple, ptr):
        self.key = key
        self.cfg = cfg_tuple
        self.ptr = ptr
        self.handles: set[int] = set()
        self.experts_per_token = cfg_tuple[2]
        self.world_size = cfg_tuple[3]
        # A step's kernels are enqueued by the last rank to call, so the tensors of the
        # ranks that called earlier are kept alive until then: a temporary such as
        # ``x.to(device)`` must not go back to the caching allocator before it is read.
        # (the same holds for every phase of split mode, which is collective as well)
        self.pending: dict[str, dict[int, tuple]] = {
            f"{op}{mode}": {} for op in ("dispatch", "combine") for mode in (SPLIT_NONE, SPLIT_SEND, SPLIT_RECV)
        }
        # Widest expert_y element (bytes) that split-mode staging has been reserved for;
        # -1 = none reserved yet.
        self.split_reserved = -1

    def hold(self, kind: str, fptr: int, tensors: tuple) -> None:
        held = self.pending[kind]
        held[fptr] = tensors
        if len(held) >= self.world_size:
            held.clear()

    def release(self, fptr: int) -> None:
        """A handle that is destroyed in the middle of a step takes its half-made calls along."""
        for held in self.pending.values():
            held.pop(fptr, None)


_worlds: dict[str, _World] = {}
_handle_world: dict[int, _World] = {}
_registry_lock = threading.Lock()


def world_of(fptr: int) -> _World:
    return _handle_world[fptr]


def _create(
    transport: str,
    max_num_tokens: int,
    num_experts: int,
    experts_per_token: int,
    rank: int,
    world_size: int,
    dp_size: int,
    hidden_dim: int,
    hidden_dim_bytes: int,
    hidden_dim_scale_bytes: int,
    group_name: str,
) -> int:
    lib = load_library()
    cfg_tuple = (
        max_num_tokens,
        num_experts,
        experts_per_token,
        world_size,
        dp_size,
        hidden_dim,
        hidden_dim_bytes,
        hidden_dim_scale_bytes,
    )
    key = f"{transport}:{group_name}"
    with _registry_lock:
        world = _worlds.get(key)
        if world is not None and world.cfg != cfg_tuple:
            raise RuntimeError(
                f"pplx_kernels: group '{group_name}' already holds a world with a different "
                f"configuration {world.cfg}; destroy its ranks first or use another group_name"
            )
        if world is None:
            if min(cfg_tuple) < 0 or world_size <= 0 or dp_size <= 0:
                raise RuntimeError("pplx_kernels: invalid argument: negative or zero size")
            cfg = Config(*cfg_tuple)
            ptr = ctypes.c_void_p()
            device = torch.cuda.current_device() if torch.cuda.is_available() else 0
            check_status(lib.pplx_a2a_world_create(ctypes.byref(cfg), device, ctypes.byref(ptr)))
            world = _World(key, cfg_tuple, ptr.value)
            _worlds[key] = world
        if rank < 0:
            raise RuntimeError("pplx_kernels: invalid argument: negative rank")
        handle = ctypes.c_void_p()
        try:
            check_status(lib.pplx_a2a_create(world.ptr, rank, ctypes.byref(handle)))
        except RuntimeError:
            if not world.handles:
                lib.pplx_a2a_world_destroy(world.ptr)
                del _worlds[key]
            raise
        world.handles.add(handle.value)
        _handle_world[handle.value] = world
        return handle.value


def _destroy(fptr: int) -> None:
    lib = load_library()
    with _registry_lock:
        world = _handle_world.pop(fptr, None)
        if world is None:
            raise RuntimeError(f"pplx_kernels: unknown all-to-all handle {fptr:#x}")
        check_status(lib.pplx_a2a_destroy(fptr))
        world.handles.discard(fptr)
        world.release(fptr)
        if not world.handles:
            check_status(lib.pplx_a2a_world_destroy(world.ptr))
            _worlds.pop(world.key, None)


def _destroy_all() -> None:
    """Interpreter exit: release every world while Python and the HIP runtime are still up;
    AllToAll.__del__ finds nothing left to do afterwards."""
    try:
        lib = load_library()
    except ImportError:
        return
    with _registry_lock:
        for fptr in list(_handle_world):
            lib.pplx_a2a_destroy(fptr)
        _handle_world.clear()
        for world in list(_worlds.values()):
            lib.pplx_a2a_world_destroy(world.ptr)
        _worlds.clear()


atexit.register(_destroy_all)


def reserve_split(world: _World, expert_y_elem_bytes: int) -> None:
    """Split send / recv calls go through staging that the library never allocates inside
    dispatch / combine.  The reference's callers do not know of it, so the binding reserves it
    the first time a rank splits a call (and widens it for a wider ``expert_y`` dtype); like
    any allocation this synchronises and cannot happen under stream capture: run one eager
    step before capturing split calls, or call this up front."""
    if world.split_reserved >= expert_y_elem_bytes:
        return
    check_status(load_library().pplx_a2a_world_reserve_split(world.ptr, expert_y_elem_bytes))
    world.split_reserved = expert_y_elem_bytes


def is_live(fptr: int) -> bool:
    return fptr in _handle_world


def _create_intranode(
    max_num_tokens: int,
    num_experts: int,
    experts_per_token: int,
    rank: int,
    world_size: int,
    dp_size: int,
    hidden_dim: int,
    hidden_dim_bytes: int,
    hidden_dim_scale_bytes: int,
    group_name: str,
) -> int:
    return _create(
        "intranode",
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


def _create_internode(
    max_num_tokens: int,
    num_experts: int,
    experts_per_token: int,
    rank: int,
    world_size: int,
    dp_size: int,
    hidden_dim: int,
    hidden_dim_bytes: int,
    hidden_dim_scale_bytes: int,
) -> int:
    # One HBM has no second transport: the internode constructor attaches to a
    # loopback world of its own and runs the same kernels.
    return _create(
        "internode",
        max_num_tokens,
        num_experts,
        experts_per_token,
        rank,
        world_size,
        dp_size,
        hidden_dim,
        hidden_dim_bytes,
        hidden_dim_scale_bytes,
        "default",
    )


# ---------------------------------------------------------------------------
# Tensor checks (csrc/bindings/all_to_all_ops.cpp:19-24) and argument packing
# ---------------------------------------------------------------------------
def _check(cond: bool, msg: str) -> None:
    if not cond:
        raise RuntimeError(msg)


def _check_tensor(ndim: int, x: torch.Tensor, name: str) -> None:
    # (messages are only formatted on failure: these run on every call of the hot path)
    if not x.is_cuda:
        raise RuntimeError(f"Tensor {name} must be on GPU")
    if not x.is_contiguous():
        raise RuntimeError(f"Tensor {name} must be contiguous")
    if x.dim() != ndim:
        raise RuntimeError(f"Tensor {name} must be {ndim} dimensional")


def _check_bound_m(bound_m: torch.Tensor | None) -> None:
    if bound_m is not None:
        _check_tensor(1, bound_m, "boundM.value()")
        _check(bound_m.dtype == torch.uint32, "boundM must be of type UInt32")
        _check(bound_m.numel() == 1, "boundM must be a scalar tensor")


def split_mode(do_send: bool, do_recv: bool) -> int:
    """getSplitMode, csrc/bindings/all_to_all_ops.cpp:110-120."""
    if do_send and do_recv:
        return SPLIT_NONE
    if do_send:
        return SPLIT_SEND
    if do_recv:
        return SPLIT_RECV
    raise RuntimeError("Invalid split mode")


def pack_dispatch_args(
    experts_per_token: int,
    out_expert_num_tokens: torch.Tensor,
    out_expert_x: torch.Tensor,
    out_expert_x_scale: torch.Tensor | None,
    dp_x: torch.Tensor,
    dp_x_scale: torch.Tensor | None,
    indices: torch.Tensor,
    bound_m: torch.Tensor | None,
    out: DispatchArgs | None = None,
) -> DispatchArgs:
    """Checks of csrc/bindings/all_to_all_ops.cpp:135-161 and the views of :165-195."""
    _check_tensor(1, out_expert_num_tokens, "outExpertNumTokens")
    _check(out_expert_num_tokens.dtype == torch.int32, "outExpertNumTokens must be of type Int")
    _check_tensor(3, out_expert_x, "outExpertX")
    if out_expert_x_scale is not None:
        _check(out_expert_x_scale.is_cuda, "Tensor outExpertXScale must be on GPU")
        _check(out_expert_x_scale.dim() == 3, "Tensor outExpertXScale must be 3 dimensional")
        _check(out_expert_x_scale.dtype == torch.float32, "outExpertXScale must be of type Float")
    _check_tensor(2, dp_x, "dpX")
    if dp_x_scale is not None:
        _check(dp_x_scale.is_cuda, "Tensor dpXScale must be on GPU")
        _check(dp_x_scale.dim() == 2, "Tensor dpXScale must be 2 dimensional")
        _check(dp_x_scale.dtype == torch.float32, "dpXScale must be of type Float")
    _check_tensor(2, indices, "indices")
    _check(indices.dtype == torch.uint32, "indices must be of type UInt32")
    _check_bound_m(bound_m)
    _check(indices.size(0) == dp_x.size(0), "indices.size(0) must be equal to dpX.size(0)")
    _check(
        indices.size(1) == experts_per_token,
        "indices.size(1) must be equal to the experts per token",
    )

    a = out if out is not None else DispatchArgs()
    a.out_expert_num_tokens = out_expert_num_tokens.data_ptr()
    a.out_expert_num_tokens_stride = out_expert_num_tokens.stride(0)
    esz = out_expert_x.element_size()
    a.out_expert_x = out_expert_x.data_ptr()
    a.out_expert_x_stride_row = out_expert_x.stride(1) * esz
    a.out_expert_x_stride_expert = out_expert_x.stride(0) * esz
    a.out_expert_x_rows = out_expert_x.size(1)
    if out_expert_x_scale is not None:
        a.out_expert_x_scale = out_expert_x_scale.data_ptr()
        a.out_expert_x_scale_stride_elem = out_expert_x_scale.stride(2)
        a.out_expert_x_scale_stride_row = out_expert_x_scale.stride(1)
        a.out_expert_x_scale_stride_expert = out_expert_x_scale.stride(0)
    else:
        a.out_expert_x_scale = None
        a.out_expert_x_scale_stride_elem = 0
        a.out_expert_x_scale_stride_row = 0
        a.out_expert_x_scale_stride_expert = 0
    a.dp_x = dp_x.data_ptr()
    a.dp_x_stride_row = dp_x.stride(0) * dp_x.element_size()
    if dp_x_scale is not None:
        a.dp_x_scale = dp_x_scale.data_ptr()
        a.dp_x_scale_stride_elem = dp_x_scale.stride(1)
        a.dp_x_scale_stride_row = dp_x_scale.stride(0)
    else:
        a.dp_x_scale = None
        a.dp_x_scale_stride_elem = 0
        a.dp_x_scale_stride_row = 0
    a.indices = indices.data_ptr()
    a.m = indices.size(0)
    a.bound_m = bound_m.data_ptr() if bound_m is not None else None
    return a


def pack_combine_args(
    out_tokens: torch.Tensor,
    indices: torch.Tensor,
    weights: torch.Tensor,
    expert_y: torch.Tensor,
    bound_m: torch.Tensor | None,
    out: CombineArgs | None = None,
) -> CombineArgs:
    """Checks of csrc/bindings/all_to_all_ops.cpp:249-259, dtype switch of :265-310 and
    the element-stride views of :222-235."""
    _check_tensor(2, out_tokens, "outTokens")
    _check_tensor(2, indices, "indices")
    _check(indices.dtype == torch.uint32, "indices must be of type UInt32")
    _check_tensor(2, weights, "weights")
    _check(weights.dtype == torch.float32, "weights must be of type Float")
    _check_tensor(3, expert_y, "expertY")
    _check_bound_m(bound_m)
    _check(expert_y.dtype in DTYPE_CODE, "Unsupported dtype for expertY")
    _check(out_tokens.dtype in (torch.bfloat16, torch.float16), "Unsupported dtype for outTokens")

    a = out if out is not None else CombineArgs()
    a.out_tokens = out_tokens.data_ptr()
    a.out_tokens_stride_row = out_tokens.stride(0)
    a.out_dtype = DTYPE_CODE[out_tokens.dtype]
    a.indices = indices.data_ptr()
    a.weights = weights.data_ptr()
    a.weights_stride_row = weights.stride(0)
    a.expert_y = expert_y.data_ptr()
    a.expert_y_stride_row = expert_y.stride(1)
    a.expert_y_stride_expert = expert_y.stride(0)
    a.expert_y_rows = expert_y.size(1)
    a.in_dtype = DTYPE_CODE[expert_y.dtype]
    a.m = indices.size(0)
    a.bound_m = bound_m.data_ptr() if bound_m is not None else None
    return a


def _current_stream(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def _dispatch(
    fptr: int,
    out_expert_num_tokens: torch.Tensor,
    out_expert_x: torch.Tensor,
    out_expert_x_scale: torch.Tensor | None,
    dp_x: torch.Tensor,
    dp_x_scale: torch.Tensor | None,
    indices: torch.Tensor,
    bound_m: torch.Tensor | None,
    do_send: bool,
    do_recv: bool,
) -> None:
    lib = load_library()
    world = _handle_world.get(fptr)
    if world is None:
        raise RuntimeError("pplx_kernels: invalid state: the handle has been destroyed")
    args = pack_dispatch_args(
        world.experts_per_token, out_expert_num_tokens, out_expert_x, out_expert_x_scale, dp_x,
        dp_x_scale, indices, bound_m,
    )  # fmt: skip
    mode = split_mode(do_send, do_recv)
    if mode != SPLIT_NONE:
        reserve_split(world, 0)
    # The library selects the world's device for the launch and restores the caller's; the
    # stream is the current one of the tensors' device (csrc/bindings/all_to_all_ops.cpp:163,194).
    check_status(lib.pplx_a2a_dispatch(fptr, ctypes.byref(args), mode, _current_stream(indices)))
    world.hold(
        f"dispatch{mode}",
        fptr,
        (out_expert_num_tokens, out_expert_x, out_expert_x_scale, dp_x, dp_x_scale, indices, bound_m),
    )


def _combine(
    fptr: int,
    out_tokens: torch.Tensor,
    indices: torch.Tensor,
    weights: torch.Tensor,
    expert_y: torch.Tensor,
    bound_m: torch.Tensor | None,
    do_send: bool,
    do_recv: bool,
) -> None:
    lib = load_library()
    world = _handle_world.get(fptr)
    if world is None:
        raise RuntimeError("pplx_kernels: invalid state: the handle has been destroyed")
    args = pack_combine_args(out_tokens, indices, weights, expert_y, bound_m)
    mode = split_mode(do_send, do_recv)
    if mode != SPLIT_NONE:
        reserve_split(world, expert_y.element_size())
    check_status(lib.pplx_a2a_combine(fptr, ctypes.byref(args), mode, _current_stream(indices)))
    world.hold(f"combine{mode}", fptr, (out_tokens, indices, weights, expert_y, bound_m))


def _fake_dispatch(*args, **kwargs) -> None:
    """Meta kernel: traces as a no-op (csrc/bindings/all_to_all_ops.cpp:198-209)."""


def _fake_combine(*args, **kwargs) -> None:
    """Meta kernel: traces as a no-op (csrc/bindings/all_to_all_ops.cpp:313-322)."""


# ---------------------------------------------------------------------------
# torch.ops.pplx_kernels registration (csrc/bindings/all_to_all_ops.cpp:329-391)
# ---------------------------------------------------------------------------
_CREATE_ARGS = (
    "int max_num_tokens, int num_experts, int experts_per_token, int rank, int world_size, "
    "int dp_size, int hidden_dim, int hidden_dim_bytes, int hidden_dim_scale_bytes"
)
_DISPATCH_SCHEMA = (
    "(int fptr, Tensor! out_expert_num_tokens, Tensor! out_expert_x, Tensor!? out_expert_x_scale, "
    "Tensor dp_x, Tensor? dp_x_scale, Tensor indices, Tensor? bound_m, bool do_send, bool do_recv) -> ()"
)
_COMBINE_SCHEMA = (
    "(int fptr, Tensor! out_tokens, Tensor indices, Tensor weights, Tensor expert_y, "
    "Tensor? bound_m, bool do_send, bool do_recv) -> ()"
)

_torch_lib = torch.library.Library("pplx_kernels", "DEF")
_torch_lib.define("all_to_all_destroy(int fptr) -> ()")
_torch_lib.impl("all_to_all_destroy", _destroy, "CompositeExplicitAutograd")
_torch_lib.define(f"all_to_all_intranode_create({_CREATE_ARGS}, str group_name) -> int")
_torch_lib.impl("all_to_all_intranode_create", _create_intranode, "CompositeExplicitAutograd")
_torch_lib.define(f"all_to_all_internode_create({_CREATE_ARGS}) -> int")
_torch_lib.impl("all_to_all_internode_create", _create_internode, "CompositeExplicitAutograd")
for _transport in ("intranode", "internode"):
    _torch_lib.define(f"all_to_all_{_transport}_dispatch{_DISPATCH_SCHEMA}")
    _torch_lib.impl(f"all_to_all_{_transport}_dispatch", _dispatch, "CUDA")
    _torch_lib.impl(f"all_to_all_{_transport}_dispatch", _fake_dispatch, "Meta")
    _torch_lib.define(f"all_to_all_{_transport}_combine{_COMBINE_SCHEMA}")
    _torch_lib.impl(f"all_to_all_{_transport}_combine", _combine, "CUDA")
    _torch_lib.impl(f"all_to_all_{_transport}_combine", _fake_combine, "Meta")

_ops = torch.ops.pplx_kernels
