"""Loads the native libraries of the package and exposes their entry points.

Two shared objects sit next to this file (built by ``make -C pplx-kernels_amd/csrc``):

* ``_C.so`` -- the torch operator layer (``csrc/torch_ops.cpp``), the counterpart of the
  reference's ``csrc/bindings/all_to_all_ops.cpp`` + ``bindings.cpp``.  Importing it registers
  ``torch.ops.pplx_kernels.all_to_all_{intranode,internode}_{create,dispatch,combine}`` and
  ``all_to_all_destroy`` with the reference's schemas (``all_to_all_ops.cpp:329-391``), as the
  reference's loader does with ``torch.ops.load_library`` (``src/pplx_kernels/ops.py:8-16``);
  its module functions ``_C.dispatch`` / ``_C.combine`` are the same code without the op
  dispatcher, which ``AllToAll`` uses for eager calls.
* ``libpplx_kernels.so`` -- the C ABI of ``include/pplx_a2a.h`` (kernels + host layer, no
  torch types), which ``_C.so`` links against and which ``LoopbackWorld`` and the tests also
  reach through ``ctypes``.

A missing or unloadable library is an ``ImportError``: there is no fallback implementation.
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
    "pplx_a2a_world_of",
    "pplx_a2a_dispatch",
    "pplx_a2a_combine",
    "pplx_a2a_world_dispatch",
    "pplx_a2a_world_combine",
    "pplx_a2a_static_step",
    "pplx_a2a_world_recorded_calls",
    "pplx_a2a_world_abandon_step",
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
        lib.pplx_a2a_world_of.argtypes = [vp]
        lib.pplx_a2a_world_of.restype = vp
        lib.pplx_a2a_world_recorded_calls.argtypes = [vp, i32, i32, ctypes.POINTER(u32)]
        lib.pplx_a2a_world_abandon_step.argtypes = [vp, u32, ctypes.POINTER(u32)]
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
# The torch operator layer
# ---------------------------------------------------------------------------
_BINDING_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "_C.so")
try:
    from . import _C  # noqa: E402  (registers torch.ops.pplx_kernels)
except ImportError as exc:
    raise ImportError(
        f"cannot load {_BINDING_PATH} ({exc}): build it with `make -C pplx-kernels_amd/csrc` "
        "(or __graft_entry__.build()); there is no fallback implementation"
    ) from exc

_ops = torch.ops.pplx_kernels
# Interpreter exit: release every world while Python and the HIP runtime are still up;
# AllToAll.__del__ finds nothing left to do afterwards.
atexit.register(_C.destroy_all)

ABANDON_DISPATCH, ABANDON_COMBINE = 1, 2


class WorldRef:
    """The world a rank handle is attached to: ``ptr`` is its ``pplx_a2a_world_t *``."""

    def __init__(self, fptr: int) -> None:
        self.fptr = fptr
        self.ptr = _C.world_ptr(fptr)


def world_of(fptr: int) -> WorldRef:
    return WorldRef(fptr)


def reserve_split(world: WorldRef, expert_y_elem_bytes: int) -> None:
    """Split send / recv calls go through staging that the library never allocates inside
    dispatch / combine.  The reference's callers do not know of it, so the operator layer
    reserves it the first time a rank splits a dispatch (``expert_y_elem_bytes`` 0) or a combine
    (non-zero); like any allocation this synchronises and cannot happen under stream capture:
    run one eager step before capturing split calls, or call this up front.  What has been
    reserved never moves."""
    _C.reserve_split(world.fptr, expert_y_elem_bytes)


def abandon_step(fptr: int, which: int = ABANDON_DISPATCH | ABANDON_COMBINE) -> int:
    """Drops the calls recorded for the step being assembled in the world of ``fptr`` (and the
    tensors kept alive for them); returns how many calls were dropped.  The operator layer does
    this by itself when a rank's arguments are refused after other ranks have called."""
    return _C.abandon_step(fptr, which)


def is_live(fptr: int) -> bool:
    return _C.is_live(fptr)


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
