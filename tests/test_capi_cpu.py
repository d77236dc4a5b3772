"""CPU-only checks of the drop-in boundary: the C-ABI library loads, exports every symbol
that ``include/pplx_a2a.h`` declares, validates configurations without a GPU, and the
Python binding layer raises the reference's errors before anything reaches the device.
No compute call is made here."""

from __future__ import annotations

import ctypes
import os
import re

import pytest
import torch

from pplx_kernels import AllToAll, ops

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "pplx_a2a.h")


def declared_symbols() -> list[str]:
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(pplx_a2a_[a-z_0-9]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = ops.load_library()
    names = declared_symbols()
    assert len(names) >= 23
    for name in names:
        assert hasattr(lib, name), f"{name} is declared in include/pplx_a2a.h but not exported"
    assert sorted(ops.EXPORTED_SYMBOLS) == names
    assert re.fullmatch(rb"\d+\.\d+\.\d+", lib.pplx_a2a_version())


def test_library_is_built_from_the_sources_in_the_tree():
    """The library reports a hash of the sources it was built from; a kernel edit without a
    rebuild (tests load what is built, they do not build) shows up here."""
    import glob
    import hashlib

    csrc = os.path.join(ROOT, "pplx-kernels_amd", "csrc")
    files = sorted(
        os.path.basename(p)
        for pat in ("*.hip", "a2a_*.h", "a2a_capi.cpp")
        for p in glob.glob(os.path.join(csrc, pat))
    )
    h = hashlib.sha256()
    for name in files:
        h.update(open(os.path.join(csrc, name), "rb").read())
    h.update(open(HEADER, "rb").read())
    assert ops.load_library().pplx_a2a_build_id().decode() == h.hexdigest()[:16], (
        "libpplx_kernels.so is stale: run `make -C pplx-kernels_amd/csrc`"
    )


def test_operator_layer_is_built_from_the_sources_in_the_tree():
    import hashlib

    h = hashlib.sha256()
    h.update(open(os.path.join(ROOT, "pplx-kernels_amd", "csrc", "torch_ops.cpp"), "rb").read())
    h.update(open(HEADER, "rb").read())
    assert ops._C.build_id() == h.hexdigest()[:16], "pplx_kernels/_C.so is stale: run `make -C pplx-kernels_amd/csrc`"


def test_ctypes_structs_match_the_header_layout():
    # 8-byte fields throughout, except the trailing (u32 m) and the i32 dtypes, which pad to 8.
    assert ctypes.sizeof(ops.Config) == 56
    assert ctypes.sizeof(ops.DispatchArgs) == 18 * 8
    assert ctypes.sizeof(ops.CombineArgs) == 12 * 8
    assert ops.DispatchArgs.bound_m.offset == 17 * 8
    assert ops.CombineArgs.in_dtype.offset == 10 * 8 and ops.CombineArgs.m.offset == 10 * 8 + 4


def _create(cfg: tuple) -> tuple[int, str]:
    lib = ops.load_library()
    c = ops.Config(*cfg)
    out = ctypes.c_void_p()
    st = lib.pplx_a2a_world_create(ctypes.byref(c), 0, ctypes.byref(out))
    return st, lib.pplx_a2a_last_error().decode()


# (max_num_tokens, num_experts, experts_per_token, world_size, dp_size, hidden_dim, bytes, scale bytes)
GOOD = (128, 256, 8, 8, 1, 7168, 7168, 224)


@pytest.mark.parametrize(
    "field,value,message",
    [
        (6, 7160, "invalid hidden dim bytes"),  # not a multiple of 16 (all_to_all.cpp:32)
        (7, 220, "invalid hidden dim scale bytes"),  # (all_to_all.cpp:33)
        (7, 7168 + 16, "invalid hidden dim bytes"),  # scale bytes > row bytes (all_to_all.cpp:39)
        (4, 3, "multiple of dp_size"),
        (1, 100, "multiple of world_size"),
        (2, 0, "experts_per_token"),
        (2, 65, "experts_per_token"),
        (0, 0, "max_num_tokens"),
        (3, 0, "world_size"),
    ],
)
def test_world_create_rejects_bad_configs(field, value, message):
    cfg = list(GOOD)
    cfg[field] = value
    st, err = _create(tuple(cfg))
    assert st == 1, (st, err)
    assert message in err


def test_world_create_needs_a_gpu_for_good_configs():
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    st, err = _create(GOOD)
    assert st == 3 and "hip" in err.lower()  # HIP error, not a silent fallback
    with pytest.raises(RuntimeError, match="HIP error"):
        AllToAll.intranode(128, 256, 8, 0, 8, 1, 7168, 7168, 224)


def test_null_arguments_are_status_codes_not_crashes():
    lib = ops.load_library()
    assert lib.pplx_a2a_world_create(None, 0, None) == 1
    assert lib.pplx_a2a_create(None, 0, None) == 1
    assert lib.pplx_a2a_dispatch(None, None, 0, None) == 1
    assert lib.pplx_a2a_combine(None, None, 0, None) == 1
    assert lib.pplx_a2a_world_dispatch(None, None, None) == 1
    assert lib.pplx_a2a_world_faults(None, None, None) == 1
    assert lib.pplx_a2a_world_reserve_split(None, 2) == 1
    assert lib.pplx_a2a_world_abandon_step(None, 3, None) == 1
    assert lib.pplx_a2a_world_recorded_calls(None, 0, 0, None) == 1
    assert lib.pplx_a2a_world_of(None) is None
    assert lib.pplx_a2a_graph_launch(None, None) == 1
    assert lib.pplx_a2a_destroy(None) == 0 and lib.pplx_a2a_world_destroy(None) == 0
    assert lib.pplx_a2a_graph_destroy(None) == 0


def test_binding_checks_fire_before_the_device():
    """The tensor checks of csrc/bindings/all_to_all_ops.cpp:135-161,249-259 run on CPU tensors."""
    n, k, h = 4, 2, 64
    i32 = torch.zeros(2, dtype=torch.int32)
    x3 = torch.zeros(2, 8, h, dtype=torch.bfloat16)
    x2 = torch.zeros(n, h, dtype=torch.bfloat16)
    idx = torch.zeros(n, k, dtype=torch.uint32)
    with pytest.raises(RuntimeError, match="Tensor outExpertNumTokens must be on GPU"):
        ops.pack_dispatch_args(k, i32, x3, None, x2, None, idx, None)
    with pytest.raises(RuntimeError, match="Tensor outTokens must be on GPU"):
        ops.pack_combine_args(x2, idx, torch.zeros(n, k), x3, None)
    with pytest.raises(RuntimeError, match="Invalid split mode"):
        ops.split_mode(False, False)
    assert (ops.split_mode(True, True), ops.split_mode(True, False), ops.split_mode(False, True)) == (0, 1, 2)


def test_operator_layer_checks_fire_before_the_device():
    """The same checks in the compiled operator layer (pplx_kernels._C), which the per-rank
    API goes through: CPU tensors are refused with the reference's messages, wrong Python types
    are TypeErrors, and a CPU tensor handed to the registered op finds no kernel."""
    C = ops._C
    n, k, h = 4, 2, 64
    i32 = torch.zeros(2, dtype=torch.int32)
    x3 = torch.zeros(2, 8, h, dtype=torch.bfloat16)
    x2 = torch.zeros(n, h, dtype=torch.bfloat16)
    idx = torch.zeros(n, k, dtype=torch.uint32)
    with pytest.raises(RuntimeError, match="Tensor outExpertNumTokens must be on GPU"):
        C.dispatch(0, i32, x3, None, x2, None, idx, None, True, True)
    with pytest.raises(RuntimeError, match="Tensor outTokens must be on GPU"):
        C.combine(0, x2, idx, torch.zeros(n, k), x3, None, True, True)
    with pytest.raises(TypeError, match="dp_x must be a Tensor, not NoneType"):
        C.dispatch(0, i32, x3, None, None, None, idx, None, True, True)
    with pytest.raises(TypeError, match="takes 10 positional arguments but 3 were given"):
        C.dispatch(0, i32, x3)
    with pytest.raises(TypeError, match="fptr must be an int"):
        C.combine("0", x2, idx, torch.zeros(n, k), x3, None, True, True)
    with pytest.raises(NotImplementedError):
        torch.ops.pplx_kernels.all_to_all_intranode_dispatch(0, i32, x3, None, x2, None, idx, None, True, True)
    with pytest.raises(RuntimeError, match="unknown all-to-all handle"):
        torch.ops.pplx_kernels.all_to_all_destroy(12345)
    with pytest.raises(RuntimeError, match="the handle has been destroyed"):
        C.world_ptr(12345)
    assert C.is_live(12345) is False
    with pytest.raises(RuntimeError, match="negative rank"):
        torch.ops.pplx_kernels.all_to_all_intranode_create(8, 8, 2, -1, 4, 1, 64, 128, 0, "g")
    with pytest.raises(RuntimeError, match="negative or zero size"):
        torch.ops.pplx_kernels.all_to_all_internode_create(8, 8, 2, 0, 0, 1, 64, 128, 0)


def test_op_schemas_match_the_reference():
    """csrc/bindings/all_to_all_ops.cpp:329-391: names, mutability and argument order."""
    for transport in ("intranode", "internode"):
        d = getattr(torch.ops.pplx_kernels, f"all_to_all_{transport}_dispatch").default._schema
        assert [a.name for a in d.arguments] == [
            "fptr", "out_expert_num_tokens", "out_expert_x", "out_expert_x_scale", "dp_x",
            "dp_x_scale", "indices", "bound_m", "do_send", "do_recv",
        ]  # fmt: skip
        assert [a.name for a in d.arguments if a.alias_info and a.alias_info.is_write] == [
            "out_expert_num_tokens", "out_expert_x", "out_expert_x_scale",
        ]  # fmt: skip
        c = getattr(torch.ops.pplx_kernels, f"all_to_all_{transport}_combine").default._schema
        assert [a.name for a in c.arguments] == [
            "fptr", "out_tokens", "indices", "weights", "expert_y", "bound_m", "do_send", "do_recv",
        ]  # fmt: skip
        assert [a.name for a in c.arguments if a.alias_info and a.alias_info.is_write] == ["out_tokens"]
    assert hasattr(torch.ops.pplx_kernels, "all_to_all_destroy")
    assert hasattr(torch.ops.pplx_kernels, "all_to_all_intranode_create")
    assert hasattr(torch.ops.pplx_kernels, "all_to_all_internode_create")


def test_meta_kernels_are_no_ops():
    """Fake implementations let torch.compile trace the ops (all_to_all_ops.cpp:198-209,313-322)."""
    m = lambda *s, dt=torch.bfloat16: torch.empty(*s, dtype=dt, device="meta")  # noqa: E731
    torch.ops.pplx_kernels.all_to_all_intranode_dispatch(
        0, m(2, dt=torch.int32), m(2, 8, 64), None, m(4, 64), None, m(4, 2, dt=torch.uint32), None, True, True
    )
    torch.ops.pplx_kernels.all_to_all_intranode_combine(
        0, m(4, 64), m(4, 2, dt=torch.uint32), m(4, 2, dt=torch.float32), m(2, 8, 64), None, True, True
    )


def _gpu_kernels_of(path: str) -> list[dict]:
    """Kernel metadata (AMDGPU code-object notes, msgpack) of every gfx code object embedded in
    a host shared library."""
    import struct

    import msgpack

    data = open(path, "rb").read()
    kernels: list[dict] = []
    pos = data.find(b"\x7fELF")
    while pos >= 0:
        if data[pos + 4] == 2 and struct.unpack_from("<H", data, pos + 18)[0] == 224:  # ELF64, EM_AMDGPU
            (e_shoff,) = struct.unpack_from("<Q", data, pos + 0x28)
            e_shentsize, e_shnum = struct.unpack_from("<HH", data, pos + 0x3A)
            for i in range(e_shnum):
                sh = pos + e_shoff + i * e_shentsize
                (sh_type,) = struct.unpack_from("<I", data, sh + 4)
                sh_offset, sh_size = struct.unpack_from("<QQ", data, sh + 0x18)
                if sh_type != 7:  # SHT_NOTE
                    continue
                p, end = pos + sh_offset, pos + sh_offset + sh_size
                while p < end:
                    namesz, descsz, ntype = struct.unpack_from("<III", data, p)
                    p += 12
                    name = data[p : p + namesz]
                    p += (namesz + 3) & ~3
                    desc = data[p : p + descsz]
                    p += (descsz + 3) & ~3
                    if ntype == 32 and name.startswith(b"AMDGPU"):  # NT_AMDGPU_METADATA
                        meta = msgpack.unpackb(desc, raw=False, strict_map_key=False)
                        kernels += meta.get("amdhsa.kernels", [])
        pos = data.find(b"\x7fELF", pos + 4)
    return kernels


def test_no_kernel_spills_or_uses_scratch():
    """A kernel that spills registers needs scratch memory: its launch is several microseconds
    slower and its spill traffic competes with the rows.  Every kernel of the library has to fit
    its registers (this caught the 14- and 16-register row variants of the one-launch dispatch
    under a 1024-thread workgroup)."""
    kernels = _gpu_kernels_of(ops._LIB_PATH)
    assert len(kernels) > 100
    assert {k[".name"].split("ILi")[0] for k in kernels}  # names parsed
    offenders = [
        (k[".name"], k[".private_segment_fixed_size"], k.get(".vgpr_spill_count", 0), k.get(".sgpr_spill_count", 0))
        for k in kernels
        if k[".private_segment_fixed_size"] or k.get(".vgpr_spill_count", 0) or k.get(".sgpr_spill_count", 0)
    ]
    assert not offenders, offenders


def test_bench_refuses_more_than_one_gpu():
    """Every simulated rank shares one GPU's HBM: `bench.py --gpus N` with N above 1 (or under a
    launcher that sets WORLD_SIZE) exits with a message that says so, before it touches a GPU."""
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ)
    env.pop("WORLD_SIZE", None)
    for argv, extra in ((["--gpus", "2"], {}), ([], {"WORLD_SIZE": "8"})):
        done = subprocess.run(
            [sys.executable, os.path.join(root, "bench.py"), *argv],
            env={**env, **extra}, capture_output=True, text=True, timeout=120,
        )  # fmt: skip
        assert done.returncode == 2, done
        assert "single-GPU loopback" in done.stderr and "--gpus 1" in done.stderr
        assert done.stdout == ""
