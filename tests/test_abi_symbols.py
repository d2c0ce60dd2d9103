"""The C-ABI library loads without a GPU and exports exactly what include/mi_ep.h declares."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "mi_ep.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mi_ep_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_surface():
    names = declared_functions()
    for required in ("mi_ep_get_dispatch_layout", "mi_ep_dispatch_layout", "mi_ep_dispatch",
                     "mi_ep_combine", "mi_ep_workspace_bytes", "mi_ep_workspace_init"):
        assert required in names


def test_library_exports_every_declared_symbol():
    from commbench_amd import _lib
    assert os.path.exists(_lib.LIB_PATH), "build with `python -m commbench_amd.build`"
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared_functions():
        assert hasattr(lib, name), f"{name} declared in mi_ep.h but not exported"
    assert sorted(_lib.SIGNATURES) == declared_functions()


def test_ctypes_signatures_match_the_header_argument_by_argument():
    """Every parameter of every declaration is bound with the matching ctypes kind."""
    import ctypes
    from commbench_amd import _lib
    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    seen = 0
    for m in re.finditer(r"\b(mi_ep_[a-z0-9_]+)\s*\(([^)]*)\)\s*;", text):
        name, params = m.group(1), m.group(2).strip()
        restype, argtypes = _lib.SIGNATURES[name]
        plist = [] if params in ("void", "") else [p.strip() for p in params.split(",")]
        assert len(plist) == len(argtypes), name
        for p, t in zip(plist, argtypes):
            if "*" in p:
                assert t in (ctypes.c_void_p, ctypes.POINTER(ctypes.c_int)), (name, p)
            elif p.startswith("size_t"):
                assert t is ctypes.c_size_t, (name, p)
            elif p.startswith("long long"):
                assert t is ctypes.c_longlong, (name, p)
            elif p.startswith("unsigned int"):
                assert t is ctypes.c_uint, (name, p)
            else:
                assert p.startswith("int ") and t is ctypes.c_int, (name, p)
        seen += 1
    assert seen == len(_lib.SIGNATURES)


def test_host_only_entry_points():
    """Calls that touch no device: version, error strings, workspace sizing, argument checks."""
    from commbench_amd import _lib
    lib = _lib.load()
    assert lib.mi_ep_abi_version() == 3
    assert _lib.strerror(0) == "ok"
    assert _lib.strerror(-22) == "invalid argument"
    assert _lib.strerror(-28) == "workspace too small"
    # 256-byte header + ceil(T/256) tiles x (E + R) 8-byte status words
    assert lib.mi_ep_workspace_bytes(8192, 8, 256, 8) == 256 + 32 * 264 * 8
    assert lib.mi_ep_workspace_bytes(1, 1, 1, 1) == 256 + 1 * 2 * 8
    # one 16-byte entry per route slot of every 256-token tile
    assert lib.mi_ep_route_order_bytes(8192, 8) == 32 * 256 * 8 * 16
    assert lib.mi_ep_route_order_bytes(257, 3) == 2 * 256 * 3 * 16
    assert lib.mi_ep_route_order_bytes(0, 8) == 0
    assert _lib.strerror(-7).startswith("shape exceeds the static scratch")
    # destination order (4): long rows, enough tiles for all eight dies, long enough runs per expert,
    # and only on a device with eight dies of at least 4 MiB L2 each; token order (2) otherwise
    BY_TOKEN, BY_DESTINATION, DIES, L2 = 2, 4, 8, 4 << 20
    assert lib.mi_ep_dispatch_schedule_for(8192, 8, 256, 14336, DIES, L2) == BY_DESTINATION
    assert lib.mi_ep_dispatch_schedule_for(4096, 8, 256, 14336, DIES, L2) == BY_DESTINATION
    assert lib.mi_ep_dispatch_schedule_for(16384, 8, 128, 8192, DIES, L2) == BY_DESTINATION
    assert lib.mi_ep_dispatch_schedule_for(8192, 8, 256, 2048, DIES, L2) == BY_TOKEN      # 2 KiB rows
    assert lib.mi_ep_dispatch_schedule_for(1024, 8, 256, 14336, DIES, L2) == BY_TOKEN     # 4 tiles for 8 dies
    assert lib.mi_ep_dispatch_schedule_for(8192, 2, 1024, 14336, DIES, L2) == BY_TOKEN    # half a row per tile and expert
    assert lib.mi_ep_dispatch_schedule_for(8192, 8, 256, 16384, DIES, L2) == BY_TOKEN     # a tile's rows exceed L2
    assert lib.mi_ep_dispatch_schedule_for(8192, 8, 256, 14336, 1, L2) == BY_TOKEN        # one die (another partition mode)
    assert lib.mi_ep_dispatch_schedule_for(8192, 8, 256, 14336, DIES, 2 << 20) == BY_TOKEN  # smaller L2
    assert lib.mi_ep_dispatch_schedule_for(8192, 8, 256, 14336, 0, 0) == BY_TOKEN         # traits unknown
    assert lib.mi_ep_dispatch_schedule_for(8192, 8, 256, 100, DIES, L2) == -22
    # the per-rank format, the pull form and the host twins check their arguments before any launch
    assert lib.mi_ep_dispatch_ranks(None, None, None, None, None, 0, None, None, 4, 2, 3, 8, 32, 0, 0, 0,
                                    None, None, None, None, None, None, None, None, 0, None) == -22   # 8 % 3
    assert lib.mi_ep_dispatch_ranks(None, None, None, None, None, 0, None, None, 4, 2, 2, 8, 24, 0, 0, 0,
                                    None, None, None, None, None, None, None, None, 0, None) == -22   # 24 % 16
    assert lib.mi_ep_combine_rank_weights(None, None, None, 4, 9, 0, None, None, None) == -22        # 9 slots
    assert lib.mi_ep_combine_rank_weights(None, None, None, 4, 2, 0, None, None, None) == -22        # nothing asked for
    assert lib.mi_ep_dispatch_ranks_strided_scales(None, None, 1, 1, None, None, None, 0, None, None, 4, 2, 3, 8, 32,
                                                   0, 0, 0, None, None, 1, 1, None, None, None, None, None, None,
                                                   0, None) == -22                                  # 8 % 3
    assert lib.mi_ep_dispatch_cached(None, None, None, 4, 4, 24, 0, None, None, None, 0, None) == -22
    assert lib.mi_ep_dispatch(None, None, None, None, None, None, None, None, 4, 2, 8, 1, 32, 0,
                              None, None, None, None, None, None, 0, 8, None) == -22   # null tables (and an unknown flag)
    assert lib.mi_ep_host_dispatch_layout(None, 4, 2, 2, 8, 0, 0, None, None, None, None, None, None, None, None,
                                          None, 0, None, None, None, None) == -22       # alignment 0
    assert lib.mi_ep_host_get_dispatch_layout(None, None, None, None, None, 4, 2, 2, 8) == -22
    assert lib.mi_ep_host_dispatch(None, None, None, None, 4, 2, 2, 8, 1, 24, 0, None, None, None, None,
                                   None, None, None, None, None, None, 0) == -22
    assert lib.mi_ep_host_combine(None, 0, None, None, None, None, 4, 2, 12, None) == -22
    assert lib.mi_ep_host_dispatch_ranks(None, None, None, None, 4, 2, 2, 8, 24, 0, 0, 0, None, None, None,
                                         None, None, None, None, None, None, 0) == -22       # 24 % 16, no psum
    assert lib.mi_ep_host_dispatch_cached(None, None, None, 4, 4, 24, 0, None, None) == -22
    assert lib.mi_ep_workspace_bytes(8192, 8, 256, 9) == 0       # more than 8 ranks
    assert lib.mi_ep_workspace_bytes(8192, 9, 256, 8) == 0       # more than 8 slots
    assert lib.mi_ep_workspace_bytes(8192, 8, 250, 8) == 0       # experts not divisible by ranks
    # Argument errors are reported before any launch.
    assert lib.mi_ep_get_dispatch_layout(None, None, None, None, None, 4, 2, 9, 18, None) == -22
    assert lib.mi_ep_get_dispatch_layout(None, None, None, None, None, 4, 9, 2, 8, None) == -22
    assert lib.mi_ep_get_dispatch_layout(None, None, None, None, None, 4, 2, 3, 8, None) == -22
    assert lib.mi_ep_dispatch_layout(None, 4, 2, 2, 8, 0, 0, None, None, None, None, None, None, None,
                                     None, None, 0, None, None, None, None, None, 0, None) == -22     # alignment 0
    assert lib.mi_ep_dispatch_layout_static(None, 4, 2, 2, 8, 0, 0, None, None, None, None, None, None, None,
                                            None, None, 0, None, None, None, None, None, None) == -22  # alignment 0
    assert lib.mi_ep_dispatch_layout_static(None, 1 << 20, 2, 8, 1024, 1, 0, None, None, None, None, None, None, None,
                                            None, None, 0, None, None, None, None, None, None) == -7   # beyond the scratch
    assert lib.mi_ep_workspace_set_wait_limit(None, 1, None) == -22
    assert lib.mi_ep_combine(None, 0, None, None, None, None, None, None, 4, 2, 12, None, None, None, 0, None) == -22
    assert lib.mi_ep_combine(None, 0, None, None, None, None, None, None, 1 << 28, 8, 16, None, None, None,
                             0, None) == -22                                           # T * K beyond 2^30
    assert lib.mi_ep_combine(None, 0, None, None, None, None, None, None, 0, 2, 16, None, None, None,
                             2, None) == -22                                           # unknown flag
    assert lib.mi_ep_dispatch(None, None, None, None, None, None, None, None, 4, 2, 8, 1, 24, 0,
                              None, None, None, None, None, None, 0, 0, None) == -22   # 24 % 16 != 0


def test_python_surface_rejects_bad_arguments_like_the_reference():
    """Same conditions and wording as the reference's constructor checks (example042 .cu:96-107)."""
    import torch
    from commbench_amd import ops
    topk = torch.zeros((4, 2), dtype=torch.int64)
    with pytest.raises(ValueError, match="GPU"):
        ops.get_dispatch_layout(topk, 8, 2)
    with pytest.raises(ValueError, match=r"num_ranks must be in \[1, 8\]"):
        ops.Buffer(16, 2, 18, 9, device="cpu")
    with pytest.raises(ValueError, match=r"num_topk must be in \[1, 8\]"):
        ops.Buffer(16, 9, 16, 8, device="cpu")
    with pytest.raises(ValueError, match="divisible"):
        ops.Buffer(16, 2, 10, 4, device="cpu")


def test_header_is_plain_c_and_cxx(tmp_path):
    """include/mi_ep.h must be consumable from C (the FFI boundary) and from C++."""
    import subprocess
    c_src = tmp_path / "use.c"
    c_src.write_text('#include "mi_ep.h"\nint main(void) { return mi_ep_abi_version() == MI_EP_ABI_VERSION ? 0 : 1; }\n')
    inc = os.path.join(ROOT, "include")
    libdir = os.path.join(ROOT, "commbench_amd")
    exe = tmp_path / "use_c"
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-pedantic", f"-I{inc}", str(c_src), "-o", str(exe),
                    f"-L{libdir}", "-lmi_ep", f"-Wl,-rpath,{libdir}", "-Wl,-rpath,/opt/rocm/lib"], check=True)
    assert subprocess.run([str(exe)]).returncode == 0
    cxx_src = tmp_path / "use.cc"
    cxx_src.write_text('#include "mi_ep.h"\nint main() { return mi_ep_workspace_bytes(256, 8, 256, 8) == 256 + 264 * 8 ? 0 : 1; }\n')
    exe2 = tmp_path / "use_cxx"
    subprocess.run(["g++", "-std=c++17", "-Wall", "-Werror", f"-I{inc}", str(cxx_src), "-o", str(exe2),
                    f"-L{libdir}", "-lmi_ep", f"-Wl,-rpath,{libdir}", "-Wl,-rpath,/opt/rocm/lib"], check=True)
    assert subprocess.run([str(exe2)]).returncode == 0
