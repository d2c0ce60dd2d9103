"""The run-time compilation plug-in (commbench_amd/jit.py): sources built with fixed shapes, with and
without an overlaid source file; everything here runs without a GPU (compilation and argument checks)."""
import os
import shutil

from commbench_amd import _lib, jit
from commbench_amd import build as hip_build

SHAPES = dict(num_topk=8, num_experts=256, num_ranks=8, row_bytes=14336, hidden=7168)   # target, c2, c3


def test_fixed_shape_library_exports_the_abi_and_refuses_other_shapes():
    jit.init_jit()
    path = jit.compile_library(**SHAPES)
    assert os.path.exists(path) and path == jit.library_path(**SHAPES)
    assert jit.compile_library(**SHAPES) == path                      # second call: from the cache
    lib = jit.load_library(**SHAPES)
    for name in _lib.SIGNATURES:
        assert hasattr(lib, name), name
    assert lib.mi_ep_abi_version() == _lib.load().mi_ep_abi_version()
    # the fixed shapes pass the argument checks, any other is refused before a device is touched
    assert lib.mi_ep_workspace_bytes(8192, 8, 256, 8) == _lib.load().mi_ep_workspace_bytes(8192, 8, 256, 8)
    assert lib.mi_ep_workspace_bytes(8192, 4, 256, 8) == 0            # top-4
    assert lib.mi_ep_workspace_bytes(8192, 8, 128, 8) == 0            # 128 experts
    assert lib.mi_ep_workspace_bytes(8192, 8, 256, 4) == 0            # 4 ranks
    assert lib.mi_ep_get_dispatch_layout(None, None, None, None, None, 0, 2, 8, 256, None) == -22
    combine = lambda lib_, hidden: lib_.mi_ep_combine(None, 0, None, None, None, None, None, None, 0, 8, hidden,
                                                      None, None, None, 0, None)
    assert combine(lib, 7168) == 0 and combine(lib, 4096) == -22 and combine(_lib.load(), 4096) == 0
    dispatch = lambda lib_, row_bytes, experts: lib_.mi_ep_dispatch(
        None, None, None, None, None, None, None, None, 0, 8, experts, 1, row_bytes, 0, None, None, None, None,
        None, None, 0, 0, None)
    assert dispatch(lib, 14336, 256) == dispatch(_lib.load(), 14336, 256)     # same verdict on its own shape
    assert dispatch(lib, 8192, 256) == -22 and dispatch(lib, 14336, 128) == -22
    # partial fixing: only what was named is constant
    assert jit.library_path(num_topk=8) != jit.library_path(**SHAPES) != jit.library_path()


def test_overlay_file_stands_in_for_the_shipped_source(tmp_path):
    """A file of the overlay folder named like a shipped source replaces it (the reference overlays
    one header of its include tree): here a copy of ep_abi.hip with another error text."""
    src = os.path.join(hip_build.CSRC_DIR, "ep_abi.hip")
    text = open(src).read()
    assert 'return "workspace too small";' in text
    (tmp_path / "ep_abi.hip").write_text(text.replace('return "workspace too small";', 'return "overlaid text";'))
    cache = tmp_path / "cache"
    try:
        jit.init_jit(overlay_root=str(tmp_path), cache_dir=str(cache))
        assert jit.source_files()["ep_abi.hip"] == str(tmp_path / "ep_abi.hip")
        assert jit.source_files()["ep_layout.hip"] == os.path.join(hip_build.CSRC_DIR, "ep_layout.hip")
        lib = jit.load_library(num_topk=2)
        assert lib.mi_ep_strerror(-28) == b"overlaid text"
        assert _lib.load().mi_ep_strerror(-28) == b"workspace too small"
        assert lib.mi_ep_workspace_bytes(256, 2, 8, 2) > 0 and lib.mi_ep_workspace_bytes(256, 3, 8, 2) == 0
    finally:
        jit.init_jit()
        shutil.rmtree(cache, ignore_errors=True)
