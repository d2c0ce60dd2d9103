"""Structural guarantees of the shipped package: no CPU fallback, no use of the checker."""
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "commbench_amd")


def _package_sources():
    for base, _, files in os.walk(PKG):
        for name in files:
            if name.endswith((".py", ".hip", ".h", ".hpp", ".cpp")):
                yield os.path.join(base, name)
    for name in os.listdir(os.path.join(ROOT, "include")):
        yield os.path.join(ROOT, "include", name)


def test_package_never_touches_the_checker():
    for path in _package_sources():
        text = open(path).read()
        assert not re.search(r"\boracle\b|ep_oracle", text), f"{path} refers to the CPU checker"


def test_missing_library_is_an_error_not_a_fallback(monkeypatch):
    from commbench_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", os.path.join(PKG, "no_such_library.so"))
    with pytest.raises(ImportError, match="no CPU fallback"):
        _lib.load()


def test_hip_sources_are_gfx950_only():
    """No CUDA/HIP dual paths, no hipify leftovers, no Triton."""
    for path in _package_sources():
        text = open(path).read()
        assert "__HIP_PLATFORM_AMD__" not in text and "__CUDACC__" not in text, path
        assert "cuda_runtime" not in text and "triton" not in text.lower(), path


def test_bench_refuses_more_than_one_gpu():
    """The benchmark measures one GPU; asking for more exits with a message, before any GPU work."""
    import subprocess
    import sys
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"],
                          capture_output=True, text=True, timeout=120)
    assert proc.returncode == 2
    assert "one GPU only" in proc.stderr and proc.stdout.strip() == ""


def test_host_twins_stay_out_of_the_device_entry_points():
    """Only ep_host.hip may allocate or copy; the device entry points enqueue and return."""
    for name in ("ep_abi.hip", "ep_layout.hip", "ep_permute.hip", "ep_combine.hip"):
        text = open(os.path.join(PKG, "csrc", name)).read()
        text = re.sub(r"//.*", "", text)
        assert "hipMalloc" not in text and "hipFree" not in text and "hipMemset" not in text, name
