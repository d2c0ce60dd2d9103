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
