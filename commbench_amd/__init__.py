"""MI355X-native MoE dispatch layout / permute / combine behind a C ABI (include/mi_ep.h)."""
from . import workloads  # noqa: F401

__all__ = ["ops", "workloads", "build"]
