"""MI355X-native ring-attention forward engine (gfx950 HIP kernels behind a C ABI)."""
from .configs import WORKLOADS, Workload  # noqa: F401

__all__ = ["WORKLOADS", "Workload"]
