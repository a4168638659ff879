"""Native kernels: building, loading and calling them."""
from .library import KernelBuildError, build_all, load_hip_module, load_host_library

__all__ = ["KernelBuildError", "build_all", "load_hip_module", "load_host_library"]
