from .build import BuildError, build_all, build_module, load_module
from .hip import GatedLinearWeights, HipKernels, KernelError, LinearWeights

__all__ = [
    "BuildError",
    "GatedLinearWeights",
    "HipKernels",
    "KernelError",
    "LinearWeights",
    "build_all",
    "build_module",
    "load_module",
]
