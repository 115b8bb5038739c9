"""Native-module equivalents: `difflogic_hip` and `convlogic_hip` expose the function sets of the
reference's `difflogic_cuda` and `convlogic_cuda` extension modules on top of the C ABI."""
from . import _lib, convlogic_hip, difflogic_hip
from .graph import GraphedStep

__all__ = ["_lib", "difflogic_hip", "convlogic_hip", "GraphedStep"]
