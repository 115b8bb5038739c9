"""convlogic_amd: MI355X (gfx950) implementation of the logic-layer hot path of convolutional
differentiable logic gate networks.

  convlogic_amd.difflogic   LogicLayer, GroupSum, PackBitsTensor, ...   (mirror of the `difflogic` package)
  convlogic_amd.convlogic   ConvLogicLayer, TreeLogicLayer, PoolLogicLayer, model topologies (mirror of `convlogic`)
  convlogic_amd.hip         function sets of the native extension modules, on the C ABI of
                            include/convlogic_amd.h (libconvlogic_amd.so); GraphedStep: HIP-graph replay of a training step
"""
from .convlogic import (ConvLogicCifarModel, ConvLogicFunction, ConvLogicLayer, ConvLogicMnistModel, FullConvLogicFunction, PoolLogicLayer, TreeLogicFunction,
                        TreeLogicLayer)
from .difflogic import GradFactor, GroupSum, LogicLayer, LogicLayerCudaFunction, PackBitsTensor
from .hip import GraphedStep

__all__ = ["ConvLogicLayer", "ConvLogicFunction", "FullConvLogicFunction", "PoolLogicLayer", "TreeLogicLayer",
           "TreeLogicFunction", "LogicLayer", "GroupSum", "LogicLayerCudaFunction", "PackBitsTensor", "GradFactor", "ConvLogicCifarModel",
           "ConvLogicMnistModel", "GraphedStep"]
