from .convlogic_layer import ConvLogicFunction, ConvLogicLayer, FullConvLogicFunction, PoolLogicLayer
from .treelogic_layer import TreeLogicFunction, TreeLogicLayer

__all__ = ["ConvLogicLayer", "ConvLogicFunction", "FullConvLogicFunction", "PoolLogicLayer", "TreeLogicLayer",
           "TreeLogicFunction"]
