from .binarize import apply_thresholds, compute_thresholds, distributive_thresholds, pack_thresholds, uniform_thresholds
from .convlogic_layer import ConvLogicFunction, ConvLogicLayer, FullConvLogicFunction, PoolLogicLayer
from .model import ConvLogicCifarModel, ConvLogicMnistModel
from .treelogic_layer import TreeLogicFunction, TreeLogicLayer

__all__ = ["ConvLogicLayer", "ConvLogicFunction", "FullConvLogicFunction", "PoolLogicLayer", "TreeLogicLayer",
           "TreeLogicFunction", "ConvLogicCifarModel", "ConvLogicMnistModel", "apply_thresholds",
           "compute_thresholds", "distributive_thresholds", "pack_thresholds", "uniform_thresholds"]
