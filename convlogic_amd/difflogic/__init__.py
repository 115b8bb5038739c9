from .compiled_model import CompiledLogicNet
from .difflogic import GroupSum, LogicLayer, LogicLayerCudaFunction
from .functional import GradFactor, bin_op, bin_op_s, get_unique_connections
from .packbitstensor import PackBitsTensor

__all__ = ["LogicLayer", "GroupSum", "LogicLayerCudaFunction", "PackBitsTensor", "GradFactor", "bin_op", "bin_op_s",
           "get_unique_connections", "CompiledLogicNet"]
