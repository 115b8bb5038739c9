"""TreeLogicLayer: one level of pairwise logic gates over the last dimension.
Interface of the reference's src/convlogic/treelogic_layer.py."""
import torch
from torch import nn
from torch.autograd import Function

from ..difflogic.functional import GradFactor, bin_op_s
from ..difflogic.packbitstensor import PackBitsTensor
from ..hip import convlogic_hip


class TreeLogicFunction(Function):
    """x [N,C,H,W,2*Xo], w_prob [C,Xo,16] -> [N,C,H,W,Xo] (src/convlogic/treelogic_layer.py:15-30)."""

    @staticmethod
    def forward(ctx, x, w_prob):
        x = x.contiguous()
        w_prob = w_prob.contiguous()
        ctx.save_for_backward(x, w_prob)
        return convlogic_hip.treelogic_forward(x, w_prob)

    @staticmethod
    def backward(ctx, grad_y):
        grad_y = grad_y.contiguous()
        x, w_prob = ctx.saved_tensors
        grad_x = convlogic_hip.treelogic_backward_x(grad_y, x, w_prob) if ctx.needs_input_grad[0] else None
        grad_w = convlogic_hip.treelogic_backward_weight(grad_y, x) if ctx.needs_input_grad[1] else None
        return grad_x, grad_w


def gate_probabilities(logits, training, dtype):
    """softmax while training, one-hot of the arg-max gate in eval
    (src/convlogic/treelogic_layer.py:102-106, src/convlogic/convlogic_layer.py:321-325)."""
    if training:
        return torch.nn.functional.softmax(logits, dim=-1)
    return torch.nn.functional.one_hot(logits.argmax(-1), num_classes=16).to(dtype=dtype)


class TreeLogicLayer(nn.Module):
    """input_bits values per (n, c, y, x) are combined pairwise, (0,1), (2,3), ..., by input_bits/2
    learned gates per channel (src/convlogic/treelogic_layer.py:33-81)."""

    def __init__(self, channels: int, input_bits: int, residual_init: bool = False, implementation: str = "cuda",
                 grad_factor: float = 1.0):
        super().__init__()
        assert input_bits % 2 == 0, "input_bits must be even"
        self.channels, self.input_bits = channels, input_bits
        self.implementation, self.grad_factor = implementation, grad_factor
        if residual_init:
            logits = torch.zeros(channels, input_bits // 2, 16)
            logits[..., 3] = 5.0
        else:
            logits = torch.randn(channels, input_bits // 2, 16)
        self.weights = nn.Parameter(logits)

    def forward(self, x):
        assert x.shape[-1] == self.input_bits, (
            f"Expected input last dimension to be {self.input_bits}, but got {x.shape[-1]}")
        x = x.contiguous()
        if self.grad_factor != 1.0 and not isinstance(x, PackBitsTensor):
            x = GradFactor.apply(x, self.grad_factor)
        if self.implementation == "cuda":
            return self.forward_cuda(x)
        if self.implementation == "python":
            return self.forward_python(x)
        raise ValueError(f"Unknown implementation {self.implementation!r}")

    def forward_cuda(self, x):
        # the kernels read the probabilities in x's element type (the bindings reject any other)
        w_prob = gate_probabilities(self.weights, self.training, x.dtype).to(x.dtype).contiguous()
        return TreeLogicFunction.apply(x, w_prob)

    def forward_python(self, x):
        c, gates = x.shape[1], x.shape[-1] // 2
        w_prob = gate_probabilities(self.weights, self.training, x.dtype).view(1, c, 1, 1, gates, 16)
        return bin_op_s(x[..., 0::2], x[..., 1::2], w_prob)

    def extra_repr(self):
        return f"channels={self.channels}, input_bits={self.input_bits}"
