"""Network topologies of the reference's src/convlogic/model.py as plain nn.Modules: the caller side of
the logic-layer kernels.  Constructor arguments, layer order and the `network` attribute are the
reference's, so parameters are drawn in the same RNG order and state_dict keys (`network.<i>.weights`,
`network.<i>.selection`, `network.<i>.indices_0`, ...) match checkpoints written from there (the
Lightning wrapper of src/convlogic/model.py:111-200 prefixes them with `model.`)."""
import weakref

import torch
from torch import nn

from ..difflogic import GroupSum, LogicLayer
from ..difflogic.difflogic import logic_layer_group_sum
from .convlogic_layer import ConvLogicLayer


# per network: (dtype, device), the layers that take a fold made ahead, and the bookkeeping of that launch (kept outside the
# module so that copies and pickles of a network carry no host pointers)
_FOLD_PLANS = weakref.WeakKeyDictionary()


_PREFOLD_MIN_ELEMS = 20 << 19                                     # 512 Ki rows of logits


def _prefold(owner, network, x, mode=True):
    """Folds the logits of all layers of a training step in ONE launch and leaves each layer its (probabilities,
    coefficients): softmax and fold are then no part of the layers' forward launches -- the LogicLayers run their plain
    streaming kernel, the deep blocks skip their set-up launch.  Same values as the per-layer folds (tested)."""
    from ..hip import difflogic_hip
    cache = _FOLD_PLANS.get(owner)
    if cache is not None and cache[0] == (x.dtype, x.device):
        _, picked, plan = cache
        weights = [m._parameters["weights"] for m in picked]
        if plan is None:                                             # nothing to fold when the cache was made: look again
            cache = None
        elif not (plan.matches(weights) and all(m.prefold_candidate() is w for m, w in zip(picked, weights))):
            cache = None
    if cache is None:
        layers = [m for m in network if isinstance(m, (ConvLogicLayer, LogicLayer))]
        picked = [m for m in layers for w in [m.prefold_candidate()] if w is not None and w.dtype == x.dtype and w.device == x.device]
        picked = picked[:difflogic_hip.FOLD_MANY_MAX]
        weights = [m._parameters["weights"] for m in picked]
        plan = difflogic_hip.FoldPlan([w.detach() for w in weights]) if len(picked) >= 2 else None
        _FOLD_PLANS[owner] = ((x.dtype, x.device), picked, plan)
    if plan is None:
        return
    # An eager step of a small network is bound by the host, where the bookkeeping of this launch costs more than the
    # layers' own allocations save (C5: +15 us per step): by default only networks whose step the GPU bounds fold ahead;
    # prefold = "always" is for small networks whose step is replayed from a HIP graph (C5: 0.385 -> 0.379 ms).
    if mode != "always" and plan.total < _PREFOLD_MIN_ELEMS:
        return
    for m, (probs, folded) in zip(picked, difflogic_hip.fold_many([w.detach() for w in weights], plan)):
        m.set_prefold(probs, folded)


def _forward(owner, x):
    """The network on x.  In training on the GPU two things happen that a plain nn.Sequential call would not do: the
    logits of all layers are folded in one launch where that pays (`prefold`), and the last LogicLayer and the GroupSum
    behind it run as one autograd node (`fused_tail`, default on), whose backward needs no GroupSum launch."""
    net = owner.network
    if not (owner.training and isinstance(x, torch.Tensor) and x.is_cuda and torch.is_grad_enabled()):
        return net(x)
    mode = owner.__dict__.get("prefold", True)                       # True: where it pays, "always", False
    if mode:
        _prefold(owner, net, x, mode)
    n = len(net)
    if (owner.__dict__.get("fused_tail", True) and n >= 2 and isinstance(net[n - 2], LogicLayer) and isinstance(net[n - 1], GroupSum)
            and not (net._forward_hooks or net._forward_pre_hooks)):
        h = x
        for i, m in enumerate(net):
            if i == n - 2:
                break
            h = m(h)
        return logic_layer_group_sum(net[n - 2], net[n - 1], h)
    return net(x)


def _block(c_in, c_out, implementation, **kw):
    return ConvLogicLayer(in_channels=c_in, out_channels=c_out, residual_init=True, complete=True,
                          implementation=implementation, **kw)


def _head(dims, tau, implementation):
    fc = [LogicLayer(a, b, grad_factor=1, residual_init=True, implementation=implementation) for a, b in zip(dims, dims[1:])]
    return [nn.Flatten(), *fc, GroupSum(k=10, tau=tau)]


class ConvLogicCifarModel(nn.Module):
    """Four 3x3 / padding 1 blocks of k, 4k, 16k, 32k kernels (each halves the image), then three
    LogicLayers of 10, 5 and 2.5 times the flattened width (doubled from k = 1024) and a 10-class
    GroupSum (src/convlogic/model.py:11-60)."""

    def __init__(self, k_param=32, input_channels=3, input_size=32, tau=20, implementation="cuda"):
        super().__init__()
        self.input_size = input_size
        self.k_param = k_param
        self.extra_layers = 2 if k_param >= 1024 else 1
        widths = [input_channels] + [m * k_param for m in (1, 4, 16, 32)]
        blocks = [_block(a, b, implementation, padding=1, groups=1) for a, b in zip(widths, widths[1:])]
        side = input_size // 2 ** len(blocks)
        flat = widths[-1] * side * side
        m = self.extra_layers
        dims = [flat, m * flat * 10, m * flat * 5, m * (flat * 10) // 4]
        # the last block feeds nn.Flatten and a LogicLayer, which reads feature-major memory: when the block's kernels
        # can write that layout (4x4 images on the GPU) its output is the [N, C, 2, 2] view of a [C, 2, 2, N] tensor
        blocks[-1].feature_major_output = implementation == "cuda"
        # the network's input is the thresholded image (src/convlogic/data.py:46-50): every element is 0 or 1
        blocks[0].binary_input = implementation == "cuda"
        self.network = nn.Sequential(*blocks, *_head(dims, tau, implementation))

    def forward(self, x):
        return _forward(self, x)


class ConvLogicMnistModel(nn.Module):
    """A 5x5 / padding 0 block of k kernels (28 -> 24 -> 12), two 3x3 / padding 1 blocks of 3k and 9k
    kernels (-> 6 -> 3), then LogicLayers 81k -> 1280k -> 640k -> 320k and a 10-class GroupSum
    (src/convlogic/model.py:63-108)."""

    def __init__(self, input_channels=1, input_size=28, k_param=32, tau=6.5, implementation="cuda"):
        super().__init__()
        k = k_param
        blocks = [_block(input_channels, k, implementation, kernel=5, padding=0),
                  _block(k, 3 * k, implementation, kernel=3, padding=1),
                  _block(3 * k, 9 * k, implementation, kernel=3, padding=1)]
        blocks[0].binary_input = implementation == "cuda"          # binarised digits, as in the CIFAR topology
        self.network = nn.Sequential(*blocks, *_head([81 * k, 1280 * k, 640 * k, 320 * k], tau, implementation))

    def forward(self, x):
        return _forward(self, x)
