"""LogicLayer / GroupSum with the constructor arguments, parameter and buffer names of the
reference's src/difflogic/difflogic.py, on HIP kernels for gfx950.

implementation="cuda" runs the HIP kernels (on ROCm builds of torch the device type is still
"cuda") and raises if the GPU or the compiled library is missing.  implementation="python" is the
reference's second, explicitly selected backend: plain torch ops on whatever device the tensors
live on.
"""
import numpy as np
import torch

from ..hip import difflogic_hip
from .functional import GradFactor, bin_op_s, get_unique_connections
from .packbitstensor import PackBitsTensor


def _reverse_wiring(idx0, idx1, in_dim):
    """CSR map input -> neurons reading it; neuron y is listed under idx0[y] before idx1[y] and
    neurons appear in increasing order inside every list (same layout as the python loop of
    src/difflogic/difflogic.py:71-87)."""
    out_dim = len(idx0)
    target = np.stack([idx0, idx1], axis=1).reshape(-1)                 # [y0.a, y0.b, y1.a, ...]
    neuron = np.repeat(np.arange(out_dim, dtype=np.int64), 2)
    order = np.argsort(target, kind="stable")
    start = np.zeros(in_dim + 1, dtype=np.int64)
    np.cumsum(np.bincount(target, minlength=in_dim), out=start[1:])
    return torch.from_numpy(start), torch.from_numpy(neuron[order].copy())


class LogicLayer(torch.nn.Module):
    """out_dim two-input logic gate neurons over in_dim features (src/difflogic/difflogic.py:14-90)."""

    def __init__(self, in_dim: int, out_dim: int, grad_factor: float = 1.0, implementation: str = None,
                 connections: str = "random", residual_init: bool = False):
        super().__init__()
        if residual_init:                       # gate 3 ("A") gets logit 5 -> p = 0.908
            logits = torch.zeros(out_dim, 16)
            logits[:, 3] = 5.0
        else:
            logits = torch.randn(out_dim, 16)
        self.weights = torch.nn.Parameter(logits)
        self.in_dim, self.out_dim, self.grad_factor = in_dim, out_dim, grad_factor

        if implementation is None:
            implementation = "cuda" if torch.cuda.is_available() else "python"
        assert implementation in ["cuda", "python"], f"Invalid implementation: {implementation}"
        self.implementation = implementation

        self.connections = connections
        assert self.connections in ["random", "unique"], self.connections
        a, b = self.get_connections(self.connections)
        self.register_buffer("indices_0", a.to(torch.int64))
        self.register_buffer("indices_1", b.to(torch.int64))

        if self.implementation == "cuda":
            start, flat = _reverse_wiring(self.indices_0.cpu().numpy(), self.indices_1.cpu().numpy(), in_dim)
            self.register_buffer("given_x_indices_of_y_start", start)
            self.register_buffer("given_x_indices_of_y", flat)
            self._reverse_built = (self.indices_0._version, self.indices_1._version)

        self.num_neurons = out_dim
        self.num_weights = out_dim

    def forward(self, x):
        if isinstance(x, PackBitsTensor):
            assert not self.training, "PackBitsTensor is not supported for the differentiable training mode."
            assert x.is_cuda, (f"PackBitsTensor is only supported for CUDA, but got device {x.device}. "
                               "If you want fast inference on CPU, please use CompiledDiffLogicModel.")
        elif self.grad_factor != 1.0:
            x = GradFactor.apply(x, self.grad_factor)

        if self.implementation == "cuda":
            if isinstance(x, PackBitsTensor):
                return self.forward_cuda_eval(x)
            return self.forward_cuda(x)
        if self.implementation == "python":
            return self.forward_python(x)
        raise ValueError(f"Unsupported implementation: {self.implementation}")

    def _gate_weights(self, dtype):
        if self.training:
            return torch.nn.functional.softmax(self.weights, dim=-1).to(dtype)
        return torch.nn.functional.one_hot(self.weights.argmax(-1), 16).to(dtype)

    def forward_python(self, x):
        assert x.shape[-1] == self.in_dim, (x.shape[-1], self.in_dim)
        a, b = x[..., self.indices_0], x[..., self.indices_1]
        w = self._gate_weights(torch.float32 if not self.training else self.weights.dtype)
        return bin_op_s(a, b, w)

    def forward_cuda(self, x):
        if self.training:
            assert x.is_cuda, f"x must be a CUDA tensor, got device: {x.device}"
        assert x.ndim == 2, x.ndim
        assert x.shape[1] == self.in_dim, (tuple(x.shape[::-1]), self.in_dim)
        key = self._wiring_key()
        self._check_wiring(key)
        weights, buffers = self._parameters["weights"], self._buffers
        if (self.training and weights.dtype == x.dtype and x.dtype in (torch.float32, torch.float64)
                and weights.is_contiguous() and weights.device == x.device):
            # a sample-major batch is transposed inside the Function (and its gradient on the way back): one autograd
            # node per layer instead of two
            prefolded = self._take_prefold(weights)
            inside = prefolded is None and _transposes_with_kernel(x)
            return _LogicLayerLogitsFunction.apply(x if inside else _feature_major(x), buffers["indices_0"], buffers["indices_1"],
                                                   weights, buffers["given_x_indices_of_y_start"],
                                                   buffers["given_x_indices_of_y"], self._sole_consumers(key), inside,
                                                   prefolded).transpose(0, 1)
        xt = _feature_major(x)
        w = self._gate_weights(xt.dtype)
        args = (xt, self.indices_0, self.indices_1, w, self.given_x_indices_of_y_start, self.given_x_indices_of_y)
        if self.training:
            return LogicLayerCudaFunction.apply(*args).transpose(0, 1)
        with torch.no_grad():
            return LogicLayerCudaFunction.apply(*args).transpose(0, 1)

    def prefold_candidate(self):
        """The logits a network may fold for this layer ahead of its forward call (one launch for all its layers,
        difflogic_hip.fold_many), or None when the layer's training path does not take the result."""
        w = self._parameters["weights"]
        if (self.implementation == "cuda" and self.training and w.is_cuda and w.is_contiguous()
                and w.dtype in (torch.float32, torch.float64)):
            return w
        return None

    def set_prefold(self, probs, folded):
        w = self._parameters["weights"]
        self.__dict__["_prefold"] = (w._version, w.data_ptr(), probs, folded)

    def _take_prefold(self, weights):
        """The pair left by set_prefold() if it was made from the weights as they are now (it is used once)."""
        pf = self.__dict__.pop("_prefold", None)
        if pf is not None and pf[0] == weights._version and pf[1] == weights.data_ptr() and pf[2].dtype == weights.dtype:
            return pf[2], pf[3]
        return None

    def forward_cuda_eval(self, x: PackBitsTensor):
        """Replaces x.t by the layer output (src/difflogic/difflogic.py:149-164)."""
        assert not self.training
        assert isinstance(x, PackBitsTensor)
        assert x.t.shape[0] == self.in_dim, (x.t.shape, self.in_dim)
        # gate ids = arg-max of the logits, taken on every call as the reference does (src/difflogic/difflogic.py:161): no
        # cache that an in-place update of `weights.data` (EMA swaps, legacy optimisers) could leave stale.  Where the row
        # layout allows, the evaluation kernel takes the arg-max itself and the call is one launch.
        x.t = difflogic_hip.eval_planned_logits(x.t, self.indices_0, self.indices_1, self.weights.detach(), self._eval_plan())
        return x

    def _wiring_key(self):
        # (buffers and parameters straight from their dicts: nn.Module.__getattr__ costs a microsecond per lookup, and
        # this key is taken on every call)
        a, b = self._buffers["indices_0"], self._buffers["indices_1"]
        return (a._version, b._version, a.data_ptr(), b.data_ptr(), self._parameters["weights"].device)

    def _check_wiring(self, key=None):
        """The kernels index x with indices_0 / indices_1 without bounds checks: an index outside [0, in_dim) must
        raise here instead of faulting the GPU.  Checked on the first launch and again whenever the buffers were
        modified in place (version counter) or replaced; writes through `.data` bypass the counter -- call
        invalidate() after those."""
        key = key or self._wiring_key()
        if self.__dict__.get("_wiring_checked") != key:
            for name, idx in (("indices_0", self.indices_0), ("indices_1", self.indices_1)):
                if idx.dtype != torch.int64 or tuple(idx.shape) != (self.out_dim,):
                    raise ValueError(f"{name} must be int64 [{self.out_dim}], got {idx.dtype} {tuple(idx.shape)}")
                if idx.numel() and (int(idx.min()) < 0 or int(idx.max()) >= self.in_dim):
                    raise ValueError(f"{name} holds an input index outside [0, {self.in_dim})")
            if self.implementation == "cuda":                        # the reverse map of the input gradient
                for name, n in (("given_x_indices_of_y_start", self.in_dim + 1), ("given_x_indices_of_y", 2 * self.out_dim)):
                    t = getattr(self, name)
                    if t.dtype != torch.int64 or tuple(t.shape) != (n,) or t.device != self.indices_0.device or not t.is_contiguous():
                        raise ValueError(f"{name} must be a contiguous int64 [{n}] on the device of the wiring")
                if not (self.indices_0.is_contiguous() and self.indices_1.is_contiguous()
                        and self.indices_0.device == self.indices_1.device == self.weights.device):
                    raise ValueError("indices_0 / indices_1 must be contiguous and on the device of the weights")
                # The reverse map belongs to the wiring it was built from: after an in-place rewiring or a state_dict
                # that replaced the indices it is rebuilt here (into the same buffers), so the input gradient never walks
                # the lists of an older wiring.  (The reference builds it once, src/difflogic/difflogic.py:71-87.)
                built = (self.indices_0._version, self.indices_1._version)
                if self.__dict__.get("_reverse_built") != built:
                    start, flat = _reverse_wiring(self.indices_0.cpu().numpy(), self.indices_1.cpu().numpy(), self.in_dim)
                    with torch.no_grad():
                        self.given_x_indices_of_y_start.copy_(start)
                        self.given_x_indices_of_y.copy_(flat)
                    self._reverse_built = built
            self._wiring_checked = key

    def invalidate(self):
        """Drops everything derived from the wiring buffers (range check, consumer analysis, packed walk plan, reverse map).  Needed only after writing indices_0 / indices_1 through `.data`, which the version
        counters do not see."""
        self._wiring_checked = self._sole_cache = self._plan_cache = self._reverse_built = None

    def _load_from_state_dict(self, *args, **kwargs):
        super()._load_from_state_dict(*args, **kwargs)
        self.invalidate()

    def _sole_consumers(self, key=None):
        """True when every input feature is read by exactly one neuron operand (the halving layers of the
        reference's models, 2*out_dim == in_dim): both gradients then come from one kernel.  Rechecked when the
        wiring buffers were modified in place or moved."""
        if 2 * self.out_dim != self.in_dim:
            return False
        key = key or self._wiring_key()
        cached = self.__dict__.get("_sole_cache")
        if cached is None or cached[0] != key:
            uses = torch.bincount(torch.cat([self.indices_0, self.indices_1]), minlength=self.in_dim)
            cached = (key, bool((uses == 1).all().item()))
            self._sole_cache = cached
        return cached[1]

    def _eval_plan(self):
        """Walk order of the wiring graph for the packed evaluation kernel; rebuilt when the wiring
        buffers were modified in place or moved to another device."""
        self._check_wiring()
        key = self._wiring_key()
        cached = getattr(self, "_plan_cache", None)
        if cached is None or cached[0] != key:
            cached = (key, difflogic_hip.eval_plan(self.indices_0, self.indices_1, self.in_dim))
            self._plan_cache = cached
        return cached[1]

    def extra_repr(self):
        return "{}, {}, {}".format(self.in_dim, self.out_dim, "train" if self.training else "eval")

    def get_connections(self, connections):
        assert self.out_dim * 2 >= self.in_dim, (
            f"The number of neurons ({self.out_dim}) must not be smaller than half of the "
            f"number of inputs ({self.in_dim}) because otherwise not all inputs could be "
            "used or considered.")
        if connections == "random":
            # every input is used floor/ceil(2*out/in) times (src/difflogic/difflogic.py:175-181)
            slots = torch.randperm(2 * self.out_dim) % self.in_dim
            slots = torch.randperm(self.in_dim)[slots].reshape(2, self.out_dim)
            return slots[0].to(torch.int64), slots[1].to(torch.int64)
        if connections == "unique":
            return get_unique_connections(self.in_dim, self.out_dim)
        raise ValueError(connections)


class _FeatureMajor(torch.autograd.Function):
    """[batch, features] -> contiguous [features, batch] through the tiled HIP transpose, and the same for the
    gradient on the way back: whoever receives it (a leaf's .grad, Flatten, a conv block) wants it contiguous, and
    a transposed view would be copied there by a generic strided kernel."""

    @staticmethod
    def forward(ctx, x):
        return difflogic_hip.transpose(x)

    @staticmethod
    def backward(ctx, grad):
        if grad.is_cuda and grad.is_contiguous() and grad.element_size() in (1, 2, 4, 8):
            return difflogic_hip.transpose(grad)
        return grad.transpose(0, 1)


def _transposes_with_kernel(x):
    """True for a dense sample-major device tensor whose feature-major copy the tiled HIP transpose makes (a
    transposed view of a feature-major tensor needs no copy at all)."""
    return (x.is_cuda and x.dim() == 2 and x.is_contiguous() and not x.transpose(0, 1).is_contiguous()
            and x.element_size() in (1, 2, 4, 8))


def _feature_major(x):
    """[batch, features] -> contiguous [features, batch].  A transposed view of a feature-major
    tensor (what the previous LogicLayer returned) is used as is, without a copy."""
    xt = x.transpose(0, 1)
    if xt.is_contiguous():
        return xt
    if _transposes_with_kernel(x):
        return _FeatureMajor.apply(x)
    return xt.contiguous()


class GroupSum(torch.nn.Module):
    """Sums k groups of outputs and divides by tau; packed inputs give raw integer counts
    (src/difflogic/difflogic.py:188-211)."""

    def __init__(self, k: int, tau: float = 1.0):
        super().__init__()
        self.k, self.tau = k, tau

    def forward(self, x):
        if isinstance(x, PackBitsTensor):
            return x.group_sum(self.k)
        assert x.shape[-1] % self.k == 0, (x.shape, self.k)
        if (x.is_cuda and x.dim() == 2 and x.dtype in (torch.float32, torch.float64) and x.numel() > 0
                and x.transpose(0, 1).is_contiguous() and not x.is_contiguous()):
            # the transposed view of a feature-major tensor, as a LogicLayer returns it: summed in that layout
            return _GroupSumFeatureMajor.apply(x, self.k, self.tau)
        return x.reshape(*x.shape[:-1], self.k, x.shape[-1] // self.k).sum(-1) / self.tau

    def extra_repr(self):
        return f"k={self.k}, tau={self.tau}"


class _GroupSumFeatureMajor(torch.autograd.Function):
    """Per-class sums / tau of x [batch, features] that is a transposed view of a contiguous [features, batch]
    tensor; the gradient comes back in the same layout (a transposed view again, no copies).  The division by
    tau happens inside the two kernels (as a product with 1 / tau, which is what torch computes for `sum / tau` on the
    device)."""

    @staticmethod
    def forward(ctx, x, k, tau):
        ctx.features, ctx.tau = x.shape[1], tau
        return difflogic_hip.group_sum(x.transpose(0, 1), k, tau)

    @staticmethod
    def backward(ctx, grad_out):
        return difflogic_hip.group_sum_backward(grad_out.contiguous(), ctx.features, ctx.tau).transpose(0, 1), None, None


class LogicLayerCudaFunction(torch.autograd.Function):
    """y[out,B] = layer(x[in,B]); gradients w.r.t. x and the gate probabilities w
    (src/difflogic/difflogic.py:214-230)."""

    @staticmethod
    def forward(ctx, x, a, b, w, given_x_indices_of_y_start, given_x_indices_of_y):
        ctx.save_for_backward(x, a, b, w, given_x_indices_of_y_start, given_x_indices_of_y)
        return difflogic_hip.forward(x, a, b, w)

    @staticmethod
    def backward(ctx, grad_y):
        x, a, b, w, start, flat = ctx.saved_tensors
        grad_y = grad_y if grad_y.is_contiguous() else _contiguous_2d(grad_y)
        grad_x = grad_w = None
        if ctx.needs_input_grad[0]:
            grad_x = difflogic_hip.backward_x(x, a, b, w, grad_y, start, flat)
        if ctx.needs_input_grad[3]:
            grad_w = difflogic_hip.backward_w(x, a, b, grad_y)
        return grad_x, None, None, grad_w, None, None, None


# One walk over the consumer lists gives both gradients whenever a row of the batch fits one pass of a wavefront
# (backward_fused_fits): C1 16 -> 12 us, first LogicLayer of the k=32 CIFAR net 41 -> 30 us, 131072 -> 1.31 M neurons
# x 128 samples 1554 -> 1131 us against the input-gradient and weight-gradient kernels run one after the other.


class _LogicLayerLogitsFunction(torch.autograd.Function):
    """Training path of the module: y[out,B] as a function of the LOGITS; the softmax runs inside forward and
    its backward is fused into the weight-gradient kernel (same values as softmax + LogicLayerCudaFunction up
    to rounding)."""

    @staticmethod
    def forward(ctx, x, a, b, logits, given_x_indices_of_y_start, given_x_indices_of_y, sole_consumers=False,
                sample_major_input=False, prefolded=None):
        if prefolded is not None:                                    # (probs, folded) of these logits, made by the network for all
            w, folded = prefolded                                    # its layers in one launch: the forward is the plain streaming kernel
            y = difflogic_hip.forward_folded(x, a, b, folded)
        elif sample_major_input:                                     # x is [B, in]: its gradient goes back in that layout
            y, w, folded, x = difflogic_hip.forward_logits(x, a, b, logits.detach(), validate=False, sample_major_x=True)
        else:
            y, w, folded = difflogic_hip.forward_logits(x, a, b, logits.detach(), validate=False)   # the module has checked its buffers
        ctx.save_for_backward(x, a, b, w, folded, given_x_indices_of_y_start, given_x_indices_of_y)
        ctx.sole_consumers = sole_consumers
        ctx.sample_major_input = sample_major_input
        return y

    @staticmethod
    def backward(ctx, grad_y):
        x, a, b, w, folded, start, flat = ctx.saved_tensors
        fused = (not ctx.sole_consumers and ctx.needs_input_grad[0] and ctx.needs_input_grad[3]
                 and difflogic_hip.backward_fused_fits(x))
        if fused and not grad_y.is_contiguous() and grad_y.is_cuda and grad_y.dim() == 2 and grad_y.transpose(0, 1).is_contiguous():
            # the gradient of a [B, out] consumer arrives as a transposed view: its feature-major copy is made by the call
            # that computes both gradients
            gy_sm = grad_y.transpose(0, 1)
            grad_x, grad_l = difflogic_hip.backward_fused(x, a, b, folded, w, gy_sm, start, flat, validate=_needs_check(gy_sm, x),
                                                          sample_major_grad_x=ctx.sample_major_input, sample_major_grad_y=True)
            return grad_x, None, None, grad_l, None, None, None, None, None
        grad_y = grad_y if grad_y.is_contiguous() else _contiguous_2d(grad_y)
        grad_x = grad_l = None
        if ctx.sole_consumers and ctx.needs_input_grad[0] and ctx.needs_input_grad[3]:
            grad_x, grad_l = difflogic_hip.backward_sole(x, a, b, folded, w, grad_y, validate=_needs_check(grad_y, x))
        elif fused:
            # (a sample-major input takes its gradient sample-major straight from the kernel)
            grad_x, grad_l = difflogic_hip.backward_fused(x, a, b, folded, w, grad_y, start, flat, validate=_needs_check(grad_y, x),
                                                          sample_major_grad_x=ctx.sample_major_input)
            return grad_x, None, None, grad_l, None, None, None, None, None
        else:
            if ctx.needs_input_grad[0]:
                grad_x = difflogic_hip.backward_x_folded(x, a, b, folded, grad_y, start, flat, validate=_needs_check(grad_y, x))
            if ctx.needs_input_grad[3]:
                grad_l = difflogic_hip.backward_logits(x, a, b, w, grad_y, validate=_needs_check(grad_y, x))
        if ctx.sample_major_input and grad_x is not None:
            grad_x = difflogic_hip.transpose(grad_x)
        return grad_x, None, None, grad_l, None, None, None, None, None


class _LogicLayerGroupSumFunction(torch.autograd.Function):
    """A halving LogicLayer and the GroupSum behind it (the last two modules of the reference's networks,
    src/convlogic/model.py:55-57) as ONE autograd node: the forward is the two forward launches of the modules; the
    backward hands the gradient of the GroupSum's output [B, k] to the layer's one-pass kernel, which forms the gradient of
    its own output from it -- no launch that writes that [features, B] tensor and none that reads it back.  Same values
    as the two modules, bit for bit."""

    @staticmethod
    def forward(ctx, x, a, b, logits, k, tau, prefolded=None):
        if prefolded is not None:
            w, folded = prefolded
            y = difflogic_hip.forward_folded(x, a, b, folded)
        else:
            y, w, folded = difflogic_hip.forward_logits(x, a, b, logits.detach(), validate=False)
        ctx.save_for_backward(x, a, b, w, folded)
        ctx.k, ctx.tau = k, tau
        return difflogic_hip.group_sum(y, k, tau)

    @staticmethod
    def backward(ctx, grad_out):
        x, a, b, w, folded = ctx.saved_tensors
        grad_out = grad_out.contiguous()
        grad_x, grad_l = difflogic_hip.backward_sole_classes(x, a, b, folded, w, grad_out, ctx.k, ctx.tau,
                                                            validate=_needs_check(grad_out, x))
        return grad_x, None, None, grad_l, None, None, None


def logic_layer_group_sum(layer, group_sum, x):
    """group_sum(layer(x)) -- through one autograd node (_LogicLayerGroupSumFunction) when `layer` is a halving
    LogicLayer in training mode on the GPU, else through the two modules."""
    weights = layer._parameters["weights"]
    if (isinstance(layer, LogicLayer) and isinstance(group_sum, GroupSum) and layer.implementation == "cuda" and layer.training
            and torch.is_grad_enabled() and isinstance(x, torch.Tensor) and x.is_cuda and x.ndim == 2 and x.shape[1] == layer.in_dim
            and layer.grad_factor == 1.0 and weights.dtype == x.dtype and x.dtype in (torch.float32, torch.float64)
            and weights.is_contiguous() and weights.device == x.device and layer.out_dim % group_sum.k == 0 and x.shape[0] > 0
            and group_sum.tau != 0 and not _has_forward_hooks(layer) and not _has_forward_hooks(group_sum)):
        key = layer._wiring_key()
        layer._check_wiring(key)
        if layer._sole_consumers(key):
            buffers = layer._buffers
            return _LogicLayerGroupSumFunction.apply(_feature_major(x), buffers["indices_0"], buffers["indices_1"], weights,
                                                     group_sum.k, group_sum.tau, layer._take_prefold(weights))
    return group_sum(layer(x))


def _has_forward_hooks(module):
    """Hooks that only a call of the module itself would run."""
    return bool(module._forward_hooks or module._forward_pre_hooks)


def _needs_check(grad_y, x):
    """The tensors a Function saved were validated on the way in; the incoming gradient is what can still differ
    (autograd hands over the output's shape, but a caller-made gradient may have another dtype or device)."""
    return grad_y.dtype != x.dtype or grad_y.device != x.device


def _contiguous_2d(t):
    tt = t.transpose(0, 1)
    if t.is_cuda and t.dim() == 2 and tt.is_contiguous():
        return difflogic_hip.transpose(tt)      # t is a transposed view: one tiled transpose
    return t.contiguous()
