"""ConvLogicLayer, its autograd functions and PoolLogicLayer.
Interface of the reference's src/convlogic/convlogic_layer.py, on HIP kernels for gfx950."""
import torch
from torch import nn
from torch.autograd import Function

from ..difflogic.functional import GradFactor, bin_op_s
from ..difflogic.packbitstensor import PackBitsTensor
from ..hip import convlogic_hip
from .treelogic_layer import gate_probabilities


class ConvLogicFunction(Function):
    """Split layer: 4 leaf gates per kernel, [N,C,Ho,Wo,4] (src/convlogic/convlogic_layer.py:16-33)."""

    @staticmethod
    def forward(ctx, x, w_prob, selection, stride_h, stride_w, pad_h, pad_w, kernel_h, kernel_w):
        x, w_prob, selection = x.contiguous(), w_prob.contiguous(), selection.contiguous()
        y = convlogic_hip.convlogic_forward(x, w_prob, selection, stride_h, stride_w, pad_h, pad_w, kernel_h, kernel_w)
        ctx.save_for_backward(x, w_prob, selection)
        ctx.geometry = (stride_h, stride_w, pad_h, pad_w)
        return y

    @staticmethod
    def backward(ctx, grad_y):
        grad_y = grad_y.contiguous()
        x, w_prob, selection = ctx.saved_tensors
        grad_x = grad_w = None
        if ctx.needs_input_grad[0]:
            grad_x = convlogic_hip.convlogic_backward_x(grad_y, x, w_prob, selection, *ctx.geometry)
        if ctx.needs_input_grad[1]:
            grad_w = convlogic_hip.convlogic_backward_weight(grad_y, x, selection, *ctx.geometry)
        return grad_x, grad_w, None, None, None, None, None, None, None


class FullConvLogicFunction(Function):
    """Fused block: taps -> 4 leaf gates -> 2 gates -> root gate -> 2x2/2 max pool
    (src/convlogic/convlogic_layer.py:36-82).  Only the pooled output and one byte per pooled value
    (which window position won) are kept for backward; the leaf and middle planes are produced on
    request (return_intermediate) by a separate kernel."""

    @staticmethod
    def forward(ctx, x, w_prob, selection, stride_h, stride_w, pad_h, pad_w, kernel_h, kernel_w,
                return_intermediate=False, return_indices=False):
        x1, w_prob, selection = x.contiguous(), w_prob.contiguous(), selection.contiguous()
        geo = (stride_h, stride_w, pad_h, pad_w)
        y, argmax = convlogic_hip.full_convlogic_forward(x1, w_prob, selection, *geo, kernel_h, kernel_w)
        ctx.save_for_backward(x1, w_prob, selection, argmax)
        ctx.geometry = geo
        extra = []
        if return_intermediate:
            extra += list(convlogic_hip.full_convlogic_intermediates(x1, w_prob, selection, *geo, kernel_h, kernel_w))
        if return_indices:
            extra.append(convlogic_hip.argmax_to_indices(argmax, 2 * argmax.shape[3]))
        if not extra:
            return y
        ctx.mark_non_differentiable(*extra)
        return (y, *extra)

    @staticmethod
    def backward(ctx, grad_y, *_unused):
        grad_y = grad_y.contiguous()
        x1, w_prob, selection, argmax = ctx.saved_tensors
        grad_x = grad_w = None
        if ctx.needs_input_grad[0] and ctx.needs_input_grad[1]:
            grad_x, grad_w = convlogic_hip.full_convlogic_backward(grad_y, x1, w_prob, argmax, selection, *ctx.geometry)
        elif ctx.needs_input_grad[0]:
            grad_x = convlogic_hip.full_convlogic_backward_x(grad_y, x1, w_prob, argmax, selection, *ctx.geometry)
        elif ctx.needs_input_grad[1]:
            grad_w = convlogic_hip.full_convlogic_backward_weight(grad_y, x1, w_prob, argmax, selection, *ctx.geometry)
        return grad_x, grad_w, None, None, None, None, None, None, None, None, None


class _FullConvLogicLogitsFunction(Function):
    """Training path of the module: the complete block as a function of the LOGITS.  The softmax runs inside
    forward, its backward is fused into the weight-gradient kernel, so a step has no separate softmax nodes
    (same values as softmax + FullConvLogicFunction up to rounding)."""

    @staticmethod
    def forward(ctx, x, logits, selection, stride_h, stride_w, pad_h, pad_w, kernel_h, kernel_w, feature_major=False, plan=None,
                prefolded=None):
        # prefolded: (probs, folded) of these logits, made by the network for all its layers in one launch (fold_many)
        x1, selection, logits = x.contiguous(), selection.contiguous(), logits.contiguous()
        geo = (stride_h, stride_w, pad_h, pad_w)
        ctx.geometry, ctx.kernel = geo, (kernel_h, kernel_w)
        ctx.plan = plan                                              # (plan bytes, signature) of the layer for this input shape, or None
        # y in memory as [C, Ho/2, Wo/2, N] where asked for and possible, handed out as the [N, C, Ho/2, Wo/2] view of it:
        # nn.Flatten and the LogicLayer behind it then work on that memory without a transposed copy, and so does the
        # way back
        fm = feature_major and convlogic_hip.feature_major_supported(x1, logits.shape[0], *geo, kernel_h, kernel_w)
        ctx.feature_major = fm
        if plan is not None:
            # the forward launch also leaves the folded coefficients for the planned backward pass and -- when the input
            # needs a gradient and the kernels of this shape read one -- the zero-padded copy of x it staged
            y, argmax, w_prob, folded, *rest = convlogic_hip.full_convlogic_forward_logits(
                x1, logits.detach(), selection, *geo, kernel_h, kernel_w, feature_major=fm, want_folded=True, validate=False,
                want_padded=ctx.needs_input_grad[0], prefolded=prefolded)
            padded = rest[0] if rest else None
            ctx.save_for_backward(x1, w_prob, selection, argmax, folded, *(() if padded is None else (padded,)))
            return y.permute(3, 0, 1, 2) if fm else y
        ctx.plan = None
        y, argmax, w_prob = convlogic_hip.full_convlogic_forward_logits(x1, logits.detach(), selection, *geo, kernel_h, kernel_w,
                                                                        feature_major=fm, validate=False)
        ctx.save_for_backward(x1, w_prob, selection, argmax)
        return y.permute(3, 0, 1, 2) if fm else y

    @staticmethod
    def backward(ctx, grad_y):
        need_x, need_w = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        if ctx.plan is not None:
            x1, w_prob, selection, argmax, folded, *rest = ctx.saved_tensors
            padded = rest[0] if rest else None
            if need_w:
                ok = grad_y.dtype == x1.dtype and grad_y.device == x1.device      # everything else was validated on the way in
                grad_fm = grad_y.permute(1, 2, 3, 0)
                use_fm = ctx.feature_major and not grad_y.is_contiguous() and grad_fm.is_contiguous()
                grad_x, grad_l = convlogic_hip.full_convlogic_backward_planned(grad_fm if use_fm else grad_y.contiguous(), x1, w_prob, folded,
                                                                               argmax, selection, *ctx.plan, *ctx.geometry, need_grad_x=need_x,
                                                                               validate=not ok, feature_major=use_fm,
                                                                               padded=None if use_fm else padded, kernel=ctx.kernel)
                return grad_x, grad_l, None, None, None, None, None, None, None, None, None, None
            grad_x = convlogic_hip.full_convlogic_backward_x(grad_y.contiguous(), x1, w_prob, argmax, selection, *ctx.geometry) if need_x else None
            return grad_x, None, None, None, None, None, None, None, None, None, None, None
        x1, w_prob, selection, argmax = ctx.saved_tensors
        grad_x = grad_l = None
        grad_fm = grad_y.permute(1, 2, 3, 0)
        if (need_w and not grad_y.is_contiguous() and grad_fm.is_contiguous()
                and convlogic_hip.feature_major_supported(x1, w_prob.shape[0], *ctx.geometry, *ctx.kernel)):
            grad_x, grad_l = convlogic_hip.full_convlogic_backward_fm(grad_fm, x1, w_prob, argmax, selection, *ctx.geometry,
                                                                     need_grad_x=need_x, validate=grad_y.dtype != x1.dtype or grad_y.device != x1.device)
            return grad_x, grad_l, None, None, None, None, None, None, None, None, None, None
        grad_y = grad_y.contiguous()
        if need_w:
            grad_x, grad_l = convlogic_hip.full_convlogic_backward_logits(grad_y, x1, w_prob, argmax, selection, *ctx.geometry,
                                                                         need_grad_x=need_x)
        elif need_x:
            grad_x = convlogic_hip.full_convlogic_backward_x(grad_y, x1, w_prob, argmax, selection, *ctx.geometry)
        return grad_x, grad_l, None, None, None, None, None, None, None, None, None, None


class _FullConvLogicBinaryFunction(Function):
    """The complete block on an input that holds only 0 and 1 (the thresholded image in front of the first block,
    src/convlogic/data.py:46-50): forward through one 256-entry table per kernel, backward from the saved tap bytes
    alone.  w: the logits (is_logits, training path) or the probabilities.  Same y and pool routing as
    FullConvLogicFunction bit for bit; gradients equal up to float rounding."""

    @staticmethod
    def forward(ctx, x, w, selection, stride_h, stride_w, pad_h, pad_w, kernel_h, kernel_w, is_logits, flag):
        x1, w1, selection = x.contiguous(), w.detach().contiguous(), selection.contiguous()
        geo = (stride_h, stride_w, pad_h, pad_w)
        y, taps, bctx = convlogic_hip.bin_forward(x1, w1, selection, *geo, kernel_h, kernel_w, flag, logits=is_logits)
        ctx.save_for_backward(taps, bctx)                            # x itself is not needed again
        ctx.geometry, ctx.x_shape, ctx.is_logits = geo, tuple(x1.shape), is_logits
        return y

    @staticmethod
    def backward(ctx, grad_y):
        taps, bctx = ctx.saved_tensors
        grad_x, grad_w = convlogic_hip.bin_backward(grad_y.contiguous(), taps, bctx, ctx.x_shape, *ctx.geometry,
                                                    need_grad_x=ctx.needs_input_grad[0], need_grad_w=ctx.needs_input_grad[1],
                                                    wrt_logits=ctx.is_logits)
        return grad_x, grad_w, None, None, None, None, None, None, None, None, None


def _pair(v):
    return (v, v) if isinstance(v, int) else tuple(v)


class ConvLogicLayer(nn.Module):
    """Logic-gate convolution: every output channel reads 8 taps (from at most two input channels of
    its group) inside its receptive field and combines them with 4 gates, or with the complete
    4 -> 2 -> 1 tree followed by 2x2 OR(max)-pooling when complete=True
    (src/convlogic/convlogic_layer.py:85-160)."""

    def __init__(self, in_channels: int, out_channels: int, stride=1, padding=1, kernel=3, groups: int = 1,
                 selection=None, residual_init: bool = False, implementation: str = "cuda", grad_factor: float = 1.0,
                 complete: bool = False, return_intermediate: bool = False, return_indices: bool = False):
        super().__init__()
        self.in_channels, self.out_channels = in_channels, out_channels
        self.stride, self.padding, self.kernel = _pair(stride), _pair(padding), _pair(kernel)
        self.groups, self.grad_factor, self.complete = groups, grad_factor, complete
        self.return_intermediate, self.return_indices = return_intermediate, return_indices
        self.input_bits = 8
        self.implementation = implementation
        # A promise of the caller (the model topologies set it on their first block): every input element is 0 or 1.
        # The "cuda" path then runs the binary-input kernels where they apply; the kernels verify the promise and
        # check_binary_input() / the next forward call raise when it was broken.
        self.binary_input = False
        if implementation == "cuda" and not torch.cuda.is_available():
            raise RuntimeError("CUDA implementation requested, but CUDA is not available.")

        gates = 7 if complete else 4
        if residual_init:
            logits = torch.zeros(out_channels, gates, 16)
            logits[..., 3] = 5.0
        else:
            logits = torch.randn(out_channels, gates, 16)
        self.weights = nn.Parameter(logits)

        if selection is None:
            selection = self.generate_selection()
        self.register_buffer("selection", selection)
        assert selection.shape == (out_channels, 8)
        assert self.weights.shape[-1] == 16, f"Expected 16 logic functions, got {self.weights.shape[-1]}"
        self._check_selection()

    def _check_selection(self):
        """The kernels size their tiles from the geometry and read taps without bounds checks on the channel, row and
        column a tap names: a selection outside (in_channels, kernel) must raise here instead of faulting the GPU.
        Checked at construction, on the first launch and whenever the buffer was modified in place (version counter)
        or replaced; writes through `.data` bypass the counter -- call invalidate() after those."""
        sel = self._buffers["selection"]                             # (not through nn.Module.__getattr__: taken on every call)
        key = (sel._version, sel.data_ptr())
        if self.__dict__.get("_selection_checked") == key:
            return
        if sel.dtype != torch.int32 or tuple(sel.shape) != (self.out_channels, 8):
            raise ValueError(f"selection must be int32 [{self.out_channels}, 8], got {sel.dtype} {tuple(sel.shape)}")
        ch, row, col = self.unpack_selection(sel)
        if sel.numel() and (int(ch.max()) >= self.in_channels or int(row.max()) >= self.kernel[0] or int(col.max()) >= self.kernel[1]):
            raise ValueError(f"selection names a tap outside {self.in_channels} input channels and a "
                             f"{self.kernel[0]}x{self.kernel[1]} receptive field")
        self._selection_checked = key

    def invalidate(self):
        """Forces the next call to check the selection buffer again and to rebuild the backward plans (after a write
        through `.data`)."""
        self._selection_checked = None
        self._plans = {}

    def _backward_plan(self, x, sel):
        """(plan bytes, signature) of this layer's backward pass for inputs like x: the reverse map input channel ->
        kernels and the tap offsets of the kernels' image layout, which depend only on the selection and the geometry.
        Built on the first training step with a shape and kept (the reference's LogicLayer builds its reverse map at
        construction, src/difflogic/difflogic.py:71-87); rebuilt when the selection buffer or the library's knobs change."""
        from ..hip import _lib
        key = (tuple(x.shape), x.dtype, x.device, sel._version, sel.data_ptr(), _lib.knob_generation())
        plans = self.__dict__.setdefault("_plans", {})
        plan = plans.get(key)
        if plan is None:
            if len(plans) >= 4:                                      # a few batch shapes (training, last partial batch, evaluation)
                plans.pop(next(iter(plans)))
            plan = plans[key] = convlogic_hip.make_backward_plan(x, self.out_channels, sel, *self.stride, *self.padding, *self.kernel)
        return plan

    def prefold_candidate(self):
        """The logits a network may fold for this layer ahead of its forward call (one launch for all its layers,
        difflogic_hip.fold_many), or None when the layer's training path does not take the result."""
        w = self._parameters["weights"]
        if (self.implementation == "cuda" and self.complete and self.training and not self.return_intermediate
                and not self.return_indices and not self.__dict__.get("binary_input", False) and w.is_cuda and w.is_contiguous()
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

    def _load_from_state_dict(self, *args, **kwargs):
        super()._load_from_state_dict(*args, **kwargs)
        self.invalidate()

    def forward(self, x):
        if isinstance(x, PackBitsTensor):
            return self.forward_cuda_eval(x)
        x = x.contiguous()
        if self.grad_factor != 1.0:
            x = GradFactor.apply(x, self.grad_factor)
        if self.implementation == "cuda":
            return self.forward_cuda(x)
        if self.implementation == "python":
            return self.forward_python_full(x) if self.complete else self.forward_python(x)
        raise ValueError(f"Unknown implementation {self.implementation!r}")

    def unpack_selection(self, selection: torch.Tensor):
        return (selection >> 16) & 0xFFFF, (selection >> 8) & 0xFF, selection & 0xFF

    def _tap_values(self, x):
        """[N,C,Ho,Wo,8] tap values, zero outside the image: tap t of kernel c at (oy,ox) reads
        x[n, ch, oy*sh + ry - ph, ox*sw + rx - pw] (src/convlogic/convlogic_layer.py:262-282)."""
        (sh, sw), (ph, pw), (kh, kw) = self.stride, self.padding, self.kernel
        h, w = x.shape[2], x.shape[3]
        ho, wo = (h + 2 * ph - kh) // sh + 1, (w + 2 * pw - kw) // sw + 1
        ch, ry, rx = (t.long() for t in self.unpack_selection(self.selection))
        xp = torch.nn.functional.pad(x, (pw, pw, ph, ph))
        rows = (torch.arange(ho, device=x.device) * sh).view(1, ho, 1, 1) + ry.view(-1, 1, 1, 8)
        cols = (torch.arange(wo, device=x.device) * sw).view(1, 1, wo, 1) + rx.view(-1, 1, 1, 8)
        shape = (self.out_channels, ho, wo, 8)
        return xp[:, ch.view(-1, 1, 1, 8).expand(shape), rows.expand(shape), cols.expand(shape)]

    def forward_python(self, x):
        """Torch-op implementation of the 4-leaf layer -> [N,C,Ho,Wo,4]."""
        taps = self._tap_values(x)
        w_prob = gate_probabilities(self.weights[:, 0:4], self.training, self.weights.dtype)
        return bin_op_s(taps[..., 0::2], taps[..., 1::2], w_prob.view(1, self.out_channels, 1, 1, 4, 16))

    def forward_python_full(self, x):
        """Torch-op implementation of the complete block: gates 0:4 on the tap pairs, gates 4:6 on the
        leaf pairs, gate 6 on top, then 2x2 max pooling (src/convlogic/convlogic_layer.py:231-316)."""
        c = self.out_channels
        level = self._tap_values(x.contiguous())
        for lo, hi in ((0, 4), (4, 6), (6, 7)):
            w_prob = gate_probabilities(self.weights[:, lo:hi], self.training, x.dtype).view(1, c, 1, 1, hi - lo, 16)
            level = bin_op_s(level[..., 0::2], level[..., 1::2], w_prob)
        return PoolLogicLayer()(level)

    def forward_cuda(self, x):
        self._check_selection()
        if x.dim() != 4 or x.shape[1] != self.in_channels:          # the taps index channels of x without bounds checks
            raise RuntimeError(f"Expected x of shape [N, {self.in_channels}, H, W], got {tuple(x.shape)}")
        x = x.contiguous()
        sel = self._buffers["selection"].contiguous()
        weights = self._parameters["weights"]
        geo = (*self.stride, *self.padding, *self.kernel)
        if (self.__dict__.get("binary_input") and self.complete and not self.return_intermediate and not self.return_indices
                and x.is_cuda and x.dtype == torch.float32 and weights.dtype == torch.float32 and weights.device == x.device
                and sel.device == x.device and convlogic_hip.bin_supported(x, self.out_channels, *geo)):
            flag = self._binary_flag()
            if flag.raised():
                flag.clear()
                raise RuntimeError("ConvLogicLayer(binary_input=True) was given an input with elements other than 0 and 1")
            if self.training and weights.is_contiguous():
                return _FullConvLogicBinaryFunction.apply(x, weights, sel, *geo, True, flag)
            w_prob = gate_probabilities(self.weights, self.training, x.dtype).to(x.dtype).contiguous()
            return _FullConvLogicBinaryFunction.apply(x, w_prob, sel, *geo, False, flag)
        if (self.complete and self.training and not self.return_intermediate and not self.return_indices and x.is_cuda
                and weights.dtype == x.dtype and x.dtype in (torch.float32, torch.float64) and weights.is_contiguous()
                and weights.device == x.device and sel.device == x.device):
            plan = self._backward_plan(x, sel)
            return _FullConvLogicLogitsFunction.apply(x, weights, sel, *geo, self.__dict__.get("feature_major_output", False), plan,
                                                      self._take_prefold(weights) if plan is not None else None)
        # the kernels read the probabilities in x's element type (the bindings reject any other)
        w_prob = gate_probabilities(self.weights, self.training, x.dtype).to(x.dtype).contiguous()
        if self.complete:
            return FullConvLogicFunction.apply(x, w_prob, sel, *geo, self.return_intermediate, self.return_indices)
        return ConvLogicFunction.apply(x, w_prob, sel, *geo)

    def _binary_flag(self):
        flag = self.__dict__.get("_bin_flag")
        if flag is None:
            flag = self.__dict__["_bin_flag"] = convlogic_hip.BinaryFlag()
        return flag

    def check_binary_input(self):
        """Waits for the device and raises if a forward call since the last check saw an input element other than 0 or 1
        although binary_input was set (without this call the violation is reported by the next forward call that runs
        after the offending launch has finished)."""
        flag = self.__dict__.get("_bin_flag")
        if flag is None:
            return
        torch.cuda.synchronize()
        if flag.raised():
            flag.clear()
            raise RuntimeError("ConvLogicLayer(binary_input=True) was given an input with elements other than 0 and 1")

    def forward_cuda_eval(self, x: PackBitsTensor):
        """Packed-bit inference of the complete block on a group-major image batch: replaces x.t by the
        block output, 64 samples per word (the counterpart of LogicLayer.forward_cuda_eval,
        src/difflogic/difflogic.py:149-164, for the fused block; arg-max gates as in :321-325 of
        src/convlogic/convlogic_layer.py, max pool of {0,1} values = OR)."""
        assert not self.training, "packed evaluation needs eval mode"
        assert self.complete, "packed evaluation is implemented for the complete block only"
        if self.implementation != "cuda":
            raise RuntimeError("packed evaluation needs implementation='cuda'")
        assert x.image and x.t.dim() == 4 and x.t.shape[1] == self.in_channels, (x.image, tuple(x.t.shape), self.in_channels)
        self._check_selection()
        x.t = convlogic_hip.full_convlogic_eval_packed(x.t.contiguous(), self._eval_gates(), self.selection.contiguous(),
                                                       *self.stride, *self.padding, *self.kernel,
                                                       feature_major=getattr(self, "feature_major_output", False))
        return x

    def _eval_gates(self):
        """uint8 [C, 7] arg-max gate ids, taken from the logits on every call (one small launch; nothing cached that an
        in-place update of `weights.data` could leave stale)."""
        from ..hip import difflogic_hip
        return difflogic_hip.gate_argmax(self.weights.detach().contiguous())

    def extra_repr(self):
        return f"in_channels={self.in_channels}, out_channels={self.out_channels}, groups={self.groups}"

    def generate_selection(self) -> torch.Tensor:
        """Random taps, int32 [out_channels, 8] packed ch << 16 | row << 8 | col.  Draws from the global
        torch generator in the order of src/convlogic/convlogic_layer.py:377-452 (two channels per
        kernel inside its group, a channel pick per tap, rows, columns, then re-draws of the second tap
        of a pair that landed on the first), so equal seeds give equal selections."""
        dev = self.weights.device
        taps, (kh, kw) = self.input_bits, self.kernel
        c_out, c_in, groups = self.out_channels, self.in_channels, self.groups

        # input channels are split into `groups` nearly equal runs; output channels likewise
        sizes = [c_in // groups + (1 if gi < c_in % groups else 0) for gi in range(groups)]
        first = [sum(sizes[:gi]) for gi in range(groups)]
        group_of = torch.clamp(torch.arange(c_out, device=dev) // (c_out // groups), 0, groups - 1)
        pair = torch.empty((c_out, 2), dtype=torch.int32, device=dev)
        for gi in range(groups):
            members = (group_of == gi).nonzero(as_tuple=True)[0]
            if members.numel() > 0:
                for slot in range(2):
                    pick = torch.randint(0, sizes[gi], (members.numel(),), device=dev)
                    pair[members, slot] = (pick + first[gi]).to(torch.int32)

        which = torch.randint(0, 2, (c_out, taps), device=dev, dtype=torch.int32)
        ch = torch.where(which == 0, pair[:, 0:1], pair[:, 1:2]).expand(c_out, taps).contiguous()
        rows = torch.randint(0, kh, (c_out, taps), device=dev, dtype=torch.int32)
        cols = torch.randint(0, kw, (c_out, taps), device=dev, dtype=torch.int32)

        # the two taps of a gate must not be the same element (same position on different channels is fine)
        for t in range(0, taps, 2):
            same = (ch[:, t] == ch[:, t + 1]) & (rows[:, t] == rows[:, t + 1]) & (cols[:, t] == cols[:, t + 1])
            if kh * kw == 1 and bool(same.any()):
                # a window of one element has no other position to draw: the reference's loop (:437-448) would never end
                raise ValueError("a 1x1 kernel cannot give the two inputs of a gate different taps once both draw the same channel")
            for c in same.nonzero(as_tuple=True)[0].tolist():
                while True:
                    r = torch.randint(0, kh, (1,), device=dev, dtype=torch.int32)
                    q = torch.randint(0, kw, (1,), device=dev, dtype=torch.int32)
                    if (r.item(), q.item()) != (rows[c, t].item(), cols[c, t].item()):
                        rows[c, t + 1], cols[c, t + 1] = r, q
                        break
        return (ch << 16) | (rows << 8) | cols


class PoolLogicLayer(nn.Module):
    """Max pooling, the OR of a logic network (src/convlogic/convlogic_layer.py:455-480)."""

    def __init__(self, kernel=2, stride=2, return_indices=False):
        super().__init__()
        self.kernel, self.stride, self.return_indices = _pair(kernel), _pair(stride), return_indices

    def forward(self, x):
        if x.ndim == 5:
            if x.size(4) != 1:
                raise ValueError(f"Expected last dim=1, got {x.size(4)}")
            x = x.view(x.shape[:4])
        elif x.ndim != 4:
            raise ValueError("Input must be 4D or 5D")
        return nn.functional.max_pool2d(x, self.kernel, self.stride, return_indices=self.return_indices)
