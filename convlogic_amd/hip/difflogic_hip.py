"""Function set of the reference's `difflogic_cuda` module (src/difflogic/cuda/difflogic.cpp:15-34)
on top of the HIP C ABI.  Tensors are feature-major ([features, batch]) as in the reference."""
import torch

from . import _lib
from ._lib import check, check_input, dtype_code, stream_ptr

_WORD_DTYPE = {8: torch.int8, 16: torch.int16, 32: torch.int32, 64: torch.int64}
_I64 = torch.int64


def _wiring(x, a, b, out_dim):
    """x [in, B] with the wiring a, b int64 [out] on x's device -> (in_dim, batch)."""
    check_input(x, "x")
    if x.dim() != 2:
        raise RuntimeError(f"x must be 2-D [in_dim, batch], got {tuple(x.shape)}")
    check_input(a, "a", _I64, (out_dim,))
    check_input(b, "b", _I64, (out_dim,))
    _lib.check_same_device(x, a, b)
    return x.shape


def _reverse_map(x, start, flat, out_dim):
    check_input(start, "given_x_indices_of_y_start", _I64, (x.shape[0] + 1,))
    check_input(flat, "given_x_indices_of_y", _I64, (2 * out_dim,))
    _lib.check_same_device(x, start, flat)


def forward(x, a, b, w):
    """y[out, B]; difflogic_cuda.forward (src/difflogic/cuda/difflogic_kernel.cu:89-126)."""
    out_dim = w.shape[0] if w.dim() else -1
    in_dim, batch = _wiring(x, a, b, out_dim)
    check_input(w, "w", x.dtype, (out_dim, 16))
    y = torch.empty((out_dim, batch), dtype=x.dtype, device=x.device)
    if y.numel():
        check(_lib.load().clg_fc_forward(dtype_code(x, half_ok=True), x.data_ptr(), a.data_ptr(), b.data_ptr(), w.data_ptr(), y.data_ptr(),
                                         in_dim, out_dim, batch, stream_ptr(x)))
    return y


def backward_w(x, a, b, grad_y):
    """grad_w[out, 16]; difflogic_cuda.backward_w (difflogic_kernel.cu:128-173)."""
    out_dim = grad_y.shape[0] if grad_y.dim() else -1
    in_dim, batch = _wiring(x, a, b, out_dim)
    check_input(grad_y, "grad_y", x.dtype, (out_dim, batch))
    gw = torch.empty((out_dim, 16), dtype=x.dtype, device=x.device)
    check(_lib.load().clg_fc_backward_w(dtype_code(x, half_ok=True), x.data_ptr(), a.data_ptr(), b.data_ptr(), grad_y.data_ptr(),
                                        gw.data_ptr(), in_dim, out_dim, batch, stream_ptr(x)))
    return gw


def backward_logits(x, a, b, w, grad_y, validate=True):
    """Gradient w.r.t. the logits [out, 16] when w = softmax(logits): backward_w and the softmax backward
    in one kernel."""
    out_dim = grad_y.shape[0] if grad_y.dim() else -1
    if validate:
        _wiring(x, a, b, out_dim)
        check_input(w, "w", x.dtype, (out_dim, 16))
        check_input(grad_y, "grad_y", x.dtype, (out_dim, x.shape[1]))
    in_dim, batch = x.shape
    gl = torch.empty((out_dim, 16), dtype=x.dtype, device=x.device)
    check(_lib.load().clg_fc_backward_logits(dtype_code(x), x.data_ptr(), a.data_ptr(), b.data_ptr(), w.data_ptr(),
                                             grad_y.data_ptr(), gl.data_ptr(), in_dim, out_dim, batch, stream_ptr(x)))
    return gl


def fold(w_in, from_logits, want_probs=True):
    """[out, 16] logits or probabilities -> (probabilities or None, folded coefficients [out, 4])."""
    check_input(w_in, "w")
    if w_in.dim() != 2 or w_in.shape[1] != 16:
        raise RuntimeError(f"w must have shape [out_dim, 16], got {tuple(w_in.shape)}")
    out_dim = w_in.shape[0]
    probs = torch.empty_like(w_in) if want_probs else None
    folded = torch.empty((out_dim, 4), dtype=w_in.dtype, device=w_in.device)
    check(_lib.load().clg_fc_fold(dtype_code(w_in), int(bool(from_logits)), w_in.data_ptr(),
                                  probs.data_ptr() if want_probs else 0, folded.data_ptr(), out_dim, stream_ptr(w_in)))
    return probs, folded


FOLD_MANY_MAX = 16


class FoldPlan:
    """What fold_many() needs of a fixed list of logit tensors besides a fresh output buffer: row counts, chunk sizes
    and shapes, and the host arrays of the call (kept by a network across its training steps)."""

    def __init__(self, logits_list):
        import ctypes
        n = len(logits_list)
        if not 1 <= n <= FOLD_MANY_MAX:
            raise RuntimeError(f"fold_many takes 1 to {FOLD_MANY_MAX} tensors, got {n}")
        first = logits_list[0]
        for t in logits_list:
            check_input(t, "logits", first.dtype)
            if t.device != first.device or t.dim() < 2 or t.shape[-1] != 16:
                raise RuntimeError("fold_many: logits must share a device and have 16 entries per row")
        self.n, self.dtype, self.device, self.code = n, first.dtype, first.device, dtype_code(first)
        self.rows = [t.numel() // 16 for t in logits_list]
        self.sizes = [s for r in self.rows for s in (16 * r, 4 * r)]
        self.shapes = [s for t in logits_list for s in (tuple(t.shape), (*t.shape[:-1], 4))]
        self.total = 20 * sum(self.rows)
        self.ptrs = tuple(t.data_ptr() for t in logits_list)
        self.logits_arr = (ctypes.c_void_p * n)(*self.ptrs)
        self.rows_arr = (ctypes.c_int64 * n)(*self.rows)
        self.out_arr = ctypes.c_void_p * n
        self.elem = first.element_size()

    def matches(self, logits_list):
        return len(logits_list) == self.n and all(t.data_ptr() == p and t.dtype == self.dtype and t.numel() == 16 * r and t.is_contiguous()
                                                  for t, p, r in zip(logits_list, self.ptrs, self.rows))


def fold_many(logits_list, plan=None):
    """softmax + fold of up to 16 logit tensors [..., 16] of one dtype and device in ONE launch -> a list of
    (probs, folded) with probs shaped like the logits and folded [..., 4]; each pair lives in one buffer, probabilities
    first (the layout full_convlogic_forward_logits(prefolded=...) and the block's backward expect).  Row by row the
    values of fold(from_logits=True).  plan: a FoldPlan made from the same tensors (saves the per-call bookkeeping)."""
    if plan is None or not plan.matches(logits_list):
        plan = FoldPlan(logits_list)
    buf = torch.empty((plan.total,), dtype=plan.dtype, device=plan.device)
    chunks = buf.split_with_sizes(plan.sizes)
    views = [c.view(s) for c, s in zip(chunks, plan.shapes)]
    base, at, pp, fp = buf.data_ptr(), 0, [], []
    for r in plan.rows:
        pp.append(base + at * plan.elem)
        fp.append(base + (at + 16 * r) * plan.elem)
        at += 20 * r
    check(_lib.load().clg_fold_many(plan.code, plan.n, plan.logits_arr, plan.out_arr(*pp), plan.out_arr(*fp), plan.rows_arr,
                                    stream_ptr(buf)))
    return list(zip(views[0::2], views[1::2]))


def forward_folded(x, a, b, folded):
    """forward() with the folded coefficients [out, 4] of fold() in place of w."""
    out_dim = folded.shape[0] if folded.dim() else -1
    in_dim, batch = _wiring(x, a, b, out_dim)
    check_input(folded, "folded", x.dtype, (out_dim, 4))
    y = torch.empty((out_dim, batch), dtype=x.dtype, device=x.device)
    check(_lib.load().clg_fc_forward_folded(dtype_code(x), x.data_ptr(), a.data_ptr(), b.data_ptr(), folded.data_ptr(),
                                            y.data_ptr(), in_dim, out_dim, batch, stream_ptr(x)))
    return y


def forward_logits(x, a, b, logits, validate=True, sample_major_x=False):
    """fold(from_logits=True) + forward_folded() in one launch -> (y [out, B], probs [out, 16], folded [out, 4]).
    sample_major_x: x is [B, in]; the same call makes its feature-major copy [in, B] first and returns it as a fourth
    value (the backward functions read it)."""
    out_dim = logits.shape[0]
    if validate:
        if logits.dim() != 2 or logits.shape[1] != 16 or logits.dtype != x.dtype or x.dtype not in _lib._DTYPES:
            raise RuntimeError(f"forward_logits expects float32/float64 logits [out, 16] of x's dtype, got {tuple(logits.shape)} {logits.dtype}")
        if sample_major_x:
            check_input(x, "x")
            if x.dim() != 2:
                raise RuntimeError(f"x must be 2-D, got {tuple(x.shape)}")
            check_input(a, "a", _I64, (out_dim,))
            check_input(b, "b", _I64, (out_dim,))
            _lib.check_same_device(x, a, b)
        else:
            _wiring(x, a, b, out_dim)
        check_input(logits, "w")
    in_dim, batch = (x.shape[1], x.shape[0]) if sample_major_x else x.shape
    y = torch.empty((out_dim, batch), dtype=x.dtype, device=x.device)
    probs = torch.empty_like(logits)
    folded = torch.empty((out_dim, 4), dtype=x.dtype, device=x.device)
    if not sample_major_x:
        check(_lib.load().clg_fc_forward_logits(dtype_code(x), x.data_ptr(), a.data_ptr(), b.data_ptr(), logits.data_ptr(),
                                                probs.data_ptr(), folded.data_ptr(), y.data_ptr(), in_dim, out_dim, batch,
                                                stream_ptr(x)))
        return y, probs, folded
    x_fm = torch.empty((in_dim, batch), dtype=x.dtype, device=x.device)
    check(_lib.load().clg_fc_forward_logits_ex(dtype_code(x), x.data_ptr(), a.data_ptr(), b.data_ptr(), logits.data_ptr(),
                                               probs.data_ptr(), folded.data_ptr(), y.data_ptr(), in_dim, out_dim, batch,
                                               1, x_fm.data_ptr(), stream_ptr(x)))
    return y, probs, folded, x_fm


def backward_x_folded(x, a, b, folded, grad_y, given_x_indices_of_y_start, given_x_indices_of_y, validate=True):
    """backward_x() with the folded coefficients [out, 4] of fold() in place of w."""
    out_dim = folded.shape[0] if folded.dim() else -1
    if validate:
        _wiring(x, a, b, out_dim)
        check_input(folded, "folded", x.dtype, (out_dim, 4))
        check_input(grad_y, "grad_y", x.dtype, (out_dim, x.shape[1]))
        _reverse_map(x, given_x_indices_of_y_start, given_x_indices_of_y, out_dim)
    in_dim, batch = x.shape
    gx = torch.empty_like(x)
    check(_lib.load().clg_fc_backward_x_folded(dtype_code(x), x.data_ptr(), a.data_ptr(), b.data_ptr(), folded.data_ptr(),
                                               grad_y.data_ptr(), given_x_indices_of_y_start.data_ptr(),
                                               given_x_indices_of_y.data_ptr(), gx.data_ptr(), in_dim, out_dim, batch,
                                               stream_ptr(x)))
    return gx


def backward_sole(x, a, b, folded, probs, grad_y, validate=True):
    """(grad_x, grad_w) in one pass for a layer whose inputs are each read by exactly one neuron operand; grad_w is
    the gradient w.r.t. the logits when probs = softmax(logits) is given, else w.r.t. the probabilities."""
    out_dim = folded.shape[0] if folded.dim() else -1
    if validate:
        _wiring(x, a, b, out_dim)
        check_input(folded, "folded", x.dtype, (out_dim, 4))
        check_input(grad_y, "grad_y", x.dtype, (out_dim, x.shape[1]))
        if probs is not None:
            check_input(probs, "w", x.dtype, (out_dim, 16))
    in_dim, batch = x.shape
    gx = torch.empty_like(x)
    gw = torch.empty((out_dim, 16), dtype=x.dtype, device=x.device)
    check(_lib.load().clg_fc_backward_sole(dtype_code(x), x.data_ptr(), a.data_ptr(), b.data_ptr(), folded.data_ptr(),
                                           probs.data_ptr() if probs is not None else 0, grad_y.data_ptr(), gx.data_ptr(),
                                           gw.data_ptr(), in_dim, out_dim, batch, stream_ptr(x)))
    return gx, gw


def backward_sole_classes(x, a, b, folded, probs, grad_out, k, tau, validate=True):
    """backward_sole() for a layer whose output goes straight into a GroupSum: grad_out [B, k] is the gradient of the
    GroupSum's output; the gradient of the layer's output (grad_out[:, class of the neuron] / tau) is formed inside the
    kernel.  Same values as group_sum_backward() + backward_sole(), bit for bit."""
    out_dim = folded.shape[0] if folded.dim() else -1
    in_dim, batch = x.shape
    if validate:
        _wiring(x, a, b, out_dim)
        check_input(folded, "folded", x.dtype, (out_dim, 4))
        check_input(grad_out, "grad_out", x.dtype, (batch, k))
        if probs is not None:
            check_input(probs, "w", x.dtype, (out_dim, 16))
    gx = torch.empty_like(x)
    gw = torch.empty((out_dim, 16), dtype=x.dtype, device=x.device)
    check(_lib.load().clg_fc_backward_sole_classes(dtype_code(x), x.data_ptr(), a.data_ptr(), b.data_ptr(), folded.data_ptr(),
                                                   probs.data_ptr() if probs is not None else 0, grad_out.data_ptr(), gx.data_ptr(),
                                                   gw.data_ptr(), in_dim, out_dim, batch, int(k), float(tau), stream_ptr(x)))
    return gx, gw


def backward_fused_fits(x):
    """True when backward_fused() covers the batch of feature-major x [in, B] in one pass."""
    return bool(_lib.load().clg_fc_backward_fused_fits(dtype_code(x), x.shape[1]))


def backward_fused(x, a, b, folded, probs, grad_y, given_x_indices_of_y_start, given_x_indices_of_y, validate=True,
                   sample_major_grad_x=False, sample_major_grad_y=False):
    """(grad_x, grad_w) of a layer with any wiring in one pass (see backward_fused_fits); grad_w is the gradient
    w.r.t. the logits when probs = softmax(logits) is given, else w.r.t. the probabilities.  Same values as
    backward_x_folded() + backward_w() / backward_logits().  sample_major_grad_x: grad_x comes back [B, in] instead of
    [in, B] (the kernel writes it transposed; same values).  sample_major_grad_y: grad_y is [B, out]; the same call makes
    its feature-major copy first."""
    out_dim = folded.shape[0] if folded.dim() else -1
    if validate:
        _wiring(x, a, b, out_dim)
        check_input(folded, "folded", x.dtype, (out_dim, 4))
        check_input(grad_y, "grad_y", x.dtype, (x.shape[1], out_dim) if sample_major_grad_y else (out_dim, x.shape[1]))
        _reverse_map(x, given_x_indices_of_y_start, given_x_indices_of_y, out_dim)
        if probs is not None:
            check_input(probs, "w", x.dtype, (out_dim, 16))
    in_dim, batch = x.shape
    gx = torch.empty((batch, in_dim) if sample_major_grad_x else (in_dim, batch), dtype=x.dtype, device=x.device)
    gw = torch.empty((out_dim, 16), dtype=x.dtype, device=x.device)
    gy_fm = torch.empty((out_dim, batch), dtype=x.dtype, device=x.device) if sample_major_grad_y else None
    check(_lib.load().clg_fc_backward_fused_ex(dtype_code(x), x.data_ptr(), a.data_ptr(), b.data_ptr(), folded.data_ptr(),
                                               probs.data_ptr() if probs is not None else None, grad_y.data_ptr(),
                                               given_x_indices_of_y_start.data_ptr(), given_x_indices_of_y.data_ptr(),
                                               gx.data_ptr(), gw.data_ptr(), in_dim, out_dim, batch,
                                               (1 if sample_major_grad_x else 0) | (2 if sample_major_grad_y else 0),
                                               gy_fm.data_ptr() if sample_major_grad_y else None, stream_ptr(x)))
    return gx, gw


def group_sum(x_fm, k, tau=1.0):
    """Feature-major activations [F, B] -> per-class sums [B, k] divided by tau, fixed summation order."""
    check_input(x_fm, "x")
    if x_fm.dim() != 2:
        raise RuntimeError(f"x must be 2-D [features, batch], got {tuple(x_fm.shape)}")
    features, batch = x_fm.shape
    if features % k != 0:
        raise ValueError(f"in_dim ({features}) has to be divisible by k ({k}) but it is not")
    lib = _lib.load()
    dt = dtype_code(x_fm)
    out = torch.empty((batch, k), dtype=x_fm.dtype, device=x_fm.device)
    if lib.clg_group_sum_once_fits(features, batch, k):               # one launch, no partial sums
        check(lib.clg_group_sum_once(dt, x_fm.data_ptr(), out.data_ptr(), features, batch, k, float(tau), stream_ptr(x_fm)))
        return out
    nbytes = lib.clg_group_sum_scratch_bytes(dt, features, batch, k)
    scratch = torch.empty((max(int(nbytes), 8),), dtype=torch.uint8, device=x_fm.device)
    check(lib.clg_group_sum(dt, x_fm.data_ptr(), out.data_ptr(), scratch.data_ptr(), features, batch, k, float(tau), stream_ptr(x_fm)))
    return out


def group_sum_backward(grad_out, features, tau=1.0):
    """[B, k] -> feature-major gradient [F, B]: every row of class g receives grad_out[:, g] / tau."""
    check_input(grad_out, "grad_out")
    if grad_out.dim() != 2 or grad_out.shape[1] < 1 or features % grad_out.shape[1] != 0:
        raise RuntimeError(f"grad_out must be [batch, k] with k dividing {features}, got {tuple(grad_out.shape)}")
    batch, k = grad_out.shape
    gx = torch.empty((features, batch), dtype=grad_out.dtype, device=grad_out.device)
    check(_lib.load().clg_group_sum_backward(dtype_code(grad_out), grad_out.data_ptr(), gx.data_ptr(), features, batch, k,
                                             float(tau), stream_ptr(grad_out)))
    return gx


def backward_x(x, a, b, w, grad_y, given_x_indices_of_y_start, given_x_indices_of_y):
    """grad_x[in, B]; difflogic_cuda.backward_x (difflogic_kernel.cu:232-269)."""
    out_dim = w.shape[0] if w.dim() else -1
    in_dim, batch = _wiring(x, a, b, out_dim)
    check_input(w, "w", x.dtype, (out_dim, 16))
    check_input(grad_y, "grad_y", x.dtype, (out_dim, batch))
    _reverse_map(x, given_x_indices_of_y_start, given_x_indices_of_y, out_dim)
    gx = torch.empty_like(x)
    check(_lib.load().clg_fc_backward_x(dtype_code(x, half_ok=True), x.data_ptr(), a.data_ptr(), b.data_ptr(), w.data_ptr(),
                                        grad_y.data_ptr(), given_x_indices_of_y_start.data_ptr(),
                                        given_x_indices_of_y.data_ptr(), gx.data_ptr(), in_dim, out_dim, batch, stream_ptr(x)))
    return gx


def transpose(x):
    """Contiguous transposed copy of a 2-D tensor through the tiled HIP transpose."""
    check_input(x, "x")
    if x.dim() != 2:
        raise RuntimeError(f"transpose expects a 2-D tensor, got {tuple(x.shape)}")
    rows, cols = x.shape
    out = torch.empty((cols, rows), dtype=x.dtype, device=x.device)
    if out.numel():
        check(_lib.load().clg_transpose_2d(x.element_size(), x.data_ptr(), out.data_ptr(), rows, cols, stream_ptr(x)))
    return out


def eval(x, a, b, w):  # noqa: A001 - name of the reference binding
    """Packed-bit layer evaluation; difflogic_cuda.eval (difflogic_kernel.cu:295-330).
    x: integer words [in, W]; w: uint8 gate ids [out]."""
    if x.dtype not in _WORD_DTYPE.values() or w.dtype != torch.uint8 or w.dim() != 1:
        raise RuntimeError("eval expects int8/16/32/64 words and uint8 gate ids [out]")
    out_dim = w.shape[0]
    in_dim, words = _wiring(x, a, b, out_dim)
    check_input(w, "w")
    y = torch.empty((out_dim, words), dtype=x.dtype, device=x.device)
    check(_lib.load().clg_fc_eval_packed(x.element_size(), x.data_ptr(), a.data_ptr(), b.data_ptr(), w.data_ptr(),
                                         y.data_ptr(), in_dim, out_dim, words, stream_ptr(x)))
    return y


def gate_argmax(logits):
    """uint8 index of the first maximum over the last dimension (16 gates) of float logits [..., 16]."""
    check_input(logits, "weights")
    if logits.dim() < 1 or logits.shape[-1] != 16:
        raise RuntimeError(f"expected logits [..., 16], got {tuple(logits.shape)}")
    gate = torch.empty(logits.shape[:-1], dtype=torch.uint8, device=logits.device)
    if gate.numel():
        check(_lib.load().clg_gate_argmax(dtype_code(logits, half_ok=True), logits.data_ptr(), gate.data_ptr(), gate.numel(),
                                          stream_ptr(logits)))
    return gate


def eval_plan(a, b, in_dim):
    """Walk order of the wiring graph for eval_planned (int32 [out], on the device of `a`).  Host
    computation, done once per wiring."""
    a_h = a.detach().to("cpu", torch.int64).contiguous()
    b_h = b.detach().to("cpu", torch.int64).contiguous()
    plan = torch.empty(a_h.shape[0], dtype=torch.int32)
    check(_lib.load().clg_fc_eval_plan(a_h.data_ptr(), b_h.data_ptr(), in_dim, a_h.shape[0], plan.data_ptr()))
    return plan.to(a.device)


def eval_planned(x, a, b, w, plan):
    """eval() in the order of `plan` (from eval_plan for the same a, b): identical result, about half
    the input traffic."""
    if x.dtype not in _WORD_DTYPE.values() or w.dtype != torch.uint8 or plan.dtype != torch.int32 or w.dim() != 1:
        raise RuntimeError("eval_planned expects int8/16/32/64 words, uint8 gate ids [out] and an int32 plan")
    out_dim = w.shape[0]
    in_dim, words = _wiring(x, a, b, out_dim)
    check_input(w, "w")
    check_input(plan, "plan")
    if tuple(plan.shape) != (out_dim,):
        raise RuntimeError("plan does not match the number of neurons")
    y = torch.empty((out_dim, words), dtype=x.dtype, device=x.device)
    check(_lib.load().clg_fc_eval_packed_planned(x.element_size(), x.data_ptr(), a.data_ptr(), b.data_ptr(), w.data_ptr(),
                                                 plan.data_ptr(), y.data_ptr(), in_dim, out_dim, words, stream_ptr(x)))
    return y


def eval_planned_logits(x, a, b, logits, plan):
    """eval_planned(x, a, b, gate_argmax(logits), plan) -- in one launch where the rows are whole 16-byte vectors of at
    least 1 KiB and the logits float32 (the kernel takes the arg-max itself), in two launches otherwise.
    LogicLayer.forward_cuda_eval (src/difflogic/difflogic.py:149-164)."""
    if x.dtype not in _WORD_DTYPE.values() or plan.dtype != torch.int32 or logits.dim() != 2 or logits.shape[1] != 16:
        raise RuntimeError("eval_planned_logits expects int8/16/32/64 words, logits [out, 16] and an int32 plan")
    out_dim = logits.shape[0]
    in_dim, words = _wiring(x, a, b, out_dim)
    check_input(logits, "weights")
    check_input(plan, "plan")
    if tuple(plan.shape) != (out_dim,):
        raise RuntimeError("plan does not match the number of neurons")
    lib = _lib.load()
    y = torch.empty((out_dim, words), dtype=x.dtype, device=x.device)
    if logits.dtype != torch.float32 or not lib.clg_fc_eval_walk_fits(x.element_size(), x.data_ptr(), y.data_ptr(), words):
        return eval_planned(x, a, b, gate_argmax(logits), plan)
    check(lib.clg_fc_eval_packed_planned_logits(x.element_size(), x.data_ptr(), a.data_ptr(), b.data_ptr(), logits.data_ptr(),
                                                plan.data_ptr(), y.data_ptr(), in_dim, out_dim, words, stream_ptr(x)))
    return y


def _alloc_words(features, batch, bit_count, device):
    if bit_count not in _WORD_DTYPE:
        raise ValueError("`bit_count` has to be in { 8, 16, 32, 64 }")
    words = -(-batch // bit_count)
    pad_len = (bit_count - batch % bit_count) % bit_count
    return torch.empty((features, words), dtype=_WORD_DTYPE[bit_count], device=device), pad_len


def tensor_packbits_cuda(t, bit_count):
    """bool [F, B] -> (words [F, ceil(B/bits)], pad_len); difflogic_kernel.cu:368-413."""
    check_input(t, "t")
    if t.dtype != torch.bool:
        raise RuntimeError("tensor_packbits_cuda expects a bool tensor")
    features, batch = t.shape
    out, pad_len = _alloc_words(features, batch, bit_count, t.device)
    check(_lib.load().clg_pack_bits(t.data_ptr(), out.data_ptr(), features, batch, bit_count, stream_ptr(t)))
    return out, pad_len


def tensor_packbits_sample_major(t, bit_count):
    """bool [B, F] (sample-major, as PackBitsTensor receives it) -> (words [F, ceil(B/bits)], pad_len),
    without the transposed bool copy."""
    check_input(t, "t")
    if t.dtype != torch.bool:
        raise RuntimeError("tensor_packbits_sample_major expects a bool tensor")
    batch, features = t.shape
    out, pad_len = _alloc_words(features, batch, bit_count, t.device)
    check(_lib.load().clg_pack_bits_sample_major(t.data_ptr(), out.data_ptr(), features, batch, bit_count, stream_ptr(t)))
    return out, pad_len


def groupbitsum(b, pad_len, k):
    """int32 [samples, k]; difflogic_cuda.groupbitsum (difflogic.cpp:22-33, difflogic_kernel.cu:450-482)."""
    check_input(b, "b")
    if b.dim() != 2 or b.dtype not in _WORD_DTYPE.values():
        raise RuntimeError(f"groupbitsum expects int8/16/32/64 words [features, words], got {tuple(b.shape)} {b.dtype}")
    features, words = b.shape
    if features % k != 0:
        raise ValueError(f"in_dim ({features}) has to be divisible by k ({k}) but it is not")
    samples = words * 8 * b.element_size() - pad_len
    out = torch.empty((samples, k), dtype=torch.int32, device=b.device)
    check(_lib.load().clg_group_bit_sum(b.element_size(), b.data_ptr(), out.data_ptr(), features, words, pad_len, k,
                                        stream_ptr(b)))
    return out
