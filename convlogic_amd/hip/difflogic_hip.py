"""Function set of the reference's `difflogic_cuda` module (src/difflogic/cuda/difflogic.cpp:15-34)
on top of the HIP C ABI.  Tensors are feature-major ([features, batch]) as in the reference."""
import torch

from . import _lib
from ._lib import check, check_input, dtype_code, stream_ptr

_WORD_DTYPE = {8: torch.int8, 16: torch.int16, 32: torch.int32, 64: torch.int64}


def forward(x, a, b, w):
    """y[out, B]; difflogic_cuda.forward (src/difflogic/cuda/difflogic_kernel.cu:89-126)."""
    for t, n in ((x, "x"), (a, "a"), (b, "b"), (w, "w")):
        check_input(t, n)
    in_dim, batch = x.shape
    out_dim = w.shape[0]
    y = torch.empty((out_dim, batch), dtype=x.dtype, device=x.device)
    if y.numel():
        check(_lib.load().clg_fc_forward(dtype_code(x, half_ok=True), x.data_ptr(), a.data_ptr(), b.data_ptr(), w.data_ptr(), y.data_ptr(),
                                         in_dim, out_dim, batch, stream_ptr(x)))
    return y


def backward_w(x, a, b, grad_y):
    """grad_w[out, 16]; difflogic_cuda.backward_w (difflogic_kernel.cu:128-173)."""
    for t, n in ((x, "x"), (a, "a"), (b, "b"), (grad_y, "grad_y")):
        check_input(t, n)
    in_dim, batch = x.shape
    out_dim = grad_y.shape[0]
    gw = torch.empty((out_dim, 16), dtype=x.dtype, device=x.device)
    check(_lib.load().clg_fc_backward_w(dtype_code(x, half_ok=True), x.data_ptr(), a.data_ptr(), b.data_ptr(), grad_y.data_ptr(),
                                        gw.data_ptr(), in_dim, out_dim, batch, stream_ptr(x)))
    return gw


def backward_logits(x, a, b, w, grad_y):
    """Gradient w.r.t. the logits [out, 16] when w = softmax(logits): backward_w and the softmax backward
    in one kernel."""
    for t, n in ((x, "x"), (a, "a"), (b, "b"), (w, "w"), (grad_y, "grad_y")):
        check_input(t, n)
    in_dim, batch = x.shape
    out_dim = grad_y.shape[0]
    gl = torch.empty((out_dim, 16), dtype=x.dtype, device=x.device)
    check(_lib.load().clg_fc_backward_logits(dtype_code(x), x.data_ptr(), a.data_ptr(), b.data_ptr(), w.data_ptr(),
                                             grad_y.data_ptr(), gl.data_ptr(), in_dim, out_dim, batch, stream_ptr(x)))
    return gl


def fold(w_in, from_logits, want_probs=True):
    """[out, 16] logits or probabilities -> (probabilities or None, folded coefficients [out, 4])."""
    check_input(w_in, "w")
    out_dim = w_in.shape[0]
    probs = torch.empty_like(w_in) if want_probs else None
    folded = torch.empty((out_dim, 4), dtype=w_in.dtype, device=w_in.device)
    check(_lib.load().clg_fc_fold(dtype_code(w_in), int(bool(from_logits)), w_in.data_ptr(),
                                  probs.data_ptr() if want_probs else 0, folded.data_ptr(), out_dim, stream_ptr(w_in)))
    return probs, folded


def forward_folded(x, a, b, folded):
    """forward() with the folded coefficients [out, 4] of fold() in place of w."""
    for t, n in ((x, "x"), (a, "a"), (b, "b"), (folded, "folded")):
        check_input(t, n)
    in_dim, batch = x.shape
    out_dim = folded.shape[0]
    y = torch.empty((out_dim, batch), dtype=x.dtype, device=x.device)
    check(_lib.load().clg_fc_forward_folded(dtype_code(x), x.data_ptr(), a.data_ptr(), b.data_ptr(), folded.data_ptr(),
                                            y.data_ptr(), in_dim, out_dim, batch, stream_ptr(x)))
    return y


def forward_logits(x, a, b, logits):
    """fold(from_logits=True) + forward_folded() in one launch -> (y [out, B], probs [out, 16], folded [out, 4])."""
    for t, n in ((x, "x"), (a, "a"), (b, "b"), (logits, "w")):
        check_input(t, n)
    if logits.dim() != 2 or logits.shape[1] != 16 or logits.dtype != x.dtype or x.dtype not in _lib._DTYPES:
        raise RuntimeError(f"forward_logits expects float32/float64 logits [out, 16] of x's dtype, got {tuple(logits.shape)} {logits.dtype}")
    in_dim, batch = x.shape
    out_dim = logits.shape[0]
    y = torch.empty((out_dim, batch), dtype=x.dtype, device=x.device)
    probs = torch.empty_like(logits)
    folded = torch.empty((out_dim, 4), dtype=x.dtype, device=x.device)
    check(_lib.load().clg_fc_forward_logits(dtype_code(x), x.data_ptr(), a.data_ptr(), b.data_ptr(), logits.data_ptr(),
                                            probs.data_ptr(), folded.data_ptr(), y.data_ptr(), in_dim, out_dim, batch,
                                            stream_ptr(x)))
    return y, probs, folded


def backward_x_folded(x, a, b, folded, grad_y, given_x_indices_of_y_start, given_x_indices_of_y):
    """backward_x() with the folded coefficients [out, 4] of fold() in place of w."""
    for t, n in ((x, "x"), (a, "a"), (b, "b"), (folded, "folded"), (grad_y, "grad_y"),
                 (given_x_indices_of_y_start, "given_x_indices_of_y_start"), (given_x_indices_of_y, "given_x_indices_of_y")):
        check_input(t, n)
    in_dim, batch = x.shape
    out_dim = folded.shape[0]
    gx = torch.empty_like(x)
    check(_lib.load().clg_fc_backward_x_folded(dtype_code(x), x.data_ptr(), a.data_ptr(), b.data_ptr(), folded.data_ptr(),
                                               grad_y.data_ptr(), given_x_indices_of_y_start.data_ptr(),
                                               given_x_indices_of_y.data_ptr(), gx.data_ptr(), in_dim, out_dim, batch,
                                               stream_ptr(x)))
    return gx


def backward_sole(x, a, b, folded, probs, grad_y):
    """(grad_x, grad_w) in one pass for a layer whose inputs are each read by exactly one neuron operand; grad_w is
    the gradient w.r.t. the logits when probs = softmax(logits) is given, else w.r.t. the probabilities."""
    for t, n in ((x, "x"), (a, "a"), (b, "b"), (folded, "folded"), (grad_y, "grad_y")):
        check_input(t, n)
    if probs is not None:
        check_input(probs, "w")
    in_dim, batch = x.shape
    out_dim = folded.shape[0]
    gx = torch.empty_like(x)
    gw = torch.empty((out_dim, 16), dtype=x.dtype, device=x.device)
    check(_lib.load().clg_fc_backward_sole(dtype_code(x), x.data_ptr(), a.data_ptr(), b.data_ptr(), folded.data_ptr(),
                                           probs.data_ptr() if probs is not None else 0, grad_y.data_ptr(), gx.data_ptr(),
                                           gw.data_ptr(), in_dim, out_dim, batch, stream_ptr(x)))
    return gx, gw


def backward_fused_fits(x):
    """True when backward_fused() covers the batch of feature-major x [in, B] in one pass."""
    return bool(_lib.load().clg_fc_backward_fused_fits(dtype_code(x), x.shape[1]))


def backward_fused(x, a, b, folded, probs, grad_y, given_x_indices_of_y_start, given_x_indices_of_y):
    """(grad_x, grad_w) of a layer with any wiring in one pass (see backward_fused_fits); grad_w is the gradient
    w.r.t. the logits when probs = softmax(logits) is given, else w.r.t. the probabilities.  Same values as
    backward_x_folded() + backward_w() / backward_logits()."""
    for t, n in ((x, "x"), (a, "a"), (b, "b"), (folded, "folded"), (grad_y, "grad_y"),
                 (given_x_indices_of_y_start, "given_x_indices_of_y_start"), (given_x_indices_of_y, "given_x_indices_of_y")):
        check_input(t, n)
    if probs is not None:
        check_input(probs, "w")
    in_dim, batch = x.shape
    out_dim = folded.shape[0]
    gx = torch.empty_like(x)
    gw = torch.empty((out_dim, 16), dtype=x.dtype, device=x.device)
    check(_lib.load().clg_fc_backward_fused(dtype_code(x), x.data_ptr(), a.data_ptr(), b.data_ptr(), folded.data_ptr(),
                                            probs.data_ptr() if probs is not None else None, grad_y.data_ptr(),
                                            given_x_indices_of_y_start.data_ptr(), given_x_indices_of_y.data_ptr(),
                                            gx.data_ptr(), gw.data_ptr(), in_dim, out_dim, batch, stream_ptr(x)))
    return gx, gw


def group_sum(x_fm, k, tau=1.0):
    """Feature-major activations [F, B] -> per-class sums [B, k] divided by tau, fixed summation order."""
    check_input(x_fm, "x")
    features, batch = x_fm.shape
    if features % k != 0:
        raise ValueError(f"in_dim ({features}) has to be divisible by k ({k}) but it is not")
    lib = _lib.load()
    dt = dtype_code(x_fm)
    nbytes = lib.clg_group_sum_scratch_bytes(dt, features, batch, k)
    scratch = torch.empty((max(int(nbytes), 8),), dtype=torch.uint8, device=x_fm.device)
    out = torch.empty((batch, k), dtype=x_fm.dtype, device=x_fm.device)
    check(lib.clg_group_sum(dt, x_fm.data_ptr(), out.data_ptr(), scratch.data_ptr(), features, batch, k, float(tau), stream_ptr(x_fm)))
    return out


def group_sum_backward(grad_out, features, tau=1.0):
    """[B, k] -> feature-major gradient [F, B]: every row of class g receives grad_out[:, g] / tau."""
    check_input(grad_out, "grad_out")
    batch, k = grad_out.shape
    gx = torch.empty((features, batch), dtype=grad_out.dtype, device=grad_out.device)
    check(_lib.load().clg_group_sum_backward(dtype_code(grad_out), grad_out.data_ptr(), gx.data_ptr(), features, batch, k,
                                             float(tau), stream_ptr(grad_out)))
    return gx


def backward_x(x, a, b, w, grad_y, given_x_indices_of_y_start, given_x_indices_of_y):
    """grad_x[in, B]; difflogic_cuda.backward_x (difflogic_kernel.cu:232-269)."""
    for t, n in ((x, "x"), (a, "a"), (b, "b"), (w, "w"), (grad_y, "grad_y"),
                 (given_x_indices_of_y_start, "given_x_indices_of_y_start"), (given_x_indices_of_y, "given_x_indices_of_y")):
        check_input(t, n)
    in_dim, batch = x.shape
    out_dim = w.shape[0]
    gx = torch.empty_like(x)
    check(_lib.load().clg_fc_backward_x(dtype_code(x, half_ok=True), x.data_ptr(), a.data_ptr(), b.data_ptr(), w.data_ptr(),
                                        grad_y.data_ptr(), given_x_indices_of_y_start.data_ptr(),
                                        given_x_indices_of_y.data_ptr(), gx.data_ptr(), in_dim, out_dim, batch, stream_ptr(x)))
    return gx


def transpose(x):
    """Contiguous transposed copy of a 2-D tensor through the tiled HIP transpose."""
    check_input(x, "x")
    rows, cols = x.shape
    out = torch.empty((cols, rows), dtype=x.dtype, device=x.device)
    if out.numel():
        check(_lib.load().clg_transpose_2d(x.element_size(), x.data_ptr(), out.data_ptr(), rows, cols, stream_ptr(x)))
    return out


def eval(x, a, b, w):  # noqa: A001 - name of the reference binding
    """Packed-bit layer evaluation; difflogic_cuda.eval (difflogic_kernel.cu:295-330).
    x: integer words [in, W]; w: uint8 gate ids [out]."""
    for t, n in ((x, "x"), (a, "a"), (b, "b"), (w, "w")):
        check_input(t, n)
    if x.dtype not in _WORD_DTYPE.values() or w.dtype != torch.uint8:
        raise RuntimeError("eval expects int8/16/32/64 words and uint8 gate ids")
    in_dim, words = x.shape
    out_dim = w.shape[0]
    y = torch.empty((out_dim, words), dtype=x.dtype, device=x.device)
    check(_lib.load().clg_fc_eval_packed(x.element_size(), x.data_ptr(), a.data_ptr(), b.data_ptr(), w.data_ptr(),
                                         y.data_ptr(), in_dim, out_dim, words, stream_ptr(x)))
    return y


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
    for t, n in ((x, "x"), (a, "a"), (b, "b"), (w, "w"), (plan, "plan")):
        check_input(t, n)
    if x.dtype not in _WORD_DTYPE.values() or w.dtype != torch.uint8 or plan.dtype != torch.int32:
        raise RuntimeError("eval_planned expects int8/16/32/64 words, uint8 gate ids and an int32 plan")
    in_dim, words = x.shape
    out_dim = w.shape[0]
    if plan.shape[0] != out_dim:
        raise RuntimeError("plan does not match the number of neurons")
    y = torch.empty((out_dim, words), dtype=x.dtype, device=x.device)
    check(_lib.load().clg_fc_eval_packed_planned(x.element_size(), x.data_ptr(), a.data_ptr(), b.data_ptr(), w.data_ptr(),
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
    features, words = b.shape
    if features % k != 0:
        raise ValueError(f"in_dim ({features}) has to be divisible by k ({k}) but it is not")
    samples = words * 8 * b.element_size() - pad_len
    out = torch.empty((samples, k), dtype=torch.int32, device=b.device)
    check(_lib.load().clg_group_bit_sum(b.element_size(), b.data_ptr(), out.data_ptr(), features, words, pad_len, k,
                                        stream_ptr(b)))
    return out
