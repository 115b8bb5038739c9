"""Function set of the reference's `convlogic_cuda` module (src/convlogic/cuda/convlogic.cpp:29-44)
on top of the HIP C ABI."""
import ctypes

import torch

from . import _lib
from ._lib import ConvGeom, check, check_input, dtype_code, stream_ptr


def _geom(x, c_out, stride_h, stride_w, pad_h, pad_w, kernel_h, kernel_w):
    n, c_in, h, w = x.shape
    return ConvGeom(n, c_in, h, w, c_out, stride_h, stride_w, pad_h, pad_w, kernel_h, kernel_w)


def _geom_from_out(x, c_out, ho, wo, stride_h, stride_w, pad_h, pad_w):
    """The backward bindings of the reference do not receive the kernel size; any kernel size that
    reproduces the conv output size describes the same index arithmetic."""
    _, _, h, w = x.shape
    return _geom(x, c_out, stride_h, stride_w, pad_h, pad_w, h + 2 * pad_h - (ho - 1) * stride_h, w + 2 * pad_w - (wo - 1) * stride_w)


def _out_size(g):
    return (g.h + 2 * g.pad_h - g.kernel_h) // g.stride_h + 1, (g.w + 2 * g.pad_w - g.kernel_w) // g.stride_w + 1


def _conv_args(x, weight, selection, gates):
    """x [N, C_in, H, W] float, weight [C, gates, 16] of x's dtype, selection int32 [C, 8]: everything on x's device."""
    check_input(x, "x")
    if x.dim() != 4:
        raise RuntimeError(f"Expected x to be 4D (N, C, H, W), but got {x.dim()}")
    c = weight.shape[0] if weight.dim() else -1
    check_input(weight, "weights", x.dtype, (c, gates, 16))
    _selection_arg(x, selection, c)
    _lib.check_same_device(x, weight)


def _selection_arg(x, selection, c):
    check_input(selection, "selection", torch.int32, (c, 8))
    _lib.check_same_device(x, selection)


def _grad_args(grad_y, x, shape):
    check_input(grad_y, "grad_y", x.dtype, shape)
    _lib.check_same_device(x, grad_y)


def _block_grad_args(grad_y, x, weight, argmax, selection, feature_major=False):
    """Arguments of the fused block's backward entry points: grad_y [N, C, Ho/2, Wo/2] (or [C, Ho/2, Wo/2, N]) of x's
    dtype, argmax uint8 [N, C, Ho/2, Wo/2] with codes 0..3, weights [C, 7, 16], selection int32 [C, 8]."""
    _conv_args(x, weight, selection, 7)
    if grad_y.dim() != 4:
        raise RuntimeError(f"Expected grad_y to be 4D, but got {grad_y.dim()}")
    n, c = x.shape[0], weight.shape[0]
    hp, wp = (grad_y.shape[1], grad_y.shape[2]) if feature_major else (grad_y.shape[2], grad_y.shape[3])
    _grad_args(grad_y, x, (c, hp, wp, n) if feature_major else (n, c, hp, wp))
    check_input(argmax, "argmax", torch.uint8, (n, c, hp, wp))
    _lib.check_same_device(x, argmax)


def _scratch(nbytes, device):
    if nbytes < 0:
        raise RuntimeError(_lib.load().clg_last_error().decode())
    return torch.empty((max(int(nbytes), 8),), dtype=torch.uint8, device=device)


# ---- split layer ------------------------------------------------------------------------------
def convlogic_forward(x, weight, selection, stride_h, stride_w, pad_h, pad_w, kernel_h, kernel_w):
    """[N,C,Ho,Wo,4]; src/convlogic/cuda/convlogic_kernel.cu:67-106."""
    _conv_args(x, weight, selection, 4)
    g = _geom(x, weight.shape[0], stride_h, stride_w, pad_h, pad_w, kernel_h, kernel_w)
    ho, wo = _out_size(g)
    y = torch.empty((g.n, g.c_out, max(ho, 0), max(wo, 0), 4), dtype=x.dtype, device=x.device)
    check(_lib.load().clg_conv4_forward(dtype_code(x), ctypes.byref(g), x.data_ptr(), weight.data_ptr(), selection.data_ptr(),
                                        y.data_ptr(), stream_ptr(x)))
    return y


def convlogic_backward_x(grad_y, x, weight, selection, stride_h, stride_w, pad_h, pad_w):
    """src/convlogic/cuda/convlogic_kernel.cu:321-359 (deterministic here)."""
    _conv_args(x, weight, selection, 4)
    if grad_y.dim() != 5:
        raise RuntimeError(f"Expected grad_y to be 5D (N, C, Ho, Wo, 4), but got {grad_y.dim()}")
    _grad_args(grad_y, x, (x.shape[0], weight.shape[0], grad_y.shape[2], grad_y.shape[3], 4))
    g = _geom_from_out(x, grad_y.shape[1], grad_y.shape[2], grad_y.shape[3], stride_h, stride_w, pad_h, pad_w)
    gx = torch.empty_like(x)
    check(_lib.load().clg_conv4_backward_x(dtype_code(x), ctypes.byref(g), grad_y.data_ptr(), x.data_ptr(), weight.data_ptr(),
                                           selection.data_ptr(), gx.data_ptr(), stream_ptr(x)))
    return gx


def convlogic_backward_weight(grad_y, x, selection, stride_h, stride_w, pad_h, pad_w):
    """[C,4,16]; src/convlogic/cuda/convlogic_kernel.cu:197-248."""
    check_input(x, "x")
    if x.dim() != 4 or grad_y.dim() != 5:
        raise RuntimeError(f"Expected x 4D and grad_y 5D (N, C, Ho, Wo, 4), but got {x.dim()} and {grad_y.dim()}")
    _grad_args(grad_y, x, (x.shape[0], grad_y.shape[1], grad_y.shape[2], grad_y.shape[3], 4))
    _selection_arg(x, selection, grad_y.shape[1])
    g = _geom_from_out(x, grad_y.shape[1], grad_y.shape[2], grad_y.shape[3], stride_h, stride_w, pad_h, pad_w)
    lib = _lib.load()
    dt = dtype_code(x)
    scratch = _scratch(lib.clg_conv4_backward_w_scratch_bytes(dt, ctypes.byref(g)), x.device)
    gw = torch.empty((g.c_out, 4, 16), dtype=x.dtype, device=x.device)
    check(lib.clg_conv4_backward_w(dt, ctypes.byref(g), grad_y.data_ptr(), x.data_ptr(), selection.data_ptr(), gw.data_ptr(),
                                   scratch.data_ptr(), stream_ptr(x)))
    return gw


# ---- tree level -------------------------------------------------------------------------------
def _tree_dims(x, xo):
    if x.dim() != 5:
        raise RuntimeError(f"Expected input tensor x to be 5D (N, C, H, W, 2*Xout), but got {x.dim()}")
    n, c, h, w, xin = x.shape
    if xin != 2 * xo:
        raise RuntimeError(f"Expected input x.size(4) (Xin) to equal 2*Xout ({2 * xo}), but got {xin}")
    return n, c, h * w


def treelogic_forward(x, weights):
    """[N,C,H,W,Xout]; src/convlogic/cuda/treelogic_kernel.cu:46-85."""
    check_input(x, "x")
    xo = weights.shape[1] if weights.dim() == 3 else -1
    n, c, pos = _tree_dims(x, xo)
    check_input(weights, "weights", x.dtype, (c, xo, 16))
    y = torch.empty(x.shape[:4] + (xo,), dtype=x.dtype, device=x.device)
    if y.numel():
        check(_lib.load().clg_tree_forward(dtype_code(x), x.data_ptr(), weights.data_ptr(), y.data_ptr(), n, c, pos, xo,
                                           stream_ptr(x)))
    return y


def treelogic_backward_x(grad_y, x, weights):
    """src/convlogic/cuda/treelogic_kernel.cu:252-285."""
    check_input(x, "x")
    xo = weights.shape[1] if weights.dim() == 3 else -1
    n, c, pos = _tree_dims(x, xo)
    check_input(weights, "weights", x.dtype, (c, xo, 16))
    check_input(grad_y, "grad_y", x.dtype, tuple(x.shape[:4]) + (xo,))
    gx = torch.empty_like(x)
    if gx.numel():
        check(_lib.load().clg_tree_backward_x(dtype_code(x), grad_y.data_ptr(), x.data_ptr(), weights.data_ptr(), gx.data_ptr(),
                                              n, c, pos, xo, stream_ptr(x)))
    return gx


def treelogic_backward_weight(grad_y, x):
    """[C,Xout,16]; src/convlogic/cuda/treelogic_kernel.cu:160-206."""
    check_input(x, "x")
    xo = grad_y.shape[4] if grad_y.dim() == 5 else -1
    n, c, pos = _tree_dims(x, xo)
    check_input(grad_y, "grad_y", x.dtype, tuple(x.shape[:4]) + (xo,))
    lib = _lib.load()
    dt = dtype_code(x)
    scratch = _scratch(lib.clg_tree_backward_w_scratch_bytes(dt, n, c, pos, xo), x.device)
    gw = torch.empty((c, xo, 16), dtype=x.dtype, device=x.device)
    check(lib.clg_tree_backward_w(dt, grad_y.data_ptr(), x.data_ptr(), gw.data_ptr(), scratch.data_ptr(), n, c, pos, xo,
                                  stream_ptr(x)))
    return gw


# ---- fused block ------------------------------------------------------------------------------
def full_convlogic_forward(x, weight, selection, stride_h, stride_w, pad_h, pad_w, kernel_h, kernel_w):
    """-> (y [N,C,Ho/2,Wo/2], argmax uint8 [N,C,Ho/2,Wo/2] = dy*2+dx of the pooled maximum).
    src/convlogic/cuda/full_convlogic_kernel.cu:147-231; the leaf / middle gate planes the reference
    also returns are not materialised (see full_convlogic_intermediates)."""
    _conv_args(x, weight, selection, 7)
    g = _geom(x, weight.shape[0], stride_h, stride_w, pad_h, pad_w, kernel_h, kernel_w)
    ho, wo = _out_size(g)
    shape = (g.n, g.c_out, max(ho, 0) // 2, max(wo, 0) // 2)
    y = torch.empty(shape, dtype=x.dtype, device=x.device)
    argmax = torch.empty(shape, dtype=torch.uint8, device=x.device)
    lib = _lib.load()
    scratch = _scratch(lib.clg_convblock_forward_scratch_bytes(dtype_code(x), ctypes.byref(g)), x.device)
    check(lib.clg_convblock_forward_ws(dtype_code(x), ctypes.byref(g), x.data_ptr(), weight.data_ptr(), selection.data_ptr(),
                                       y.data_ptr(), argmax.data_ptr(), scratch.data_ptr() if scratch is not None else None,
                                       stream_ptr(x)))
    return y, argmax


def full_convlogic_eval_packed(x, gates, selection, stride_h, stride_w, pad_h, pad_w, kernel_h, kernel_w, feature_major=False):
    """Packed-bit inference of the fused block.  x: int64 words [G, C_in, H, W], 64 samples per word
    (bit s of group g = sample 64 g + s); gates: uint8 [C, 7] arg-max gate ids; -> int64 [G, C, Ho/2, Wo/2].
    Equals the eval-mode float block on binary inputs (src/convlogic/convlogic_layer.py:231-316,321-325);
    the reference has no packed conv kernel.  feature_major: where the kernels can (4x4 images, at least 32
    groups), the result is the [G, C, Ho/2, Wo/2] VIEW of a contiguous [C, Ho/2, Wo/2, G] tensor -- the layout
    PackBitsTensor.flatten() needs, which then takes a view instead of transposing."""
    check_input(x, "x")
    check_input(gates, "gates")
    if x.dtype != torch.int64 or gates.dtype != torch.uint8 or x.dim() != 4:
        raise RuntimeError("full_convlogic_eval_packed expects int64 words [G, C, H, W] and uint8 gate ids [C, 7]")
    if gates.dim() != 2 or gates.shape[1] != 7:
        raise RuntimeError(f"full_convlogic_eval_packed expects gate ids of shape [C, 7], got {tuple(gates.shape)}")
    _selection_arg(x, selection, gates.shape[0])
    _lib.check_same_device(x, gates)
    g = _geom(x, gates.shape[0], stride_h, stride_w, pad_h, pad_w, kernel_h, kernel_w)
    ho, wo = _out_size(g)
    lib = _lib.load()
    if feature_major and lib.clg_convblock_eval_packed_fm_supported(ctypes.byref(g)):
        y = torch.empty((g.c_out, ho // 2, wo // 2, g.n), dtype=torch.int64, device=x.device)
        check(lib.clg_convblock_eval_packed_fm(ctypes.byref(g), x.data_ptr(), gates.data_ptr(), selection.data_ptr(), y.data_ptr(),
                                               stream_ptr(x)))
        return y.permute(3, 0, 1, 2)
    y = torch.empty((g.n, g.c_out, max(ho, 0) // 2, max(wo, 0) // 2), dtype=torch.int64, device=x.device)
    scratch = _scratch(lib.clg_convblock_eval_packed_scratch_bytes(ctypes.byref(g)), x.device)
    check(lib.clg_convblock_eval_packed_ws(ctypes.byref(g), x.data_ptr(), gates.data_ptr(), selection.data_ptr(), y.data_ptr(),
                                           scratch.data_ptr() if scratch is not None else None, stream_ptr(x)))
    return y


def full_convlogic_intermediates(x, weight, selection, stride_h, stride_w, pad_h, pad_w, kernel_h, kernel_w):
    """-> (x2 [N,C,Ho,Wo,4], x3 [N,C,Ho,Wo,2]), the second and third result of the reference's
    full_convlogic_forward (full_convlogic_kernel.cu:172,194)."""
    _conv_args(x, weight, selection, 7)
    g = _geom(x, weight.shape[0], stride_h, stride_w, pad_h, pad_w, kernel_h, kernel_w)
    ho, wo = _out_size(g)
    x2 = torch.empty((g.n, g.c_out, ho, wo, 4), dtype=x.dtype, device=x.device)
    x3 = torch.empty((g.n, g.c_out, ho, wo, 2), dtype=x.dtype, device=x.device)
    check(_lib.load().clg_convblock_intermediates(dtype_code(x), ctypes.byref(g), x.data_ptr(), weight.data_ptr(),
                                                  selection.data_ptr(), x2.data_ptr(), x3.data_ptr(), stream_ptr(x)))
    return x2, x3


def argmax_to_indices(argmax, wo):
    """uint8 window codes -> the reference's int32 indices in_y*Wo + in_x, [N,C,I]
    (full_convlogic_kernel.cu:138,144)."""
    n, c, hp, wp = argmax.shape
    code = argmax.to(torch.int32)
    py = torch.arange(hp, device=argmax.device, dtype=torch.int32).view(1, 1, hp, 1)
    px = torch.arange(wp, device=argmax.device, dtype=torch.int32).view(1, 1, 1, wp)
    idx = (2 * py + (code >> 1)) * wo + 2 * px + (code & 1)
    return idx.reshape(n, c, hp * wp)


def full_convlogic_backward_x(grad_y, x, weight, argmax, selection, stride_h, stride_w, pad_h, pad_w):
    """src/convlogic/cuda/full_convlogic_kernel.cu:365-461 (deterministic here)."""
    _block_grad_args(grad_y, x, weight, argmax, selection)
    g = _geom_from_out(x, grad_y.shape[1], 2 * grad_y.shape[2], 2 * grad_y.shape[3], stride_h, stride_w, pad_h, pad_w)
    lib = _lib.load()
    dt = dtype_code(x)
    scratch = _scratch(lib.clg_convblock_backward_x_scratch_bytes(dt, ctypes.byref(g)), x.device)
    gx = torch.empty_like(x)
    check(lib.clg_convblock_backward_x(dt, ctypes.byref(g), grad_y.data_ptr(), x.data_ptr(), weight.data_ptr(),
                                       selection.data_ptr(), argmax.data_ptr(), gx.data_ptr(), scratch.data_ptr(), stream_ptr(x)))
    return gx


def full_convlogic_backward_weight(grad_y, x, weight, argmax, selection, stride_h, stride_w, pad_h, pad_w):
    """[C,7,16]; src/convlogic/cuda/full_convlogic_kernel.cu:616-701."""
    _block_grad_args(grad_y, x, weight, argmax, selection)
    g = _geom_from_out(x, grad_y.shape[1], 2 * grad_y.shape[2], 2 * grad_y.shape[3], stride_h, stride_w, pad_h, pad_w)
    lib = _lib.load()
    dt = dtype_code(x)
    scratch = _scratch(lib.clg_convblock_backward_w_scratch_bytes(dt, ctypes.byref(g)), x.device)
    gw = torch.empty((g.c_out, 7, 16), dtype=x.dtype, device=x.device)
    check(lib.clg_convblock_backward_w(dt, ctypes.byref(g), grad_y.data_ptr(), x.data_ptr(), weight.data_ptr(),
                                       selection.data_ptr(), argmax.data_ptr(), gw.data_ptr(), scratch.data_ptr(), stream_ptr(x)))
    return gw


def full_convlogic_backward(grad_y, x, weight, argmax, selection, stride_h, stride_w, pad_h, pad_w):
    """-> (grad_x, grad_w [C,7,16]) in one call (the pair of calls of
    src/convlogic/convlogic_layer.py:76-81, one scratch buffer, one transition into the library)."""
    _block_grad_args(grad_y, x, weight, argmax, selection)
    g = _geom_from_out(x, grad_y.shape[1], 2 * grad_y.shape[2], 2 * grad_y.shape[3], stride_h, stride_w, pad_h, pad_w)
    lib = _lib.load()
    dt = dtype_code(x)
    scratch = _scratch(lib.clg_convblock_backward_scratch_bytes(dt, ctypes.byref(g)), x.device)
    gx = torch.empty_like(x)
    gw = torch.empty((g.c_out, 7, 16), dtype=x.dtype, device=x.device)
    check(lib.clg_convblock_backward(dt, ctypes.byref(g), grad_y.data_ptr(), x.data_ptr(), weight.data_ptr(), selection.data_ptr(),
                                     argmax.data_ptr(), gx.data_ptr(), gw.data_ptr(), scratch.data_ptr(), stream_ptr(x)))
    return gx, gw


def full_convlogic_backward_logits(grad_y, x, weight, argmax, selection, stride_h, stride_w, pad_h, pad_w, need_grad_x=True, validate=True):
    """-> (grad_x or None, grad_logits [C,7,16]) for weight = softmax(logits): the two gradients of the block
    with the softmax backward fused into the final reduction of the weight gradient."""
    if validate:
        _block_grad_args(grad_y, x, weight, argmax, selection)
    g = _geom_from_out(x, grad_y.shape[1], 2 * grad_y.shape[2], 2 * grad_y.shape[3], stride_h, stride_w, pad_h, pad_w)
    lib = _lib.load()
    dt = dtype_code(x)
    scratch = _scratch(lib.clg_convblock_backward_scratch_bytes(dt, ctypes.byref(g)), x.device)
    gx = torch.empty_like(x) if need_grad_x else None
    gl = torch.empty((g.c_out, 7, 16), dtype=x.dtype, device=x.device)
    check(lib.clg_convblock_backward_logits(dt, ctypes.byref(g), grad_y.data_ptr(), x.data_ptr(), weight.data_ptr(),
                                            selection.data_ptr(), argmax.data_ptr(), gx.data_ptr() if need_grad_x else None,
                                            gl.data_ptr(), scratch.data_ptr(), stream_ptr(x)))
    return gx, gl


def feature_major_supported(x, c_out, stride_h, stride_w, pad_h, pad_w, kernel_h, kernel_w):
    """True when the block on x can write its output feature-major (full_convlogic_forward_fm)."""
    if not (x.is_cuda and x.dim() == 4 and x.dtype in (torch.float32, torch.float64)):
        return False
    g = _geom(x, c_out, stride_h, stride_w, pad_h, pad_w, kernel_h, kernel_w)
    return bool(_lib.load().clg_convblock_fm_supported(dtype_code(x), ctypes.byref(g)))


def full_convlogic_forward_fm(x, weight, selection, stride_h, stride_w, pad_h, pad_w, kernel_h, kernel_w):
    """full_convlogic_forward() with y laid out [C, Ho/2, Wo/2, N] (contiguous); argmax stays [N,C,Ho/2,Wo/2]."""
    _conv_args(x, weight, selection, 7)
    g = _geom(x, weight.shape[0], stride_h, stride_w, pad_h, pad_w, kernel_h, kernel_w)
    ho, wo = _out_size(g)
    y = torch.empty((g.c_out, ho // 2, wo // 2, g.n), dtype=x.dtype, device=x.device)
    argmax = torch.empty((g.n, g.c_out, ho // 2, wo // 2), dtype=torch.uint8, device=x.device)
    lib = _lib.load()
    scratch = _scratch(lib.clg_convblock_forward_scratch_bytes(dtype_code(x), ctypes.byref(g)), x.device)
    check(lib.clg_convblock_forward_fm(dtype_code(x), ctypes.byref(g), x.data_ptr(), weight.data_ptr(), selection.data_ptr(),
                                       y.data_ptr(), argmax.data_ptr(), scratch.data_ptr() if scratch is not None else None,
                                       stream_ptr(x)))
    return y, argmax


def full_convlogic_forward_logits(x, logits, selection, stride_h, stride_w, pad_h, pad_w, kernel_h, kernel_w, feature_major=False,
                                  want_folded=False, validate=True, want_padded=False, prefolded=None):
    """full_convlogic_forward() from the LOGITS [C, 7, 16]: the softmax is taken inside the launch that sets the gate
    parameters up.  -> (y, argmax, probs); with feature_major (where feature_major_supported) y is laid out
    [C, Ho/2, Wo/2, N] as from full_convlogic_forward_fm().  want_folded: -> (y, argmax, probs, folded [C, 7, 4]), the
    folded coefficients of every gate for full_convlogic_backward_planned().  want_padded (with want_folded): a fifth
    result, the zero-padded copy of x that the forward kernels stage anyway and the planned backward pass would otherwise
    make in a launch of its own -- or None where the pair of kernels at this shape has no use for one.  prefolded (with
    want_folded): the (probs, folded) pair that difflogic_hip.fold_many() made from these logits -- the call then launches
    no softmax or fold of its own and returns that pair."""
    if validate:
        _conv_args(x, logits, selection, 7)
    g = _geom(x, logits.shape[0], stride_h, stride_w, pad_h, pad_w, kernel_h, kernel_w)
    ho, wo = _out_size(g)
    shape = (g.n, g.c_out, max(ho, 0) // 2, max(wo, 0) // 2)
    y = torch.empty((g.c_out, shape[2], shape[3], g.n) if feature_major else shape, dtype=x.dtype, device=x.device)
    argmax = torch.empty(shape, dtype=torch.uint8, device=x.device)
    c = logits.shape[0]
    if prefolded is not None and want_folded:
        probs, folded = prefolded
        if validate:
            check_input(probs, "prefolded probabilities", x.dtype, (c, 7, 16))
            check_input(folded, "prefolded coefficients", x.dtype, (c, 7, 4))
        if folded.data_ptr() != probs.data_ptr() + probs.numel() * probs.element_size():
            raise RuntimeError("prefolded: the folded coefficients must follow the probabilities in one buffer (fold_many)")
    elif want_folded:                                                # one buffer: probabilities, then the folded coefficients
        both = torch.empty((c * (112 + 28),), dtype=logits.dtype, device=logits.device)
        probs, folded = both[:c * 112].view(c, 7, 16), both[c * 112:].view(c, 7, 4)
    else:
        probs, folded = torch.empty_like(logits), None
    lib = _lib.load()
    scratch = _scratch(lib.clg_convblock_forward_scratch_bytes(dtype_code(x), ctypes.byref(g)), x.device)
    flags = 1 | (2 if feature_major else 0) | (4 if want_folded else 0) | (8 if prefolded is not None and want_folded else 0)
    padded = None
    if want_padded and want_folded and not feature_major:
        elems = lib.clg_convblock_padded_elems(dtype_code(x), ctypes.byref(g), 1 if scratch is not None else 0)
        if elems > 0:
            padded = torch.empty((elems,), dtype=x.dtype, device=x.device)
    if padded is not None:
        check(lib.clg_convblock_forward_padded(dtype_code(x), ctypes.byref(g), x.data_ptr(), logits.data_ptr(), selection.data_ptr(),
                                               y.data_ptr(), argmax.data_ptr(), probs.data_ptr(), flags,
                                               scratch.data_ptr() if scratch is not None else None, padded.data_ptr(), stream_ptr(x)))
    else:
        check(lib.clg_convblock_forward_ex(dtype_code(x), ctypes.byref(g), x.data_ptr(), logits.data_ptr(), selection.data_ptr(),
                                           y.data_ptr(), argmax.data_ptr(), probs.data_ptr(), flags,
                                           scratch.data_ptr() if scratch is not None else None, stream_ptr(x)))
    if want_padded:
        return y, argmax, probs, folded, padded
    if want_folded:
        return y, argmax, probs, folded
    return y, argmax, probs


def make_backward_plan(x, c_out, selection, stride_h, stride_w, pad_h, pad_w, kernel_h, kernel_w):
    """Per-layer plan of the block's backward pass for inputs of x's shape and dtype: -> (plan bytes on the device,
    signature).  Depends only on the selection and the geometry; built once and reused by every
    full_convlogic_backward_planned() call of the layer (the reverse map the reference's LogicLayer builds at
    construction, src/difflogic/difflogic.py:71-87, for the fused block)."""
    check_input(x, "x")
    if x.dim() != 4:
        raise RuntimeError(f"Expected x to be 4D (N, C, H, W), but got {x.dim()}")
    _selection_arg(x, selection, c_out)
    g = _geom(x, c_out, stride_h, stride_w, pad_h, pad_w, kernel_h, kernel_w)
    lib = _lib.load()
    dt = dtype_code(x)
    plan = _scratch(lib.clg_convblock_plan_bytes(dt, ctypes.byref(g)), x.device)
    sig = ctypes.c_int64(0)
    check(lib.clg_convblock_plan(dt, ctypes.byref(g), selection.data_ptr(), plan.data_ptr(), ctypes.byref(sig), stream_ptr(x)))
    return plan, sig.value


def full_convlogic_backward_planned(grad_y, x, weight, folded, argmax, selection, plan, signature, stride_h, stride_w, pad_h, pad_w,
                                    need_grad_x=True, wrt_logits=True, validate=True, feature_major=False, padded=None, kernel=None):
    """-> (grad_x or None, grad_w [C,7,16]) with the layer's plan from make_backward_plan(): no list building, no reduce
    launch and -- with folded [C, 7, 4] from full_convlogic_forward_logits(want_folded=True) -- no set-up launch for
    blocks whose images fit LDS.  grad_w is the gradient w.r.t. the logits (weight = their softmax) or, with
    wrt_logits=False, w.r.t. the probabilities; feature_major: grad_y is laid out [C, Ho/2, Wo/2, N] (as for
    full_convlogic_backward_fm).  Same values as full_convlogic_backward(_logits / _fm)().  kernel: (kernel_h, kernel_w) the plan
    (and the padded copy) were made with; without it the largest window that gives grad_y's size is taken, which is another one
    where a stride above 1 does not divide the padded image (the plan's signature then refuses the call)."""
    c_out, ho, wo = ((grad_y.shape[0], 2 * grad_y.shape[1], 2 * grad_y.shape[2]) if feature_major     # [C, Ho/2, Wo/2, N]
                     else (grad_y.shape[1], 2 * grad_y.shape[2], 2 * grad_y.shape[3]))
    if kernel is None:
        g = _geom_from_out(x, c_out, ho, wo, stride_h, stride_w, pad_h, pad_w)
    else:
        g = _geom(x, c_out, stride_h, stride_w, pad_h, pad_w, *kernel)
        if _out_size(g) != (ho, wo):
            raise RuntimeError(f"grad_y is the gradient of a {ho // 2} x {wo // 2} pooled image, the geometry gives {_out_size(g)[0] // 2} x {_out_size(g)[1] // 2}")
    lib = _lib.load()
    dt = dtype_code(x)
    if validate:
        _block_grad_args(grad_y, x, weight, argmax, selection, feature_major=feature_major)
        if folded is not None:
            check_input(folded, "folded", x.dtype, (weight.shape[0], 7, 4))
        check_input(plan, "plan", torch.uint8)
        if plan.numel() < lib.clg_convblock_plan_bytes(dt, ctypes.byref(g)):
            raise RuntimeError("plan is smaller than clg_convblock_plan_bytes() for this geometry")
    scratch = _scratch(lib.clg_convblock_backward_scratch_bytes(dt, ctypes.byref(g)), x.device)
    gx = torch.empty_like(x) if need_grad_x else None
    gw = torch.empty((g.c_out, 7, 16), dtype=x.dtype, device=x.device)
    flags = (1 if wrt_logits else 0) | (2 if feature_major else 0)
    if padded is not None and need_grad_x:
        # the padded copy of x that full_convlogic_forward_logits(want_padded=True) left: no launch to make one
        if validate:
            check_input(padded, "padded", x.dtype, (lib.clg_convblock_padded_elems(dt, ctypes.byref(g), 1),))
        check(lib.clg_convblock_backward_planned_padded(dt, ctypes.byref(g), grad_y.data_ptr(), x.data_ptr(), weight.data_ptr(),
                                                        folded.data_ptr() if folded is not None else None, padded.data_ptr(),
                                                        selection.data_ptr(), argmax.data_ptr(), plan.data_ptr(), signature, gx.data_ptr(),
                                                        gw.data_ptr(), flags, scratch.data_ptr(), stream_ptr(x)))
        return gx, gw
    check(lib.clg_convblock_backward_planned(dt, ctypes.byref(g), grad_y.data_ptr(), x.data_ptr(), weight.data_ptr(),
                                             folded.data_ptr() if folded is not None else None, selection.data_ptr(), argmax.data_ptr(),
                                             plan.data_ptr(), signature, gx.data_ptr() if need_grad_x else None, gw.data_ptr(),
                                             flags, scratch.data_ptr(), stream_ptr(x)))
    return gx, gw


def full_convlogic_backward_fm(grad_y_fm, x, weight, argmax, selection, stride_h, stride_w, pad_h, pad_w, need_grad_x=True,
                               wrt_logits=True, validate=True):
    """-> (grad_x or None, grad_w [C,7,16]) from grad_y laid out [C, Ho/2, Wo/2, N]; grad_w is the gradient w.r.t. the
    logits (weight = their softmax) or, with wrt_logits=False, w.r.t. the probabilities."""
    if validate:
        _block_grad_args(grad_y_fm, x, weight, argmax, selection, feature_major=True)
    g = _geom_from_out(x, grad_y_fm.shape[0], 2 * grad_y_fm.shape[1], 2 * grad_y_fm.shape[2], stride_h, stride_w, pad_h, pad_w)
    lib = _lib.load()
    dt = dtype_code(x)
    scratch = _scratch(lib.clg_convblock_backward_scratch_bytes(dt, ctypes.byref(g)), x.device)
    gx = torch.empty_like(x) if need_grad_x else None
    gw = torch.empty((g.c_out, 7, 16), dtype=x.dtype, device=x.device)
    check(lib.clg_convblock_backward_fm(dt, ctypes.byref(g), grad_y_fm.data_ptr(), x.data_ptr(), weight.data_ptr(),
                                        selection.data_ptr(), argmax.data_ptr(), gx.data_ptr() if need_grad_x else None,
                                        gw.data_ptr(), 1 if wrt_logits else 0, scratch.data_ptr(), stream_ptr(x)))
    return gx, gw


# ---- input binarisation -------------------------------------------------------------------------
def _threshold_args(x, thresholds):
    check_input(x, "x")
    check_input(thresholds, "thresholds")
    if x.dtype != torch.float32 or thresholds.dtype != torch.float32 or x.dim() != 4 or thresholds.dim() != 1:
        raise RuntimeError("expected float32 images [N, C, H, W] and float32 thresholds [L]")
    n, c0, h, w = x.shape
    return n, c0, h, w, thresholds.shape[0]


def threshold_images(x, thresholds):
    """float32 [N, C, H, W] -> float32 {0,1} [N, L*C, H, W], channel l*C + c = x[:, c] > thresholds[l]
    (src/convlogic/data.py:46-50 on a batch)."""
    n, c0, h, w, levels = _threshold_args(x, thresholds)
    out = torch.empty((n, levels * c0, h, w), dtype=torch.float32, device=x.device)
    if out.numel():
        check(_lib.load().clg_threshold_images(x.data_ptr(), thresholds.data_ptr(), out.data_ptr(), n, c0, h * w, levels,
                                               stream_ptr(x)))
    return out


def threshold_pack_images(x, thresholds):
    """float32 [N, C, H, W] -> (int64 words [ceil(N/64), L*C, H, W], pad_len): the thresholded channels
    packed 64 samples per word, group-major, without materialising them as floats."""
    n, c0, h, w, levels = _threshold_args(x, thresholds)
    groups = -(-n // 64)
    out = torch.empty((groups, levels * c0, h, w), dtype=torch.int64, device=x.device)
    if out.numel():
        check(_lib.load().clg_threshold_pack_images(x.data_ptr(), thresholds.data_ptr(), out.data_ptr(), n, c0, h * w, levels,
                                                    stream_ptr(x)))
    return out, groups * 64 - n


# ---- fused block on binary inputs ---------------------------------------------------------------
def bin_supported(x, c_out, stride_h, stride_w, pad_h, pad_w, kernel_h, kernel_w):
    """True when the binary-input kernels take a block on x (float32, stride 1, at most 32 columns, at most 256 pooled
    cells per plane)."""
    if not (x.is_cuda and x.dim() == 4 and x.dtype == torch.float32):
        return False
    g = _geom(x, c_out, stride_h, stride_w, pad_h, pad_w, kernel_h, kernel_w)
    return bool(_lib.load().clg_convblock_bin_supported(dtype_code(x), ctypes.byref(g)))


class BinaryFlag:
    """One int32 in pinned host memory that the kernels set when an input promised to be binary is not: the host reads
    it without a copy or a synchronisation (a violation therefore shows at the next check after the launch has run)."""

    def __init__(self):
        self.host = torch.zeros(1, dtype=torch.int32).pin_memory()
        dev = ctypes.c_void_p(0)
        check(_lib.load().clg_host_flag_device_pointer(self.host.data_ptr(), ctypes.byref(dev)))
        self.device_ptr = dev.value

    def __deepcopy__(self, memo):                                    # a copied layer gets a flag of its own
        return BinaryFlag()

    def __reduce__(self):
        return (BinaryFlag, ())

    def raised(self):
        return bool(self.host[0].item())

    def clear(self):
        self.host.zero_()


def bin_forward(x, w, selection, stride_h, stride_w, pad_h, pad_w, kernel_h, kernel_w, flag, logits=False, validate=True):
    """Fused block on binary x (every element 0 or 1) -> (y [N,C,Ho/2,Wo/2], taps uint16 [N,C,Ho/2,Wo/2] = arg-max code
    << 8 | tap byte, ctx: the buffer the backward call needs).  w: probabilities, or the logits with logits=True.
    y and the arg-max equal full_convlogic_forward() bit for bit.  flag: a BinaryFlag, set when x is not binary."""
    if validate:
        _conv_args(x, w, selection, 7)
    g = _geom(x, w.shape[0], stride_h, stride_w, pad_h, pad_w, kernel_h, kernel_w)
    lib = _lib.load()
    dt = dtype_code(x)
    ctx = _scratch(lib.clg_convblock_bin_ctx_bytes(dt, ctypes.byref(g)), x.device)
    ho, wo = _out_size(g)
    shape = (g.n, g.c_out, ho // 2, wo // 2)
    y = torch.empty(shape, dtype=x.dtype, device=x.device)
    taps = torch.empty(shape, dtype=torch.int16, device=x.device)
    check(lib.clg_convblock_bin_forward(dt, ctypes.byref(g), x.data_ptr(), w.data_ptr(), selection.data_ptr(), y.data_ptr(),
                                        taps.data_ptr(), ctx.data_ptr(), 1 if logits else 0, flag.device_ptr, stream_ptr(x)))
    return y, taps, ctx


def bin_backward(grad_y, taps, ctx, x_shape, stride_h, stride_w, pad_h, pad_w, need_grad_x=True, need_grad_w=True, wrt_logits=False):
    """-> (grad_x or None, grad_w [C,7,16] or None) of bin_forward() from grad_y [N,C,Ho/2,Wo/2], the saved taps and ctx.
    grad_w is the gradient w.r.t. the logits with wrt_logits=True (the forward was given logits), else w.r.t. the
    probabilities."""
    check_input(grad_y, "grad_y", torch.float32, tuple(taps.shape))
    check_input(taps, "taps", torch.int16)
    check_input(ctx, "ctx", torch.uint8)
    n, c_in, h, w = x_shape
    c, hp, wp = grad_y.shape[1], grad_y.shape[2], grad_y.shape[3]
    g = ConvGeom(n, c_in, h, w, c, stride_h, stride_w, pad_h, pad_w, h + 2 * pad_h - (2 * hp - 1) * stride_h, w + 2 * pad_w - (2 * wp - 1) * stride_w)
    lib = _lib.load()
    dt = dtype_code(grad_y)
    if ctx.numel() < lib.clg_convblock_bin_ctx_bytes(dt, ctypes.byref(g)):
        raise RuntimeError("ctx is smaller than clg_convblock_bin_ctx_bytes() for this geometry")
    gx = torch.empty(x_shape, dtype=grad_y.dtype, device=grad_y.device) if need_grad_x else None
    gw = torch.empty((c, 7, 16), dtype=grad_y.dtype, device=grad_y.device) if need_grad_w else None
    scratch = _scratch(lib.clg_convblock_bin_backward_scratch_bytes(dt, ctypes.byref(g)), grad_y.device) if need_grad_w else None
    if need_grad_x or need_grad_w:
        check(lib.clg_convblock_bin_backward(dt, ctypes.byref(g), grad_y.data_ptr(), taps.data_ptr(), ctx.data_ptr(),
                                             gx.data_ptr() if need_grad_x else None, gw.data_ptr() if need_grad_w else None,
                                             1 if wrt_logits else 0, scratch.data_ptr() if need_grad_w else None, stream_ptr(grad_y)))
    return gx, gw
