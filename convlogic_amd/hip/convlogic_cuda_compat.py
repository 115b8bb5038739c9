"""Drop-in for the reference's native module `convlogic_cuda` (src/convlogic/cuda/convlogic.cpp:29-44): the same
nine function names with the reference's arities, argument order and return values, on top of the HIP C ABI.

    import convlogic_amd.hip.convlogic_cuda_compat as convlogic_cuda

lets the reference's own python (src/convlogic/convlogic_layer.py, src/convlogic/treelogic_layer.py) run unchanged.
The six split-layer functions are the ones of convlogic_hip.  The three fused-block functions differ from
convlogic_hip's (which keep one byte per pooled value instead of x2 / x3 / int32 indices): here they take and return
exactly what the reference's do,

    full_convlogic_forward(x, weight, selection, sh, sw, ph, pw, kh, kw) -> (y, x2, x3, indices)
    full_convlogic_backward_x(grad_y, x1, x2, x3, weight, indices, selection, sh, sw, ph, pw) -> (grad_x1, grad_x2, grad_x3)
    full_convlogic_backward_weight(grad_x2, grad_x3, grad_y, x1, x2, x3, indices, selection, sh, sw, ph, pw) -> grad_w

(src/convlogic/cuda/convlogic.cpp:17-26) with x2 [N,C,Ho,Wo,4] the leaf gates, x3 [N,C,Ho,Wo,2] the middle gates,
indices int32 [N,C,I] = in_y*Wo + in_x of the pooled maximum, grad_x2 [N,C,I,4] / grad_x3 [N,C,I,2] the gradients of the
leaf / middle gate outputs at the pooled position of every cell (src/convlogic/cuda/full_convlogic_kernel.cu:295-363),
and grad_w [C,7,16] w.r.t. the gate probabilities.  The input gradient comes from the fused HIP kernel; the per-level
quantities the reference's interface exposes are produced with the split-layer kernels (tree level backward at the
pooled positions), since the fused kernels never materialise them.
"""
import torch

from . import convlogic_hip
from .convlogic_hip import (convlogic_backward_weight, convlogic_backward_x, convlogic_forward, treelogic_backward_weight,  # noqa: F401
                            treelogic_backward_x, treelogic_forward)


def _indices_to_codes(indices, hp, wp, wo):
    """int32 [N,C,I] positions in the conv-output plane -> uint8 [N,C,hp,wp] window codes dy*2 + dx."""
    idx = indices.to(torch.int64)
    code = ((idx // wo) & 1) * 2 + ((idx % wo) & 1)
    return code.to(torch.uint8).view(indices.shape[0], indices.shape[1], hp, wp).contiguous()


def _scatter_to_plane(sparse, indices, ho, wo):
    """[N,C,I,K] values at the pooled positions -> dense [N,C,Ho,Wo,K] with zeros elsewhere (every cell owns its
    position, so no two values meet)."""
    n, c, i, k = sparse.shape
    dense = torch.zeros((n, c, ho * wo, k), dtype=sparse.dtype, device=sparse.device)
    dense.scatter_(2, indices.to(torch.int64).unsqueeze(-1).expand(n, c, i, k), sparse)
    return dense.view(n, c, ho, wo, k)


def _gather_from_plane(dense, indices):
    n, c, ho, wo, k = dense.shape
    i = indices.shape[2]
    return dense.view(n, c, ho * wo, k).gather(2, indices.to(torch.int64).unsqueeze(-1).expand(n, c, i, k)).contiguous()


def full_convlogic_forward(x, weight, selection, stride_h, stride_w, pad_h, pad_w, kernel_h, kernel_w):
    """-> (y [N,C,Ho/2,Wo/2], x2 [N,C,Ho,Wo,4], x3 [N,C,Ho,Wo,2], indices int32 [N,C,I]);
    src/convlogic/cuda/full_convlogic_kernel.cu:147-231."""
    geo = (stride_h, stride_w, pad_h, pad_w, kernel_h, kernel_w)
    y, argmax = convlogic_hip.full_convlogic_forward(x, weight, selection, *geo)
    x2, x3 = convlogic_hip.full_convlogic_intermediates(x, weight, selection, *geo)
    return y, x2, x3, convlogic_hip.argmax_to_indices(argmax, x2.shape[3])


def full_convlogic_backward_x(grad_y, x1, x2, x3, weight, indices, selection, stride_h, stride_w, pad_h, pad_w):
    """-> (grad_x1, grad_x2 [N,C,I,4], grad_x3 [N,C,I,2]); src/convlogic/cuda/full_convlogic_kernel.cu:365-461."""
    n, c, hp, wp = grad_y.shape
    ho, wo = x2.shape[2], x2.shape[3]
    codes = _indices_to_codes(indices, hp, wp, wo)
    grad_x1 = convlogic_hip.full_convlogic_backward_x(grad_y, x1, weight, codes, selection, stride_h, stride_w, pad_h, pad_w)
    # root gate, then the two middle gates, at the pooled position of every cell
    g_root = _scatter_to_plane(grad_y.reshape(n, c, hp * wp, 1), indices, ho, wo)
    g_x3_dense = convlogic_hip.treelogic_backward_x(g_root, x3, weight[:, 6:7].contiguous())
    g_x2_dense = convlogic_hip.treelogic_backward_x(g_x3_dense, x2, weight[:, 4:6].contiguous())
    return grad_x1, _gather_from_plane(g_x2_dense, indices), _gather_from_plane(g_x3_dense, indices)


def full_convlogic_backward_weight(grad_x2, grad_x3, grad_y, x1, x2, x3, indices, selection, stride_h, stride_w, pad_h, pad_w):
    """-> grad_w [C,7,16] w.r.t. the gate probabilities; src/convlogic/cuda/full_convlogic_kernel.cu:616-701.
    (The reference's binding does not receive the weights either: every gate's gradient follows from the gradient of
    its output and the values of its two inputs.)"""
    n, c, hp, wp = grad_y.shape
    ho, wo = x2.shape[2], x2.shape[3]
    g_leaf = _scatter_to_plane(grad_x2, indices, ho, wo)
    g_mid = _scatter_to_plane(grad_x3, indices, ho, wo)
    g_root = _scatter_to_plane(grad_y.reshape(n, c, hp * wp, 1), indices, ho, wo)
    gw = torch.empty((c, 7, 16), dtype=x1.dtype, device=x1.device)
    gw[:, 0:4] = convlogic_hip.convlogic_backward_weight(g_leaf, x1, selection, stride_h, stride_w, pad_h, pad_w)
    gw[:, 4:6] = convlogic_hip.treelogic_backward_weight(g_mid, x2)
    gw[:, 6:7] = convlogic_hip.treelogic_backward_weight(g_root, x3)
    return gw
