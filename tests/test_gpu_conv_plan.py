"""Per-layer plan of the fused block's backward pass (clg_convblock_plan / clg_convblock_backward_planned): the tables
that depend only on the selection are built once; a planned call gives the gradients of the unplanned entry points on
every kernel family (images in LDS, padded global copy, 4x4 one-sample-per-lane, any-shape gather), twice in a row,
with and without the coefficients folded by the forward launch."""
import ctypes

import pytest
import torch

import convlogic_amd as C
from convlogic_amd.hip import _lib, convlogic_hip
from tests.gpu_util import DEV, assert_grad_close, block_oracle, set_knobs

pytestmark = pytest.mark.gpu

# (n, cin, cout, h, w, stride): LDS-tiled (few and many kernels), padded-copy kernels, 4x4 images, any-shape gather
SHAPES = [(24, 1, 32, 28, 28, 1), (6, 9, 40, 32, 32, 1), (40, 128, 64, 8, 8, 1), (70, 24, 48, 4, 4, 1), (5, 3, 6, 11, 15, 2),
          (3, 64, 32, 32, 32, 1)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("shape", SHAPES)
def test_planned_backward_matches_unplanned(shape, dtype):
    n, cin, cout, h, w, stride = shape
    torch.manual_seed(n + cin)
    layer = C.ConvLogicLayer(cin, cout, stride=stride, padding=1, complete=True, implementation="cuda").to(DEV).to(dtype)
    x = torch.rand(n, cin, h, w, device=DEV, dtype=dtype)
    geo = (stride, stride, 1, 1)
    y, am, probs, folded = convlogic_hip.full_convlogic_forward_logits(x, layer.weights.detach(), layer.selection, *geo, 3, 3, want_folded=True)
    y0, am0, probs0 = convlogic_hip.full_convlogic_forward_logits(x, layer.weights.detach(), layer.selection, *geo, 3, 3)
    assert torch.equal(y, y0) and torch.equal(am, am0) and torch.equal(probs, probs0)
    # the folded coefficients are those of the probabilities: c_1 = sum of gates 8..15, c_a = p2+p3+p6+p7-p8-p9-p12-p13, ...
    p = probs.double()
    want_one = p[..., 8:].sum(-1)
    want_a = p[..., [2, 3, 6, 7]].sum(-1) - p[..., [8, 9, 12, 13]].sum(-1)
    assert (folded[..., 3].double() - want_one).abs().max().item() <= 1e-6
    assert (folded[..., 1].double() - want_a).abs().max().item() <= 1e-6
    gy = torch.randn_like(y)
    gx_ref, gl_ref = convlogic_hip.full_convlogic_backward_logits(gy, x, probs, am, layer.selection, *geo)
    _, gw_ref = convlogic_hip.full_convlogic_backward(gy, x, probs, am, layer.selection, *geo)
    plan, sig = convlogic_hip.make_backward_plan(x, cout, layer.selection, *geo, 3, 3)
    tol = 2e-5 if dtype == torch.float32 else 1e-12
    for rep in range(2):                                             # a plan is only read: the second call gives the same
        for fold in (folded, None):
            gx, gl = convlogic_hip.full_convlogic_backward_planned(gy, x, probs, fold, am, layer.selection, plan, sig, *geo)
            assert torch.equal(gx, gx_ref)                           # same kernels on the same tables
            assert (gl - gl_ref).abs().max().item() <= tol * gl_ref.abs().max().item()
        gx, gw = convlogic_hip.full_convlogic_backward_planned(gy, x, probs, folded, am, layer.selection, plan, sig, *geo, wrt_logits=False)
        assert torch.equal(gx, gx_ref) and (gw - gw_ref).abs().max().item() <= tol * gw_ref.abs().max().item()
        none, gl = convlogic_hip.full_convlogic_backward_planned(gy, x, probs, folded, am, layer.selection, plan, sig, *geo, need_grad_x=False)
        assert none is None and (gl - gl_ref).abs().max().item() <= tol * gl_ref.abs().max().item()
    if convlogic_hip.feature_major_supported(x, cout, *geo, 3, 3):     # the gradient of a feature-major output
        gy_fm = gy.permute(1, 2, 3, 0).contiguous()
        gx_fm, gl_fm = convlogic_hip.full_convlogic_backward_fm(gy_fm, x, probs, am, layer.selection, *geo)
        gx, gl = convlogic_hip.full_convlogic_backward_planned(gy_fm, x, probs, folded, am, layer.selection, plan, sig, *geo, feature_major=True)
        assert torch.equal(gx, gx_fm) and torch.equal(gl, gl_fm)
    else:
        with pytest.raises(RuntimeError, match="clg_convblock_fm_supported"):
            convlogic_hip.full_convlogic_backward_planned(gy.permute(1, 2, 3, 0).contiguous(), x, probs, folded, am, layer.selection, plan, sig,
                                                          *geo, feature_major=True, validate=False)


def test_plan_is_rejected_for_another_geometry_and_after_knob_changes(monkeypatch):
    layer = C.ConvLogicLayer(3, 8, padding=1, complete=True, implementation="cuda").to(DEV)
    x = torch.rand(4, 3, 16, 16, device=DEV)
    geo = (1, 1, 1, 1)
    y, am, probs, folded = convlogic_hip.full_convlogic_forward_logits(x, layer.weights.detach(), layer.selection, *geo, 3, 3, want_folded=True)
    plan, sig = convlogic_hip.make_backward_plan(x, 8, layer.selection, *geo, 3, 3)
    gy = torch.randn_like(y)
    convlogic_hip.full_convlogic_backward_planned(gy, x, probs, folded, am, layer.selection, plan, sig, *geo)
    with pytest.raises(RuntimeError, match="plan was made for another"):
        convlogic_hip.full_convlogic_backward_planned(gy, x, probs, folded, am, layer.selection, plan, sig + 1, *geo)
    x2 = torch.rand(6, 3, 16, 16, device=DEV)                        # another batch size: another plan
    y2, am2, probs2, folded2 = convlogic_hip.full_convlogic_forward_logits(x2, layer.weights.detach(), layer.selection, *geo, 3, 3,
                                                                        want_folded=True)
    big = torch.empty(1 << 20, dtype=torch.uint8, device=DEV)
    big[:plan.numel()] = plan
    with pytest.raises(RuntimeError, match="plan was made for another"):
        convlogic_hip.full_convlogic_backward_planned(torch.randn_like(y2), x2, probs2, folded2, am2, layer.selection, big, sig, *geo)
    set_knobs(monkeypatch, CLG_BWDX_DIRECT="1")                      # another kernel family: the old plan no longer fits
    with pytest.raises(RuntimeError, match="plan was made for another"):
        convlogic_hip.full_convlogic_backward_planned(gy, x, probs, folded, am, layer.selection, big, sig, *geo)
    # the module keys its plans on the knob generation, so it simply builds a new one
    layer.train()
    xin = x.clone().requires_grad_(True)
    layer(xin).sum().backward()
    assert torch.isfinite(xin.grad).all()


@pytest.mark.parametrize("shape", [(16, 1, 32, 28, 28), (8, 9, 64, 32, 32), (40, 128, 64, 8, 8)])
def test_module_training_path_uses_the_plan_and_matches_the_oracle(shape):
    n, cin, cout, h, w = shape
    torch.manual_seed(cin)
    layer = C.ConvLogicLayer(cin, cout, padding=1, complete=True, implementation="cuda", return_indices=False).to(DEV)
    x = torch.randint(0, 2, (n, cin, h, w), device=DEV).float().requires_grad_(True)
    grads = []
    for step in range(2):
        layer.weights.grad = x.grad = None
        y = layer(x)
        gy = torch.randn(y.shape, device=DEV, generator=torch.Generator(device=DEV).manual_seed(3))
        y.backward(gy)
        grads.append((y.detach().clone(), x.grad.clone(), layer.weights.grad.clone()))
    assert len(layer._plans) == 1
    for a, b in zip(*grads):
        assert torch.equal(a, b)                                     # same plan, same result
    _, am, _ = convlogic_hip.full_convlogic_forward_logits(x.detach(), layer.weights.detach(), layer.selection, 1, 1, 1, 1, 3, 3)
    idx = convlogic_hip.argmax_to_indices(am, w)
    routed, _, _, _, _, ll, xl, _ = block_oracle(x, layer.weights, layer.selection, (1, 1), (1, 1), (3, 3), idx)
    routed.backward(gy.cpu())
    assert (grads[0][0].cpu() - routed.detach()).abs().max().item() <= 1e-5
    assert_grad_close(grads[0][1], xl.grad, name="grad_x")
    assert_grad_close(grads[0][2], ll.grad, name="grad_logits")
    # another batch size gets a plan of its own; an in-place edit of the selection drops the old ones on the next call
    layer(x[:3].detach()).sum().backward()
    assert len(layer._plans) == 2
