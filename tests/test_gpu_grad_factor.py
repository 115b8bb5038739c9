"""grad_factor != 1 on the "cuda" layers: the forward value is unchanged and the gradient that reaches the layer's
input is grad_factor times the oracle's (GradFactor, src/difflogic/functional.py:131-139, applied at
src/difflogic/difflogic.py:100-101, src/convlogic/convlogic_layer.py:165-166, src/convlogic/treelogic_layer.py:91-92);
the gradient of the logits is not scaled."""
import pytest
import torch

import convlogic_amd as C
from oracle import convlogic_oracle as O
from tests.gpu_util import DEV, assert_grad_close, block_oracle

pytestmark = pytest.mark.gpu
F = 2.5


def test_grad_factor_logic_layer():
    torch.manual_seed(0)
    layer = C.LogicLayer(40, 64, grad_factor=F, implementation="cuda").to(DEV)
    x = torch.rand(48, 40, device=DEV, requires_grad=True)
    gy = torch.randn(48, 64, device=DEV)
    y = layer(x)
    y.backward(gy)
    xl = x.detach().cpu().requires_grad_(True)
    ll = layer.weights.detach().cpu().requires_grad_(True)
    want = O.logic_fc_forward(xl, layer.indices_0.cpu(), layer.indices_1.cpu(), torch.softmax(ll, -1))
    want.backward(gy.cpu())
    assert (y.detach().cpu() - want.detach()).abs().max().item() <= 1e-5
    assert_grad_close(x.grad, F * xl.grad, name="grad_x")
    assert_grad_close(layer.weights.grad, ll.grad, name="grad_logits")


@pytest.mark.parametrize("complete", [False, True])
def test_grad_factor_conv_layer(complete):
    torch.manual_seed(1)
    layer = C.ConvLogicLayer(3, 6, padding=1, grad_factor=F, complete=complete, implementation="cuda",
                             return_indices=complete).to(DEV)
    x = torch.rand(5, 3, 8, 10, device=DEV, requires_grad=True)
    if complete:
        y, idx = layer(x)
    else:
        y = layer(x)
    gy = torch.randn_like(y)
    y.backward(gy)
    if complete:
        ref, _, _, _, _, ll, xl, _ = block_oracle(x, layer.weights, layer.selection, (1, 1), (1, 1), (3, 3), idx)
    else:
        xl = x.detach().cpu().requires_grad_(True)
        ll = layer.weights.detach().cpu().requires_grad_(True)
        ref = O.conv4_forward(xl, torch.softmax(ll, -1), layer.selection.cpu(), (1, 1), (1, 1), (3, 3))
    ref.backward(gy.cpu())
    assert (y.detach().cpu() - ref.detach()).abs().max().item() <= 1e-5
    assert_grad_close(x.grad, F * xl.grad, name="grad_x")
    assert_grad_close(layer.weights.grad, ll.grad, name="grad_logits")


def test_grad_factor_conv_block_training_path():
    # the module's logits-in training path (no extra outputs) with grad_factor
    torch.manual_seed(3)
    layer = C.ConvLogicLayer(3, 6, padding=1, grad_factor=F, complete=True, implementation="cuda").to(DEV)
    plain = C.ConvLogicLayer(3, 6, padding=1, complete=True, implementation="cuda", selection=layer.selection.clone()).to(DEV)
    with torch.no_grad():
        plain.weights.copy_(layer.weights)
    x = torch.rand(5, 3, 8, 10, device=DEV)
    outs = []
    for m in (layer, plain):
        xi = x.clone().requires_grad_(True)
        y = m(xi)
        y.backward(torch.ones_like(y))
        outs.append((y.detach(), xi.grad, m.weights.grad))
    assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][2], outs[1][2])
    assert torch.equal(outs[0][1], outs[1][1] * F)


def test_grad_factor_tree_layer():
    torch.manual_seed(2)
    layer = C.TreeLogicLayer(5, 4, grad_factor=F, implementation="cuda").to(DEV)
    x = torch.rand(3, 5, 4, 6, 4, device=DEV, requires_grad=True)
    y = layer(x)
    gy = torch.randn_like(y)
    y.backward(gy)
    xl = x.detach().cpu().requires_grad_(True)
    ll = layer.weights.detach().cpu().requires_grad_(True)
    want = O.tree_forward(xl, torch.softmax(ll, -1))
    want.backward(gy.cpu())
    assert (y.detach().cpu() - want.detach()).abs().max().item() <= 1e-5
    assert_grad_close(x.grad, F * xl.grad, name="grad_x")
    assert_grad_close(layer.weights.grad, ll.grad, name="grad_logits")
