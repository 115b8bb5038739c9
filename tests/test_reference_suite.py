"""The reference's own test list, run against this package for both of its implementations:
"python" on the CPU (collected without a GPU) and "cuda" = the HIP library (marked gpu).

  tests/difflogic/test_difflogic_forward.py, test_difflogic_autograd.py
  tests/convlogic/test_convlogic_forward.py, test_full_convlogic_forward.py,
  test_convlogic_autograd.py, test_full_convlogic_autograd.py (smoke parts; gradchecks live in
  tests/test_gpu_conv.py and tests/test_gpu_fc.py), test_treelogic_forward.py, test_treelogic_autograd.py,
  test_poollayer.py

Each case states the property the reference checks (shape, finiteness, range, exact 0/1 on binary input,
determinism, batch size, smallest input, irregular sizes, residual init, python == cuda, split == complete).
"""
import copy

import pytest
import torch

import convlogic_amd as C
from convlogic_amd.difflogic.functional import bin_op

IMPLS = [pytest.param(("python", "cpu"), id="python"),
         pytest.param(("cuda", "cuda"), id="cuda", marks=pytest.mark.gpu)]


@pytest.fixture(params=IMPLS)
def impl_and_device(request):
    return request.param


def _finite_unit_range(y):
    assert torch.isfinite(y).all()
    assert (y >= 0.0).all() and (y <= 1.0).all()


# ---- LogicLayer ------------------------------------------------------------------------------------
@pytest.mark.parametrize("batch,in_dim,out_dim", [(2, 3, 5), (4, 4, 2), (8, 2, 3), (1, 1, 1), (1, 5, 3)])
def test_logiclayer_shape_finite_range_deterministic(impl_and_device, batch, in_dim, out_dim):
    impl, device = impl_and_device
    layer = C.LogicLayer(in_dim=in_dim, out_dim=out_dim, implementation=impl).to(device)
    x = torch.rand(batch, in_dim, device=device)
    y = layer(x)
    assert y.shape == (batch, out_dim)
    _finite_unit_range(y)
    assert torch.allclose(y, layer(x), atol=1e-6)


def test_logiclayer_binary_input_gives_0_1_in_eval(impl_and_device):
    impl, device = impl_and_device
    layer = C.LogicLayer(in_dim=3, out_dim=4, implementation=impl).to(device).eval()
    y = layer(torch.randint(0, 2, (1, 3), device=device, dtype=torch.float32))
    assert torch.all((y == 0.0) | (y == 1.0))


def test_logiclayer_all_logic_gates(impl_and_device):
    impl, device = impl_and_device
    layer = C.LogicLayer(in_dim=8, out_dim=64, implementation=impl).to(device)
    layer.indices_0.copy_(torch.tensor([0, 2, 4, 6], device=device).repeat(16))
    layer.indices_1.copy_(torch.tensor([1, 3, 5, 7], device=device).repeat(16))
    logits = torch.full((64, 16), float("-inf"), device=device)
    logits[torch.arange(64), torch.arange(64) // 4] = 0.0          # neurons 4g..4g+3 are gate g
    with torch.no_grad():
        layer.weights.copy_(logits)
    if impl == "cuda":                                           # the reverse map follows the wiring
        from convlogic_amd.difflogic.difflogic import _reverse_wiring
        start, flat = _reverse_wiring(layer.indices_0.cpu(), layer.indices_1.cpu(), 8)
        layer.given_x_indices_of_y_start.copy_(start)
        layer.given_x_indices_of_y.copy_(flat)
    rows = [0.0, 0.0, 0.0, 1.0, 1.0, 0.0, 1.0, 1.0]               # (a, b) = 00, 01, 10, 11
    y = layer(torch.tensor([rows], device=device))
    a, b = torch.tensor(rows[0::2], device=device), torch.tensor(rows[1::2], device=device)
    want = torch.stack([bin_op(a, b, g) for g in range(16)]).view(1, -1)
    assert torch.equal(y, want)


@pytest.mark.parametrize("in_dim,out_dim", [(2, 2), (3, 5), (6, 4)])
def test_logiclayer_backward_smoke(impl_and_device, in_dim, out_dim):
    impl, device = impl_and_device
    layer = C.LogicLayer(in_dim, out_dim, implementation=impl).to(device)
    x = torch.rand(3, in_dim, device=device, requires_grad=True)
    layer(x).sum().backward()
    assert x.grad.shape == x.shape and layer.weights.grad.shape == layer.weights.shape
    assert torch.isfinite(x.grad).all() and torch.isfinite(layer.weights.grad).all()


# ---- ConvLogicLayer, split (4 leaf gates) and complete (tree + pool) ---------------------------------------
def _conv(impl, device, cin, cout, complete, **kw):
    return C.ConvLogicLayer(in_channels=cin, out_channels=cout, implementation=impl, complete=complete, **kw).to(device).eval()


@pytest.mark.parametrize("complete", [False, True])
@pytest.mark.parametrize("stride,pad,kernel", [(1, 1, 3), (2, 2, 3)])
def test_convlogic_output_shape(impl_and_device, complete, stride, pad, kernel):
    impl, device = impl_and_device
    h = w = 11 + pad
    y = _conv(impl, device, 3, 2, complete, stride=stride, padding=pad, kernel=kernel)(torch.randn(2, 3, h, w, device=device))
    ho = (h + 2 * pad - kernel) // stride + 1
    assert y.shape == ((2, 2, ho // 2, ho // 2) if complete else (2, 2, ho, ho, 4))


@pytest.mark.parametrize("complete", [False, True])
def test_convlogic_finite_range_deterministic_batch(impl_and_device, complete):
    impl, device = impl_and_device
    y = _conv(impl, device, 2, 2, complete)(torch.randn(4, 2, 6, 6, device=device))
    assert torch.isfinite(y).all()
    layer = _conv(impl, device, 1, 1, complete, padding=1)
    x = torch.rand(8, 1, 6, 6, device=device)
    y = layer(x)
    assert y.shape[0] == 8
    _finite_unit_range(y)
    assert torch.allclose(y, layer(x), atol=1e-6)


@pytest.mark.parametrize("complete", [False, True])
def test_convlogic_binary_input_gives_0_1_in_eval(impl_and_device, complete):
    impl, device = impl_and_device
    y = _conv(impl, device, 2, 3, complete)(torch.randint(0, 2, (2, 2, 6, 6), device=device).float())
    assert torch.all((y == 0.0) | (y == 1.0))


def test_convlogic_small_input_and_irregular_channels(impl_and_device):
    impl, device = impl_and_device
    assert _conv(impl, device, 1, 1, True, kernel=2, padding=0)(torch.randn(1, 1, 3, 3, device=device)).shape == (1, 1, 1, 1)
    assert _conv(impl, device, 1, 1, False, kernel=2, padding=0)(torch.randn(1, 1, 2, 2, device=device)).shape == (1, 1, 1, 1, 4)
    y = _conv(impl, device, 1, 5, True)(torch.randn(1, 1, 6, 6, device=device))
    assert y.shape[1] == 5 and y.shape[-1] == 3
    y = _conv(impl, device, 5, 1, True)(torch.randn(5, 5, 4, 4, device=device))
    assert y.shape[1] == 1 and y.shape[-1] == 2


def test_convlogic_residual_init_selects_gate_a(impl_and_device):
    impl, device = impl_and_device
    layer = _conv(impl, device, 2, 2, True, stride=1, padding=1, residual_init=True)
    assert torch.all(layer.weights.argmax(-1) == 3)
    assert torch.all(_conv(impl, device, 2, 2, False, residual_init=True).weights.argmax(-1) == 3)


@pytest.mark.gpu
@pytest.mark.parametrize("complete", [False, True])
@pytest.mark.parametrize("stride,pad", [(1, 1), (1, 0), (2, 2)])
def test_convlogic_forward_python_cuda_match(complete, stride, pad):
    torch.manual_seed(0)
    layer = C.ConvLogicLayer(3, 2, stride=stride, padding=pad, kernel=3, complete=complete).to("cuda").eval()
    twin = copy.deepcopy(layer)
    twin.implementation = "python"
    x = torch.randn(4, 3, 8 + 2 * (pad == 2), 8 + 2 * (pad == 2), device="cuda")
    assert torch.allclose(twin(x), layer(x), atol=1e-6)


@pytest.mark.parametrize("complete", [False, True])
@pytest.mark.parametrize("stride,pad,kernel", [((1, 2), (1, 2), (1, 2)), ((3, 1), (3, 1), (3, 5)), (2, 2, 3)])
def test_convlogic_backward_smoke(impl_and_device, complete, stride, pad, kernel):
    impl, device = impl_and_device
    layer = C.ConvLogicLayer(1, 1, stride=stride, padding=pad, kernel=kernel, implementation=impl, complete=complete).to(device)
    size = 5
    if complete:                                                  # conv output must be even for the 2x2 pool
        pr = lambda v, i: v if isinstance(v, int) else v[i]
        for size in range(5, 12):
            outs = [(size + 2 * pr(pad, i) - pr(kernel, i)) // pr(stride, i) + 1 for i in (0, 1)]
            if all(o > 0 and o % 2 == 0 for o in outs):
                break
        else:
            pytest.skip("no square input gives even conv outputs for this geometry")
    x = torch.sigmoid(torch.rand(1, 1, size, size, device=device)).requires_grad_(True)
    layer(x).sum().backward()
    assert x.grad.shape == x.shape and layer.weights.grad.shape == layer.weights.shape
    assert torch.isfinite(x.grad).all() and torch.isfinite(layer.weights.grad).all()


# ---- TreeLogicLayer -----------------------------------------------------------------------------------
@pytest.mark.parametrize("batch,channels,bits", [(2, 3, 2), (4, 2, 2), (8, 1, 2), (1, 1, 2), (2, 5, 4), (3, 2, 8)])
def test_treelogic_shape_finite_range_deterministic(impl_and_device, batch, channels, bits):
    impl, device = impl_and_device
    layer = C.TreeLogicLayer(channels=channels, input_bits=bits, implementation=impl).to(device)
    x = torch.rand(batch, channels, 1, 1, bits, device=device)
    y = layer(x)
    assert y.shape == (batch, channels, 1, 1, bits // 2)
    _finite_unit_range(y)
    assert torch.allclose(y, layer(x), atol=1e-6)


def test_treelogic_all_logic_gates(impl_and_device):
    impl, device = impl_and_device
    layer = C.TreeLogicLayer(channels=16, input_bits=2, implementation=impl).to(device)
    logits = torch.full((16, 1, 16), float("-inf"), device=device)
    logits[torch.arange(16), 0, torch.arange(16)] = 0.0           # channel g is gate g
    with torch.no_grad():
        layer.weights.copy_(logits)
    for a in (0.0, 1.0):
        for b in (0.0, 1.0):
            x = torch.tensor([a, b], device=device).expand(1, 16, 1, 1, 2).contiguous()
            want = torch.stack([bin_op(torch.tensor(a), torch.tensor(b), g) for g in range(16)]).view(1, 16, 1, 1, 1)
            assert torch.equal(layer(x).cpu(), want)


@pytest.mark.parametrize("batch,channels,h,w,bits", [(1, 1, 1, 1, 2), (2, 3, 2, 2, 4)])
def test_treelogic_backward_smoke(impl_and_device, batch, channels, h, w, bits):
    impl, device = impl_and_device
    layer = C.TreeLogicLayer(channels, bits, implementation=impl).to(device)
    x = torch.rand(batch, channels, h, w, bits, device=device, requires_grad=True)
    layer(x).sum().backward()
    assert x.grad.shape == x.shape and layer.weights.grad.shape == layer.weights.shape


# ---- PoolLogicLayer (host tensors, as in the reference) ----------------------------------------------------
@pytest.mark.parametrize("batch,channels,h,w,kernel,stride", [(1, 1, 4, 4, 2, 2), (2, 3, 8, 8, (3, 3), (2, 2))])
def test_poollogic_forward_4d(batch, channels, h, w, kernel, stride):
    x = torch.randn(batch, channels, h, w, requires_grad=True)
    y = C.PoolLogicLayer(kernel=kernel, stride=stride)(x)
    assert torch.equal(y, torch.nn.functional.max_pool2d(x, kernel, stride))
    y.sum().backward()
    assert x.grad.shape == x.shape


@pytest.mark.parametrize("batch,channels,h,w", [(1, 1, 4, 4), (2, 2, 6, 8)])
def test_poollogic_forward_5d_and_invalid_dim(batch, channels, h, w):
    x4 = torch.randn(batch, channels, h, w)
    y = C.PoolLogicLayer(kernel=2, stride=2)(x4.unsqueeze(-1))
    assert torch.equal(y.squeeze(-1) if y.dim() == 5 else y, torch.nn.functional.max_pool2d(x4, 2, 2))
    with pytest.raises(Exception):
        C.PoolLogicLayer()(torch.randn(4, 4))
