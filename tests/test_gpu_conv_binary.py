"""GPU parity of the binary-input kernels of the fused block (clg_convblock_bin_*): y and the pooled position bit-identical
to the generic entry points, the tap byte against the tap bits gathered in torch, both gradients against the float64
oracle along the GPU's route (1e-4 relative) and against the generic kernels, at small and ragged shapes and at the
BASELINE shapes C3 / C4."""
import pytest
import torch

import convlogic_amd as C
from convlogic_amd.hip import convlogic_hip
from tests.gpu_util import DEV, assert_grad_close, block_oracle, check_pool_route

pytestmark = pytest.mark.gpu


def _binary(n, cin, h, w, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, 2, (n, cin, h, w), generator=g).float().to(DEV)


def _tap_bytes(layer, x, argmax):
    """tap byte of every pooled cell at the position `argmax` names, from the module's own tap gather"""
    taps = layer._tap_values(x)                                      # [N, C, Ho, Wo, 8]
    n, c, ho, wo, _ = taps.shape
    weights = (2 ** torch.arange(8, device=x.device)).view(1, 1, 1, 1, 8)
    byte = (taps.round().long() * weights).sum(-1)                   # [N, C, Ho, Wo]
    idx = convlogic_hip.argmax_to_indices(argmax, wo).long()         # [N, C, I]
    return byte.flatten(2).gather(2, idx).view(n, c, ho // 2, wo // 2)


SHAPES = [
    # n, cin, h, w, cout, pad, kernel
    (5, 3, 12, 12, 7, 1, 3),
    (3, 1, 28, 28, 32, 1, 3),
    (4, 9, 32, 32, 40, 1, 3),
    (2, 2, 8, 20, 5, 1, 3),
    (3, 4, 10, 18, 9, 0, 3),
    (2, 3, 16, 16, 6, 2, 5),
    (70, 2, 8, 8, 3, 1, 3),
    (3, 2, 8, 6, 5, 1, 3),                                           # rows of 3 pooled cells: written without the ordered write-out
    (2, 93, 32, 32, 48, 1, 3),                                       # the thresholded channels of the large CIFAR topology
    (3, 5, 32, 32, 600, 1, 3),                                       # more kernels than histogram parts, not a multiple of 64
    (3, 4, 32, 16, 12, 1, 3),                                        # exactly 128 pooled cells: two full blocks of 64 lanes
    (2, 6, 24, 32, 10, 1, 3),                                        # exactly 192: three
]


@pytest.mark.parametrize("n,cin,h,w,cout,pad,kernel", SHAPES)
def test_bin_forward_equals_generic(n, cin, h, w, cout, pad, kernel):
    torch.manual_seed(n * 100 + cout)
    layer = C.ConvLogicLayer(cin, cout, padding=pad, kernel=kernel, complete=True, implementation="cuda").to(DEV)
    x = _binary(n, cin, h, w, seed=7)
    geo = (1, 1, pad, pad, kernel, kernel)
    assert convlogic_hip.bin_supported(x, cout, *geo)
    flag = convlogic_hip.BinaryFlag()
    for logits in (True, False):
        w_in = layer.weights.detach() if logits else torch.softmax(layer.weights.detach(), -1)
        y, taps, _ = convlogic_hip.bin_forward(x, w_in.contiguous(), layer.selection, *geo, flag, logits=logits)
        if logits:
            y_ref, am_ref, _ = convlogic_hip.full_convlogic_forward_logits(x, w_in, layer.selection, *geo)
        else:
            y_ref, am_ref = convlogic_hip.full_convlogic_forward(x, w_in.contiguous(), layer.selection, *geo)
        t32 = taps.to(torch.int32) & 0xFFFF
        assert torch.equal(y, y_ref)
        assert torch.equal((t32 >> 8).to(torch.uint8), am_ref)
        assert torch.equal(t32 & 0xFF, _tap_bytes(layer, x, am_ref).to(torch.int32))
    torch.cuda.synchronize()
    assert not flag.raised()


@pytest.mark.parametrize("n,cin,h,w,cout,pad,kernel", SHAPES)
def test_bin_module_gradients_vs_oracle_and_generic(n, cin, h, w, cout, pad, kernel):
    torch.manual_seed(n * 10 + cin)
    layer = C.ConvLogicLayer(cin, cout, padding=pad, kernel=kernel, complete=True, implementation="cuda").to(DEV)
    x = _binary(n, cin, h, w, seed=11)
    xb = x.clone().requires_grad_(True)
    layer.binary_input = True
    y = layer(xb)
    gy = torch.randn_like(y)
    y.backward(gy)
    gl_bin = layer.weights.grad.clone()
    layer.weights.grad = None
    layer.binary_input = False
    xg = x.clone().requires_grad_(True)
    y2 = layer(xg)
    y2.backward(gy)
    assert torch.equal(y, y2)
    assert_grad_close(xb.grad, xg.grad, name="grad_x vs generic")
    assert_grad_close(gl_bin, layer.weights.grad, name="grad_logits vs generic")
    # oracle along the GPU's route
    geo = (1, 1, pad, pad, kernel, kernel)
    _, argmax, _ = convlogic_hip.full_convlogic_forward_logits(x, layer.weights.detach(), layer.selection, *geo)
    wo = w + 2 * pad - kernel + 1
    idx = convlogic_hip.argmax_to_indices(argmax, wo)
    routed, _, idx_ref, _, _, ll, xl, x4 = block_oracle(x.double(), layer.weights.detach().double(), layer.selection, (1, 1), (pad, pad),
                                                        (kernel, kernel), idx)
    check_pool_route(idx, idx_ref, x4)
    routed.backward(gy.cpu().double())
    assert (y.detach().cpu().double() - routed.detach()).abs().max().item() <= 1e-5
    assert_grad_close(xb.grad, xl.grad, name="grad_x")
    assert_grad_close(gl_bin, ll.grad, name="grad_logits")


def test_bin_eval_mode_and_probability_gradient():
    torch.manual_seed(5)
    layer = C.ConvLogicLayer(3, 12, complete=True, implementation="cuda").to(DEV)
    x = _binary(6, 3, 16, 16, seed=3)
    layer.eval()
    layer.binary_input = True
    y_bin = layer(x)
    layer.binary_input = False
    assert torch.equal(y_bin, layer(x))
    # gradient w.r.t. probabilities handed in by the caller
    w = torch.softmax(layer.weights.detach(), -1).requires_grad_(True)
    from convlogic_amd.convlogic.convlogic_layer import _FullConvLogicBinaryFunction
    flag = convlogic_hip.BinaryFlag()
    xb = x.clone().requires_grad_(True)
    yb = _FullConvLogicBinaryFunction.apply(xb, w, layer.selection, 1, 1, 1, 1, 3, 3, False, flag)
    gy = torch.randn_like(yb)
    yb.backward(gy)
    w2 = w.detach().clone().requires_grad_(True)
    x2 = x.clone().requires_grad_(True)
    y2 = C.FullConvLogicFunction.apply(x2, w2, layer.selection, 1, 1, 1, 1, 3, 3)
    y2.backward(gy)
    assert torch.equal(yb, y2)
    assert_grad_close(w.grad, w2.grad, name="grad_w")
    assert_grad_close(xb.grad, x2.grad, name="grad_x")


def test_bin_only_weight_gradient_when_input_needs_none():
    torch.manual_seed(6)
    layer = C.ConvLogicLayer(3, 9, complete=True, implementation="cuda").to(DEV)
    layer.binary_input = True
    x = _binary(4, 3, 12, 12, seed=4)
    y = layer(x)
    y.sum().backward()
    assert layer.weights.grad is not None and torch.isfinite(layer.weights.grad).all()


def test_bin_flags_non_binary_input():
    torch.manual_seed(8)
    layer = C.ConvLogicLayer(2, 4, complete=True, implementation="cuda").to(DEV)
    layer.binary_input = True
    x = _binary(3, 2, 8, 8, seed=5)
    layer(x)
    layer.check_binary_input()                                       # binary: nothing raised
    x[1, 0, 3, 3] = 0.5
    layer(x)
    with pytest.raises(RuntimeError, match="other than 0 and 1"):
        layer.check_binary_input()
    layer(_binary(3, 2, 8, 8, seed=6))                               # the flag was cleared by the report
    layer.check_binary_input()
    x[1, 0, 3, 3] = 2.0
    layer(x)
    torch.cuda.synchronize()
    with pytest.raises(RuntimeError, match="other than 0 and 1"):   # reported by the next call without an explicit check
        layer(x)


def test_bin_unsupported_shapes_fall_back():
    torch.manual_seed(9)
    x = _binary(2, 2, 40, 40, seed=1)                                # wider than a 32-bit row
    assert not convlogic_hip.bin_supported(x, 4, 1, 1, 1, 1, 3, 3)
    layer = C.ConvLogicLayer(2, 4, complete=True, implementation="cuda").to(DEV)
    layer.binary_input = True
    layer2 = C.ConvLogicLayer(2, 4, complete=True, implementation="cuda", selection=layer.selection.clone()).to(DEV)
    layer2.weights.data.copy_(layer.weights.data)
    assert torch.equal(layer(x), layer2(x))
    assert not convlogic_hip.bin_supported(_binary(2, 2, 30, 30, seed=1), 4, 1, 1, 1, 1, 3, 3)    # 225 pooled cells: not a multiple of 4
    assert not convlogic_hip.bin_supported(_binary(2, 2, 16, 16, seed=1), 4, 2, 2, 1, 1, 3, 3)    # stride 2


@pytest.mark.parametrize("piece", ["0", "2"])
def test_bin_forward_write_out_variants(piece, monkeypatch):
    # the write-out of y / taps in pieces of 4 cells (default where rows allow), 2 cells and row by row gives the same bytes
    from tests.gpu_util import set_knobs
    torch.manual_seed(12)
    layer = C.ConvLogicLayer(3, 10, complete=True, implementation="cuda").to(DEV)
    x = _binary(9, 3, 16, 16, seed=8)
    flag = convlogic_hip.BinaryFlag()
    y0, t0, _ = convlogic_hip.bin_forward(x, layer.weights.detach(), layer.selection, 1, 1, 1, 1, 3, 3, flag, logits=True)
    set_knobs(monkeypatch, CLG_BIN_PIECE=piece)
    y1, t1, _ = convlogic_hip.bin_forward(x, layer.weights.detach(), layer.selection, 1, 1, 1, 1, 3, 3, flag, logits=True)
    assert torch.equal(y0, y1) and torch.equal(t0, t1)


def test_bin_deterministic():
    torch.manual_seed(10)
    layer = C.ConvLogicLayer(9, 64, complete=True, implementation="cuda").to(DEV)
    layer.binary_input = True
    x = _binary(32, 9, 32, 32, seed=2)
    gy = None
    got = []
    for _ in range(2):
        xr = x.clone().requires_grad_(True)
        layer.weights.grad = None
        y = layer(xr)
        gy = torch.randn_like(y) if gy is None else gy
        y.backward(gy)
        got.append((y.detach().clone(), xr.grad.clone(), layer.weights.grad.clone()))
    for a, b in zip(*got):
        assert torch.equal(a, b)


def _full_size(n, cin, cout, size, x, seed, chunk):
    torch.manual_seed(seed)
    layer = C.ConvLogicLayer(cin, cout, complete=True, implementation="cuda").to(DEV)
    layer.binary_input = True
    xg = x.to(DEV).requires_grad_(True)
    y = layer(xg)
    gy = torch.randn_like(y)
    y.backward(gy)
    _, argmax, _ = convlogic_hip.full_convlogic_forward_logits(xg.detach(), layer.weights.detach(), layer.selection, 1, 1, 1, 1, 3, 3)
    idx = convlogic_hip.argmax_to_indices(argmax, size)
    gl_ref = torch.zeros(cout, 7, 16, dtype=torch.float64)
    flips = 0
    for s0 in range(0, n, chunk):
        sl = slice(s0, min(n, s0 + chunk))
        routed, _, idx_ref, _, _, ll, xl, x4 = block_oracle(xg.detach()[sl].double(), layer.weights.detach().double(), layer.selection,
                                                            (1, 1), (1, 1), (3, 3), idx[sl])
        flips += check_pool_route(idx[sl], idx_ref, x4)
        assert (y.detach()[sl].cpu().double() - routed.detach()).abs().max().item() <= 1e-5, s0
        routed.backward(gy[sl].cpu().double())
        assert_grad_close(xg.grad[sl], xl.grad, name=f"grad_x[{s0}:]")
        gl_ref += ll.grad
    assert flips <= 1e-4 * idx.numel(), flips
    assert_grad_close(layer.weights.grad, gl_ref, name="grad_logits")
    layer.check_binary_input()


def test_bin_config3_block_256x1x28x28_vs_oracle():
    g = torch.Generator().manual_seed(3)
    _full_size(256, 1, 32, 28, torch.randint(0, 2, (256, 1, 28, 28), generator=g).float(), seed=33, chunk=256)


@pytest.mark.timeout(600)
def test_bin_config4_block_256x9x32x32_vs_oracle():
    from tests.test_gpu_baseline_shapes import _c4_input
    _full_size(256, 9, 256, 32, _c4_input(256, 4), seed=44, chunk=32)
