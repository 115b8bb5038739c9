"""GPU parity of the conv-logic layers (split 4-leaf layer, tree level, fused block) against the CPU
oracle through the C ABI.  Float32 forward within 1e-5, gradients within 1e-4 relative, pool indices
exact except on near ties (|gap| <= 1e-5) which are counted."""
import pytest
import torch

import convlogic_amd as C
from convlogic_amd.hip import convlogic_hip
from oracle import convlogic_oracle as O
from tests.gpu_util import DEV, assert_grad_close, block_oracle, check_pool_route, set_knobs

pytestmark = pytest.mark.gpu

GEOMS = [(1, 1, 3), (2, 2, 4), (1, 0, 3), (1, 2, 5)]


def _pair(v):
    return (v, v)


# ---- split layer ------------------------------------------------------------------------------
@pytest.mark.parametrize("stride,pad,kernel", GEOMS + [((1, 2), (0, 1), (2, 3))])
def test_conv4_forward_backward(stride, pad, kernel):
    torch.manual_seed(1)
    st, pd, kn = (stride if isinstance(stride, tuple) else _pair(stride), pad if isinstance(pad, tuple) else _pair(pad),
                  kernel if isinstance(kernel, tuple) else _pair(kernel))
    layer = C.ConvLogicLayer(3, 5, stride=st, padding=pd, kernel=kn, implementation="cuda").to(DEV)
    x = torch.randn(4, 3, 9, 10, device=DEV, requires_grad=True)
    y = layer(x)
    gy = torch.randn_like(y)
    y.backward(gy)
    xl = x.detach().cpu().requires_grad_(True)
    ll = layer.weights.detach().cpu().requires_grad_(True)
    want = O.conv4_forward(xl, torch.softmax(ll, -1), layer.selection.cpu(), st, pd, kn)
    want.backward(gy.cpu())
    assert y.shape == want.shape and (y.detach().cpu() - want.detach()).abs().max().item() <= 1e-5
    assert_grad_close(x.grad, xl.grad, name="grad_x")
    assert_grad_close(layer.weights.grad, ll.grad, name="grad_logits")


@pytest.mark.parametrize("bits", [2, 4, 8, 6])
def test_tree_forward_backward(bits):
    torch.manual_seed(2)
    layer = C.TreeLogicLayer(5, bits, implementation="cuda").to(DEV)
    x = torch.rand(3, 5, 4, 6, bits, device=DEV, requires_grad=True)
    y = layer(x)
    gy = torch.randn_like(y)
    y.backward(gy)
    xl = x.detach().cpu().requires_grad_(True)
    ll = layer.weights.detach().cpu().requires_grad_(True)
    want = O.tree_forward(xl, torch.softmax(ll, -1))
    want.backward(gy.cpu())
    assert (y.detach().cpu() - want.detach()).abs().max().item() <= 1e-5
    assert_grad_close(x.grad, xl.grad, name="grad_x")
    assert_grad_close(layer.weights.grad, ll.grad, name="grad_logits")


def test_tree_all_logic_gates_exact():
    # reference KAT tests/convlogic/test_treelogic_forward.py:66-86
    layer = C.TreeLogicLayer(channels=16, input_bits=8, implementation="cuda").to(DEV)
    logits = torch.full((16, 4, 16), float("-inf"), device=DEV)
    for g in range(16):
        logits[g, :, g] = 0.0
    with torch.no_grad():
        layer.weights.copy_(logits)
    flat = [0.0, 0.0, 0.0, 1.0, 1.0, 0.0, 1.0, 1.0]
    x = torch.tensor(flat, device=DEV).reshape(1, 1, 1, 1, 8).expand(-1, 16, -1, -1, -1)
    a, b = torch.tensor(flat[::2]), torch.tensor(flat[1::2])
    want = torch.stack([O.bin_op(a, b, g) for g in range(16)]).view(1, 16, 1, 1, 4)
    assert torch.equal(layer(x).cpu(), want)


# ---- fused block --------------------------------------------------------------------------------
def _run_block(n, cin, cout, h, w, stride, pad, kernel, dtype=torch.float32, binary=False, seed=0, training=True):
    torch.manual_seed(seed)
    layer = C.ConvLogicLayer(cin, cout, stride=stride, padding=pad, kernel=kernel, complete=True, implementation="cuda",
                             return_indices=True).to(DEV).to(dtype)
    layer.train(training)
    if binary:
        x = torch.randint(0, 2, (n, cin, h, w), device=DEV).to(dtype)
    else:
        x = torch.randn(n, cin, h, w, device=DEV, dtype=dtype)
    x.requires_grad_(True)
    y, idx = layer(x)
    return layer, x, y, idx


@pytest.mark.parametrize("stride,pad,kernel", GEOMS)
@pytest.mark.parametrize("binary", [False, True])
@pytest.mark.parametrize("direct", [None, "1", "subset"])
def test_block_forward_backward_small(stride, pad, kernel, binary, direct, monkeypatch):
    # "1" forces the kernels that read taps from a padded global copy of x (forward and input gradient);
    # "subset" forces the forward staging of two LDS planes per kernel
    if direct == "1":
        set_knobs(monkeypatch, CLG_BWDX_DIRECT="1")
        set_knobs(monkeypatch, CLG_FWD_DIRECT="1")
        set_knobs(monkeypatch, CLG_BWDW_PADDED="1")
    if direct == "subset":
        set_knobs(monkeypatch, CLG_FWD_SUBSET="1")
        set_knobs(monkeypatch, CLG_FWD_DIRECT="0")
    if binary:
        set_knobs(monkeypatch, CLG_BWDX_CSR="1")                    # compressed channel -> kernel lists (wide layers)
    n, cin, cout, h, w = 3, 3, 6, 8 + pad, 10 + pad
    if ((h + 2 * pad - kernel) // stride + 1) % 2:
        h += stride
    if ((w + 2 * pad - kernel) // stride + 1) % 2:
        w += stride
    layer, x, y, idx = _run_block(n, cin, cout, h, w, stride, pad, kernel, binary=binary, seed=stride * 10 + pad)
    gy = torch.randn_like(y)
    y.backward(gy)
    routed, y_ref, idx_ref, _, _, ll, xl, x4 = block_oracle(x, layer.weights, layer.selection, _pair(stride), _pair(pad),
                                                            _pair(kernel), idx)
    assert y.shape == y_ref.shape and idx.dtype == torch.int32 and idx.shape == idx_ref.shape
    check_pool_route(idx, idx_ref, x4)
    assert (y.detach().cpu() - routed.detach()).abs().max().item() <= 1e-5
    routed.backward(gy.cpu())
    assert_grad_close(x.grad, xl.grad, name="grad_x")
    assert_grad_close(layer.weights.grad, ll.grad, name="grad_logits")


def test_block_binary_ties_pick_first_position():
    # binary inputs in eval mode: outputs are exactly 0/1, ties are the norm, indices must equal max_pool2d's
    layer, x, y, idx = _run_block(4, 2, 8, 12, 12, 1, 1, 3, binary=True, seed=4, training=False)
    _, y_ref, idx_ref, *_ = block_oracle(x, layer.weights, layer.selection, (1, 1), (1, 1), (3, 3), idx, training=False)
    assert torch.all((y == 0) | (y == 1))
    assert torch.equal(y.detach().cpu(), y_ref.detach()) and torch.equal(idx.cpu(), idx_ref)


def test_block_return_intermediate_matches_split_layers():
    # mirrors tests/convlogic/test_full_convlogic_forward.py:165-233
    for stride, pad in [(1, 1), (2, 2)]:
        torch.manual_seed(0)
        full = C.ConvLogicLayer(3, 2, stride=stride, padding=pad, kernel=3, implementation="cuda", complete=True,
                                return_indices=True, return_intermediate=True).to(DEV)
        conv = C.ConvLogicLayer(3, 2, stride=stride, padding=pad, kernel=3, implementation="cuda").to(DEV)
        tree1 = C.TreeLogicLayer(2, 4, implementation="cuda").to(DEV)
        tree2 = C.TreeLogicLayer(2, 2, implementation="cuda").to(DEV)
        pool = C.PoolLogicLayer(return_indices=True)
        conv.selection = full.selection
        conv.weights.data.copy_(full.weights[:, 0:4])
        tree1.weights.data.copy_(full.weights[:, 4:6])
        tree2.weights.data.copy_(full.weights[:, 6:7])
        x = torch.randn(4, 3, 10, 10, device=DEV)
        with torch.no_grad():
            y_full, x1_full, x2_full, idx_full = full(x)
            x1 = conv(x)
            x2 = tree1(x1)
            y_split, idx_split = pool(tree2(x2))
        assert torch.equal(idx_split.flatten(start_dim=2).to(torch.int32), idx_full)
        assert torch.allclose(x1, x1_full, atol=1e-6) and torch.allclose(x2, x2_full, atol=1e-6)
        assert torch.allclose(y_split, y_full, atol=1e-6)


@pytest.mark.parametrize("batch", [1, 16])
@pytest.mark.parametrize("c_in,c_out", [(1, 1), (3, 1), (1, 3)])
@pytest.mark.parametrize("stride,pad,kernel", [(1, 1, 3), (2, 2, 4)])
def test_block_gradcheck_float64(batch, c_in, c_out, stride, pad, kernel):
    # mirrors tests/convlogic/test_full_convlogic_autograd.py:36-104 (no nondet_tol needed: deterministic)
    torch.manual_seed(batch + c_in * 3 + c_out * 5 + stride)
    layer = C.ConvLogicLayer(c_in, c_out, stride=stride, padding=pad, kernel=kernel, complete=True).double().to(DEV)
    x = torch.sigmoid(torch.rand(batch, c_in, 6, 6, dtype=torch.double, device=DEV)).requires_grad_(True)
    w = layer.weights.clone().detach().requires_grad_(True)
    sel = layer.selection

    def fn(inp, logits):
        return C.FullConvLogicFunction.apply(inp, torch.softmax(logits, -1), sel, stride, stride, pad, pad, kernel, kernel, False)

    assert torch.autograd.gradcheck(fn, (x, w), eps=1e-6, atol=1e-4)


@pytest.mark.parametrize("stride,pad,kernel", [(1, 1, 3), (2, 2, 4)])
def test_conv4_and_tree_gradcheck_float64(stride, pad, kernel):
    torch.manual_seed(3)
    layer = C.ConvLogicLayer(2, 3, stride=stride, padding=pad, kernel=kernel).double().to(DEV)
    x = torch.rand(4, 2, 6, 6, dtype=torch.double, device=DEV, requires_grad=True)
    w = layer.weights.clone().detach().requires_grad_(True)
    assert torch.autograd.gradcheck(
        lambda a, l: C.ConvLogicFunction.apply(a, torch.softmax(l, -1), layer.selection, stride, stride, pad, pad, kernel, kernel),
        (x, w), eps=1e-6, atol=1e-4)
    xt = torch.rand(2, 3, 2, 2, 4, dtype=torch.double, device=DEV, requires_grad=True)
    wt = torch.randn(3, 2, 16, dtype=torch.double, device=DEV, requires_grad=True)
    assert torch.autograd.gradcheck(lambda a, l: C.TreeLogicFunction.apply(a, torch.softmax(l, -1)), (xt, wt), eps=1e-6, atol=1e-4)


@pytest.mark.parametrize("shape", [(16, 1, 32, 28, 28), (4, 9, 256, 32, 32), (8, 32, 128, 16, 16), (8, 128, 512, 8, 8),
                                   (16, 512, 1024, 4, 4), (4, 1, 8, 28, 28)])
def test_block_benchmark_shapes_vs_oracle(shape):
    # BASELINE configs 3/4 and the blocks of config 5 at reduced batch, binary inputs
    n, cin, cout, h, w = shape
    layer, x, y, idx = _run_block(n, cin, cout, h, w, 1, 1, 3, binary=True, seed=cin)
    gy = torch.randn_like(y)
    y.backward(gy)
    routed, y_ref, idx_ref, _, _, ll, xl, x4 = block_oracle(x, layer.weights, layer.selection, (1, 1), (1, 1), (3, 3), idx)
    flips = check_pool_route(idx, idx_ref, x4)
    assert flips <= 1e-4 * idx.numel(), flips
    assert (y.detach().cpu() - routed.detach()).abs().max().item() <= 1e-5
    routed.backward(gy.cpu())
    assert_grad_close(x.grad, xl.grad, name="grad_x")
    assert_grad_close(layer.weights.grad, ll.grad, name="grad_logits")


@pytest.mark.parametrize("shape", [(37, 24, 48, 4, 4), (5, 200, 40, 16, 16), (3, 64, 32, 32, 32), (9, 40, 24, 6, 6),
                                   (70, 6, 12, 2, 2), (4, 1024, 2048, 4, 4), (2, 3, 8, 64, 64), (3, 2, 6, 32, 64), (2, 4, 5, 64, 32)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_block_deep_and_wide_shapes_vs_oracle(shape, dtype):
    # few cells per sample (several samples share a wavefront, ragged last group), images too large for LDS, and images of
    # several passes of 256 pooled cells (rows of 32 and 16 cells: the no-idle-lane input gradient steps from block to block)
    n, cin, cout, h, w = shape
    layer, x, y, idx = _run_block(n, cin, cout, h, w, 1, 1, 3, dtype=dtype, seed=n)
    gy = torch.randn_like(y)
    y.backward(gy)
    routed, y_ref, idx_ref, _, _, ll, xl, x4 = block_oracle(x, layer.weights, layer.selection, (1, 1), (1, 1), (3, 3), idx)
    check_pool_route(idx, idx_ref, x4)
    assert (y.detach().cpu() - routed.detach()).abs().max().item() <= 1e-5
    routed.backward(gy.cpu())
    assert_grad_close(x.grad, xl.grad, name="grad_x")
    assert_grad_close(layer.weights.grad, ll.grad, name="grad_logits")


def test_block_config4_full_size_properties():
    # BASELINE config 4 at full size: determinism (bitwise) and linearity of the backward in grad_y
    torch.manual_seed(5)
    layer = C.ConvLogicLayer(9, 256, complete=True, implementation="cuda").to(DEV)
    v = (torch.randn(256, 3, 32, 32, device=DEV) * 0.25 + 0.5).clamp(0, 1)
    x = torch.cat([(v > t).float() for t in (0.25, 0.5, 0.75)], dim=1).requires_grad_(True)
    y = layer(x)
    y2 = layer(x)
    assert y.shape == (256, 256, 16, 16) and torch.equal(y, y2)
    assert float(y.detach().min()) >= 0 and float(y.detach().max()) <= 1
    g1, g2 = torch.randn_like(y), torch.randn_like(y)

    def grads(g):
        return torch.autograd.grad(y, (x, layer.weights), g, retain_graph=True)

    a, b, ab, a2 = grads(g1), grads(g2), grads(g1 + g2), grads(g1)
    assert torch.equal(a[0], a2[0]) and torch.equal(a[1], a2[1])
    assert_grad_close(ab[0], a[0] + b[0], name="linearity grad_x")
    assert_grad_close(ab[1], a[1] + b[1], name="linearity grad_w")
    # eval mode on binary input is exactly binary, and max pooling is an OR of the four root gates
    layer.eval()
    with torch.no_grad():
        ye = layer(x)
    assert torch.all((ye == 0) | (ye == 1))


@pytest.mark.parametrize("n,cin,cout,h,w,kernel,pad,stride,dtype", [
    (2, 2, 4, 129, 129, (100, 100), 0, 1, torch.float32), (1, 1, 3, 260, 40, (255, 3), 1, 1, torch.float64),
    (2, 3, 4, 151, 151, (120, 120), 0, 2, torch.float32), (1, 2, 3, 254, 254, (251, 251), 0, 1, torch.float32)])
@pytest.mark.parametrize("indices", [True, False])
def test_block_with_windows_as_large_as_the_image(n, cin, cout, h, w, kernel, pad, stride, dtype, indices):
    # windows of up to 255 rows: shapes that no tile or padded-copy plan takes end on the any-shape kernels
    # (per-element gather of the input gradient among them); both the reference-shaped Function (indices) and the
    # module's training path against the oracle
    torch.manual_seed(h + w)
    layer = C.ConvLogicLayer(cin, cout, stride=stride, padding=pad, kernel=kernel, complete=True, implementation="cuda",
                             return_indices=indices).to(DEV).to(dtype)
    x = torch.randn(n, cin, h, w, device=DEV, dtype=dtype, requires_grad=True)
    out = layer(x)
    y, idx = out if indices else (out, None)
    gy = torch.randn_like(y)
    y.backward(gy)
    if idx is None:                                                 # the pooled positions of the same forward, from the Function
        from convlogic_amd.hip import difflogic_hip
        probs = difflogic_hip.fold(layer.weights.detach().reshape(-1, 16), from_logits=True)[0].reshape(cout, 7, 16)
        with torch.no_grad():
            y_fn, idx = C.FullConvLogicFunction.apply(x.detach(), probs, layer.selection, stride, stride, pad, pad, *kernel, False, True)
        assert torch.equal(y, y_fn)
    routed, _, idx_ref, _, _, ll, xl, x4 = block_oracle(x, layer.weights, layer.selection, _pair(stride), _pair(pad), kernel, idx)
    tol, rel = (1e-5, 1e-4) if dtype == torch.float32 else (1e-12, 1e-10)
    size = max(1.0, x4.detach().abs().max().item())
    check_pool_route(idx, idx_ref, x4, tol=tol * size)
    assert (y.detach().cpu() - routed.detach()).abs().max().item() <= tol * size
    routed.backward(gy.cpu())
    # (most of grad_x is structurally zero here: the per-element bound is taken against a mean that those zeros pull down)
    assert_grad_close(x.grad, xl.grad, rel=rel, rel_elem=10 * rel, name="grad_x")
    assert_grad_close(layer.weights.grad, ll.grad, rel=rel, rel_elem=10 * rel, name="grad_logits")


def test_block_with_more_kernels_than_a_grid_dimension_is_refused_on_the_host():
    # 65535 kernels per block is the limit of the gradient kernels and most forward kernels (the kernel index is a grid
    # dimension): above it a call raises before anything is launched; where a forward kernel without that limit takes the
    # shape its values are the oracle's
    torch.manual_seed(1)
    layer = C.ConvLogicLayer(2, 66000, padding=1, kernel=3, complete=True, implementation="cuda", return_indices=True).to(DEV)
    x = torch.randn(2, 2, 6, 6, device=DEV, requires_grad=True)
    y, idx = layer(x)
    routed, _, idx_ref, _, _, _, _, x4 = block_oracle(x, layer.weights, layer.selection, (1, 1), (1, 1), (3, 3), idx)
    check_pool_route(idx, idx_ref, x4, tol=1e-5 * max(1.0, x4.detach().abs().max().item()))
    assert (y.detach().cpu() - routed.detach()).abs().max().item() <= 1e-5 * max(1.0, x4.detach().abs().max().item())
    with pytest.raises(RuntimeError, match="65535"):
        y.backward(torch.randn_like(y))
    with pytest.raises(RuntimeError, match="65535"):
        layer(torch.randn(3, 2, 4, 4, device=DEV))
    torch.cuda.synchronize()


def test_block_errors():
    layer = C.ConvLogicLayer(1, 1, kernel=3, padding=0, complete=True).to(DEV)
    with pytest.raises(RuntimeError, match="divisible by 2"):
        layer(torch.rand(1, 1, 5, 5, device=DEV))
    with pytest.raises(RuntimeError):
        convlogic_hip.full_convlogic_forward(torch.rand(1, 1, 6, 6), layer.weights.detach().softmax(-1), layer.selection, 1, 1, 0, 0, 3, 3)
    layer = C.ConvLogicLayer(1, 1, kernel=2, padding=0, complete=True).to(DEV).eval()
    assert layer(torch.randn(1, 1, 3, 3, device=DEV)).shape == (1, 1, 1, 1)


@pytest.mark.parametrize("shape", [(5, 3, 6, 10, 12), (64, 9, 64, 32, 32)])
def test_block_fused_softmax_backward_matches_softmax_plus_function(shape):
    # module training path (logits in) against softmax -> FullConvLogicFunction; the large shape takes the
    # padded weight-gradient kernel, the small one the any-shape kernel
    from convlogic_amd.convlogic.convlogic_layer import _FullConvLogicLogitsFunction
    n, cin, cout, h, w = shape
    for dtype, tol in ((torch.float32, 5e-5), (torch.float64, 1e-11)):
        torch.manual_seed(n)
        layer = C.ConvLogicLayer(cin, cout, padding=1, complete=True, implementation="cuda").to(DEV).to(dtype)
        x = torch.rand(n, cin, h, w, device=DEV, dtype=dtype)
        outs = []
        for fused in (True, False):
            xl = x.clone().requires_grad_(True)
            logits = torch.randn_like(layer.weights).requires_grad_(True) if not outs else outs[0][3].detach().clone().requires_grad_(True)
            geo = (1, 1, 1, 1, 3, 3)
            if fused:
                y = _FullConvLogicLogitsFunction.apply(xl, logits, layer.selection, *geo)
            else:
                y = C.FullConvLogicFunction.apply(xl, torch.softmax(logits, -1), layer.selection, *geo)
            gy = torch.randn_like(y) if not outs else outs[0][4]
            y.backward(gy)
            outs.append((y.detach(), xl.grad, logits.grad, logits, gy))
        # the forward launch takes its own softmax of the logits (one reciprocal per row), so the two routes agree to
        # rounding, not bit for bit
        assert (outs[0][0] - outs[1][0]).abs().max().item() <= (2e-6 if dtype == torch.float32 else 1e-14)
        # (a pooled cell whose two best positions tie to rounding may route its gradient to the other one)
        for k in (1, 2):
            diff, ref = (outs[0][k] - outs[1][k]).abs(), outs[1][k]
            off = (diff > tol * ref.abs().max().item()).float().mean().item()
            assert k == 2 or off <= 2e-3, (k, off)                   # input gradient: a flip moves up to 8 elements
            assert (diff.norm() / ref.norm()).item() <= 1e-2, (k, (diff.norm() / ref.norm()).item())
            assert diff.max().item() <= 5e-2 * ref.abs().max().item(), k
    # first layer of a network: no input gradient requested
    layer.train()
    y = layer(x.detach())
    y.sum().backward()
    assert layer.weights.grad is not None and torch.isfinite(layer.weights.grad).all()


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("n,cin,cout", [(32, 3, 5), (100, 24, 48), (130, 40, 17)])
def test_block_4x4_one_sample_per_lane_vs_oracle_and_staged_path(n, cin, cout, dtype, monkeypatch):
    # 4x4 images with at least 32 samples take the one-sample-per-lane forward: against the oracle, against the
    # staged kernels (bit for bit, pooling choice included), with a ragged last wavefront, and with a caller-made
    # selection whose kernels read up to eight different channels (those kernels read global memory)
    from convlogic_amd.hip import convlogic_hip
    torch.manual_seed(n + cin)
    layer, x, y, idx = _run_block(n, cin, cout, 4, 4, 1, 1, 3, dtype=dtype, seed=n)
    routed, y_ref, idx_ref, _, _, _, _, x4 = block_oracle(x, layer.weights, layer.selection, (1, 1), (1, 1), (3, 3), idx)
    check_pool_route(idx, idx_ref, x4)
    assert (y.detach().cpu() - routed.detach()).abs().max().item() <= 1e-5
    wp = torch.softmax(layer.weights.detach(), -1)
    sel_wide = layer.selection.clone()
    if cin >= 8:
        taps = torch.arange(8, device=DEV, dtype=torch.int32)
        sel_wide[1] = ((taps % cin) << 16) | ((taps % 3) << 8) | ((taps // 3) % 3)          # eight channels
        sel_wide[cout - 1] = (((taps // 3) + 2) << 16) | ((taps % 3) << 8) | (taps % 2)     # three channels
    for sel in (layer.selection, sel_wide):
        args = (x.detach(), wp, sel, 1, 1, 1, 1, 3, 3)
        y_new, a_new = convlogic_hip.full_convlogic_forward(*args)
        set_knobs(monkeypatch, CLG_FWD_4X4="0")
        y_old, a_old = convlogic_hip.full_convlogic_forward(*args)
        set_knobs(monkeypatch, CLG_FWD_4X4=None)
        assert torch.equal(y_new, y_old) and torch.equal(a_new, a_old)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("n,cin,cout", [(32, 3, 5), (100, 24, 48), (130, 40, 17), (300, 16, 64)])
def test_block_4x4_one_sample_per_lane_gradients(n, cin, cout, dtype, monkeypatch):
    # gradients of 4x4 blocks from the two one-sample-per-lane passes (tap gradients per kernel, then a per-channel
    # sum in fixed order): against the oracle through the module, and against the staged kernels through both combined
    # entry points, with a ragged last wavefront, kernels that read up to eight channels, and without grad_x
    from convlogic_amd.hip import convlogic_hip
    layer, x, y, idx = _run_block(n, cin, cout, 4, 4, 1, 1, 3, dtype=dtype, seed=n + 1)
    gy = torch.randn_like(y)
    y.backward(gy)
    routed, _, idx_ref, _, _, ll, xl, x4 = block_oracle(x, layer.weights, layer.selection, (1, 1), (1, 1), (3, 3), idx)
    check_pool_route(idx, idx_ref, x4)
    routed.backward(gy.cpu())
    assert_grad_close(x.grad, xl.grad, name="grad_x")
    assert_grad_close(layer.weights.grad, ll.grad, name="grad_logits")
    wp = torch.softmax(layer.weights.detach(), -1)
    sel_wide = layer.selection.clone()
    if cin >= 8:
        taps = torch.arange(8, device=DEV, dtype=torch.int32)
        sel_wide[1] = ((taps % cin) << 16) | ((taps % 3) << 8) | ((taps // 3) % 3)
        sel_wide[cout - 1] = (((taps // 3) + 2) << 16) | ((taps % 3) << 8) | (taps % 2)
    tol = 2e-5 if dtype == torch.float32 else 1e-12
    for sel in (layer.selection, sel_wide):
        yy, am = convlogic_hip.full_convlogic_forward(x.detach(), wp, sel, 1, 1, 1, 1, 3, 3)
        got, want = {}, {}
        for store, flag in ((got, None), (want, "0")):
            if flag is not None:
                set_knobs(monkeypatch, CLG_BWD_4X4=flag)
            store["both"] = convlogic_hip.full_convlogic_backward(gy, x.detach(), wp, am, sel, 1, 1, 1, 1)
            store["logits"] = convlogic_hip.full_convlogic_backward_logits(gy, x.detach(), wp, am, sel, 1, 1, 1, 1)
            store["no_gx"] = convlogic_hip.full_convlogic_backward_logits(gy, x.detach(), wp, am, sel, 1, 1, 1, 1, need_grad_x=False)
            if flag is not None:
                set_knobs(monkeypatch, CLG_BWD_4X4=None)
        assert got["no_gx"][0] is None and want["no_gx"][0] is None
        for key in ("both", "logits", "no_gx"):
            for a, b in zip(got[key], want[key]):
                if a is None:
                    continue
                scale = max(b.abs().max().item(), 1e-30)
                assert (a - b).abs().max().item() <= tol * scale, key


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("n,cin,cout", [(32, 3, 5), (100, 24, 48), (130, 40, 17)])
def test_block_4x4_feature_major_output(n, cin, cout, dtype):
    # the last block of a 32x32-input network can lay its output out [C, 2, 2, N] for the LogicLayer behind nn.Flatten:
    # same values as the [N, C, 2, 2] kernels bit for bit, forward and both gradients, and the module chain
    # block -> Flatten -> LogicLayer then runs without transposed copies in either direction
    from convlogic_amd.hip import convlogic_hip
    torch.manual_seed(n * 7 + cin)
    layer = C.ConvLogicLayer(cin, cout, padding=1, complete=True, implementation="cuda").to(DEV).to(dtype)
    x = torch.rand(n, cin, 4, 4, device=DEV, dtype=dtype)
    wp = torch.softmax(layer.weights.detach(), -1)
    geo = (1, 1, 1, 1)
    assert convlogic_hip.feature_major_supported(x, cout, *geo, 3, 3)
    assert not convlogic_hip.feature_major_supported(x[:8], cout, *geo, 3, 3)           # fewer than 32 samples
    assert not convlogic_hip.feature_major_supported(torch.rand(n, cin, 8, 8, device=DEV, dtype=dtype), cout, *geo, 3, 3)
    y, am = convlogic_hip.full_convlogic_forward(x, wp, layer.selection, *geo, 3, 3)
    y_fm, am_fm = convlogic_hip.full_convlogic_forward_fm(x, wp, layer.selection, *geo, 3, 3)
    assert y_fm.shape == (cout, 2, 2, n) and torch.equal(y_fm.permute(3, 0, 1, 2), y) and torch.equal(am_fm, am)
    gy = torch.randn_like(y)
    gy_fm = gy.permute(1, 2, 3, 0).contiguous()
    for need_x in (True, False):
        gx, gl = convlogic_hip.full_convlogic_backward_logits(gy, x, wp, am, layer.selection, *geo, need_grad_x=need_x)
        gx_fm, gl_fm = convlogic_hip.full_convlogic_backward_fm(gy_fm, x, wp, am, layer.selection, *geo, need_grad_x=need_x)
        assert torch.equal(gl, gl_fm) and (gx is None and gx_fm is None or torch.equal(gx, gx_fm))
    _, gw = convlogic_hip.full_convlogic_backward(gy, x, wp, am, layer.selection, *geo)
    _, gw_fm = convlogic_hip.full_convlogic_backward_fm(gy_fm, x, wp, am, layer.selection, *geo, wrt_logits=False)
    assert torch.equal(gw, gw_fm)
    with pytest.raises(RuntimeError, match="clg_convblock_fm_supported"):
        convlogic_hip.full_convlogic_forward_fm(x[:8].contiguous(), wp, layer.selection, *geo, 3, 3)
    # module chain: the same losses and gradients with and without the layout
    head = C.LogicLayer(cout * 4, cout * 8, implementation="cuda").to(DEV).to(dtype)
    gout = torch.randn(n, cout * 8, device=DEV, dtype=dtype)
    grads = {}
    for fm in (False, True):
        layer.feature_major_output = fm
        xin = x.clone().requires_grad_(True)
        layer.weights.grad = head.weights.grad = None
        h = layer(xin)
        assert h.shape == (n, cout, 2, 2) and h.is_contiguous() != fm
        out = head(torch.flatten(h, 1))
        out.backward(gout)
        grads[fm] = (out.detach(), xin.grad, layer.weights.grad.clone(), head.weights.grad.clone())
    for a, b in zip(grads[False], grads[True]):
        assert torch.equal(a, b)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("shape,env", [((6, 3, 12, 12, 10), {}), ((70, 40, 8, 8, 24), {}), ((5, 24, 8, 8, 16), {"CLG_FWD_SUBSET": "1", "CLG_FWD_DIRECT": "0"}),
                                       ((6, 12, 16, 16, 20), {"CLG_FWD_DIRECT": "1"}), ((100, 24, 4, 4, 48), {}),
                                       ((3, 2, 11, 15, 4), {})])
def test_forward_from_logits_takes_the_softmax_inside(shape, env, dtype, monkeypatch):
    # the training path hands the logits to the forward launch: the probabilities it writes out equal torch's softmax to
    # rounding, and the block output is bit for bit what the probability entry point gives on those probabilities --
    # on the staged kernels (all channels, channel subsets, one position per lane), the padded-copy kernel, the 4x4
    # kernels (both output layouts) and the any-shape kernel (stride 2 here)
    from convlogic_amd.hip import convlogic_hip
    n, cin, h, w, cout = shape
    for k, v in env.items():
        set_knobs(monkeypatch, **{k: v})
    stride = 2 if h == 11 else 1
    torch.manual_seed(n + cin + h)
    layer = C.ConvLogicLayer(cin, cout, stride=stride, padding=1, complete=True, implementation="cuda").to(DEV).to(dtype)
    x = torch.rand(n, cin, h, w, device=DEV, dtype=dtype)
    logits = layer.weights.detach()
    geo = (stride, stride, 1, 1, 3, 3)
    y, am, probs = convlogic_hip.full_convlogic_forward_logits(x, logits, layer.selection, *geo)
    assert (probs - torch.softmax(logits, -1)).abs().max().item() <= (1e-6 if dtype == torch.float32 else 1e-14)
    y_ref, am_ref = convlogic_hip.full_convlogic_forward(x, probs, layer.selection, *geo)
    assert torch.equal(y, y_ref) and torch.equal(am, am_ref)
    if convlogic_hip.feature_major_supported(x, cout, *geo):
        y_fm, am_fm, probs_fm = convlogic_hip.full_convlogic_forward_logits(x, logits, layer.selection, *geo, feature_major=True)
        assert torch.equal(y_fm.permute(3, 0, 1, 2), y) and torch.equal(am_fm, am) and torch.equal(probs_fm, probs)


def test_forward_ex_rejects_bad_options():
    # the options entry point: unknown flags, logits without a place for the probabilities, the feature-major layout on a
    # shape its kernels do not take
    import ctypes
    from convlogic_amd.hip import _lib, convlogic_hip
    lib = _lib.load()
    layer = C.ConvLogicLayer(3, 4, padding=1, complete=True, implementation="cuda").to(DEV)
    x = torch.rand(2, 3, 8, 8, device=DEV)
    g = convlogic_hip._geom(x, 4, 1, 1, 1, 1, 3, 3)
    y = torch.empty(2, 4, 4, 4, device=DEV)
    am = torch.empty(2, 4, 4, 4, device=DEV, dtype=torch.uint8)
    probs = torch.empty_like(layer.weights)
    scratch = torch.empty(1 << 16, device=DEV, dtype=torch.uint8)

    def call(flags, probs_ptr):
        return lib.clg_convblock_forward_ex(0, ctypes.byref(g), x.data_ptr(), layer.weights.data_ptr(), layer.selection.data_ptr(),
                                            y.data_ptr(), am.data_ptr(), probs_ptr, flags, scratch.data_ptr(), None)

    assert call(16, probs.data_ptr()) != 0 and b"unknown flags" in lib.clg_last_error()
    assert call(8, probs.data_ptr()) != 0 and b"CLG_FWD_FOLDED_IN goes with" in lib.clg_last_error()
    assert call(1, None) != 0 and b"probs_out" in lib.clg_last_error()
    assert call(2, probs.data_ptr()) != 0 and b"clg_convblock_fm_supported" in lib.clg_last_error()
    assert call(1, probs.data_ptr()) == 0
    torch.cuda.synchronize()
    assert (probs - torch.softmax(layer.weights.detach(), -1)).abs().max().item() <= 1e-6


def test_block_bindings_reject_mismatched_tensors():
    # float32 probabilities with a float64 x, an int64 selection, a wrong gate count: RuntimeError before any launch
    layer = C.ConvLogicLayer(3, 4, padding=1, complete=True, implementation="cuda").to(DEV)
    x = torch.rand(2, 3, 8, 8, device=DEV)
    w = torch.softmax(layer.weights.detach(), -1)
    geo = (1, 1, 1, 1, 3, 3)
    with pytest.raises(RuntimeError, match="dtype"):
        convlogic_hip.full_convlogic_forward(x.double(), w, layer.selection, *geo)
    with pytest.raises(RuntimeError, match="dtype"):
        convlogic_hip.full_convlogic_forward(x, w, layer.selection.long(), *geo)
    with pytest.raises(RuntimeError, match="shape"):
        convlogic_hip.full_convlogic_forward(x, w[:, :4].contiguous(), layer.selection, *geo)
    with pytest.raises(RuntimeError, match="shape"):
        convlogic_hip.convlogic_forward(x, w, layer.selection, *geo)          # the split layer takes 4 gates
    y, am = convlogic_hip.full_convlogic_forward(x, w, layer.selection, *geo)
    with pytest.raises(RuntimeError, match="dtype"):
        convlogic_hip.full_convlogic_backward(torch.rand_like(y), x, w, am.int(), layer.selection, 1, 1, 1, 1)
    with pytest.raises(RuntimeError, match="shape"):
        convlogic_hip.full_convlogic_backward(torch.rand(2, 4, 4, 5, device=DEV), x, w, am, layer.selection, 1, 1, 1, 1)
    # the modules cast the probabilities to x's element type themselves: float32 weights, float64 input
    yd = layer(x.double())
    assert yd.dtype == torch.float64 and (yd.float() - layer(x)).abs().max().item() <= 1e-5
    tree = C.TreeLogicLayer(4, 4, implementation="cuda").to(DEV)
    xt = torch.rand(2, 4, 3, 3, 4, device=DEV)
    assert (tree(xt.double()).float() - tree(xt)).abs().max().item() <= 1e-5
    # a selection that names a channel the input does not have, and an input with the wrong channel count
    with pytest.raises(RuntimeError, match="Expected x of shape"):
        layer(torch.rand(2, 2, 8, 8, device=DEV))
    layer.selection[0, 0] = (7 << 16) | (1 << 8) | 1
    with pytest.raises(ValueError, match="selection names a tap outside"):
        layer(x)


@pytest.mark.parametrize("stride,pad,kernel", [(1, 1, 3), (2, 2, 4)])
def test_native_module_drop_in_with_the_reference_signatures(stride, pad, kernel):
    # convlogic_cuda_compat exports the reference's nine native functions with the reference's arities
    # (src/convlogic/cuda/convlogic.cpp:17-44).  The call sequence of the reference's FullConvLogicFunction
    # (src/convlogic/convlogic_layer.py:51-56 forward, :76-81 backward) is restated here on top of it and checked
    # against the oracle: y, x2, x3, indices, and both gradients.
    import convlogic_amd.hip.convlogic_cuda_compat as convlogic_cuda

    class RefShapedFunction(torch.autograd.Function):
        @staticmethod
        def forward(ctx, x, w_prob, selection, sh, sw, ph, pw, kh, kw):
            x1 = x.contiguous()
            y, x2, x3, indices = convlogic_cuda.full_convlogic_forward(x1, w_prob, selection, sh, sw, ph, pw, kh, kw)
            ctx.save_for_backward(x1, x2, x3, w_prob, selection, indices)
            ctx.stride, ctx.padding = (sh, sw), (ph, pw)
            ctx.mark_non_differentiable(indices)
            return y, x2, x3, indices

        @staticmethod
        def backward(ctx, grad_y, *_):
            x1, x2, x3, w_prob, selection, indices = ctx.saved_tensors
            grad_x1, grad_x2, grad_x3 = convlogic_cuda.full_convlogic_backward_x(grad_y.contiguous(), x1, x2, x3, w_prob, indices,
                                                                               selection, *ctx.stride, *ctx.padding)
            grad_w = convlogic_cuda.full_convlogic_backward_weight(grad_x2, grad_x3, grad_y.contiguous(), x1, x2, x3, indices,
                                                                   selection, *ctx.stride, *ctx.padding)
            return grad_x1, grad_w, None, None, None, None, None, None, None

    torch.manual_seed(stride + 40)
    layer = C.ConvLogicLayer(3, 6, stride=stride, padding=pad, kernel=kernel, complete=True, implementation="cuda").to(DEV)
    h = 9 if stride == 1 else 12
    while ((h + 2 * pad - kernel) // stride + 1) % 2:
        h += 1
    x = torch.rand(5, 3, h, h, device=DEV, requires_grad=True)
    logits = layer.weights.detach().clone().requires_grad_(True)
    y, x2, x3, indices = RefShapedFunction.apply(x, torch.softmax(logits, -1), layer.selection, stride, stride, pad, pad, kernel, kernel)
    gy = torch.randn_like(y)
    y.backward(gy)
    routed, y_ref, idx_ref, x2_ref, x3_ref, ll, xl, x4 = block_oracle(x, logits, layer.selection, _pair(stride), _pair(pad), _pair(kernel),
                                                                      indices)
    assert indices.dtype == torch.int32 and indices.shape == idx_ref.shape
    check_pool_route(indices, idx_ref, x4)
    assert (y.detach().cpu() - routed.detach()).abs().max().item() <= 1e-5
    assert (x2.detach().cpu() - x2_ref.detach()).abs().max().item() <= 1e-5
    assert (x3.detach().cpu() - x3_ref.detach()).abs().max().item() <= 1e-5
    routed.backward(gy.cpu())
    assert_grad_close(x.grad, xl.grad, name="grad_x")
    assert_grad_close(logits.grad, ll.grad, name="grad_logits")
    # the other six names are there with the reference's arities
    for name in ("convlogic_forward", "convlogic_backward_x", "convlogic_backward_weight", "treelogic_forward",
                 "treelogic_backward_x", "treelogic_backward_weight"):
        assert callable(getattr(convlogic_cuda, name))


def test_selection_corrupted_behind_the_host_check_is_clamped_not_faulting():
    # a selection written through `.data` after the (cached) host check names a channel, row and column outside the
    # layer: every kernel decodes taps through the layer's limits, so the calls return instead of faulting the GPU
    torch.manual_seed(41)
    for binary in (False, True):
        layer = C.ConvLogicLayer(3, 6, complete=True, implementation="cuda").to(DEV)
        layer.binary_input = binary
        x = torch.randint(0, 2, (4, 3, 8, 8), device=DEV).float().requires_grad_(True)
        layer(x).sum().backward()
        bad = layer.selection.data.clone()
        bad[2, 1] = (200 << 16) | (9 << 8) | 7
        bad[4, 6] = (3 << 16) | (3 << 8) | 3
        layer.selection.data.copy_(bad)
        layer._plans = {}                                            # (plans are keyed on the version counter, which .data bypasses)
        y = layer(x)
        y.sum().backward()
        torch.cuda.synchronize()
        assert torch.isfinite(y).all() and torch.isfinite(x.grad).all() and torch.isfinite(layer.weights.grad).all()
        # the result is that of the selection forced into range
        fixed = layer.selection.clone()
        ch, ry, rx = (fixed >> 16) & 0xFFFF, (fixed >> 8) & 0xFF, fixed & 0xFF
        fixed = (ch.clamp(max=2) << 16) | (ry.clamp(max=2) << 8) | rx.clamp(max=2)
        ref = C.ConvLogicLayer(3, 6, complete=True, implementation="cuda", selection=fixed.to(torch.int32)).to(DEV)
        ref.weights.data.copy_(layer.weights.data)
        assert torch.equal(y, ref(x.detach()))
        layer.invalidate()
        with pytest.raises(ValueError, match="selection"):
            layer(x)


@pytest.mark.parametrize("n,cin,h,w,cout", [(130, 32, 16, 16, 24), (20, 128, 8, 8, 40), (6, 1100, 16, 16, 48), (9, 3, 12, 12, 5)])
def test_padded_copy_left_by_the_forward_gives_the_planned_backward_its_taps(n, cin, h, w, cout):
    # the forward leaves the zero-padded copy of x it staged (all channels in LDS: the first two shapes; the direct
    # kernel's copy: the third) and the planned backward reads it instead of making one: bit-identical gradients; shapes
    # without such a pair of kernels (the last) report 0 elements and take the plain route
    torch.manual_seed(n + cin)
    x = torch.rand(n, cin, h, w, device=DEV)
    layer = C.ConvLogicLayer(cin, cout, complete=True, implementation="cuda").to(DEV)
    logits, sel = layer.weights.detach(), layer.selection
    geo = (1, 1, 1, 1)
    plan, sig = convlogic_hip.make_backward_plan(x, cout, sel, *geo, 3, 3)
    y, am, probs, folded, padded = convlogic_hip.full_convlogic_forward_logits(x, logits, sel, *geo, 3, 3, want_folded=True, want_padded=True)
    y0, am0, probs0, folded0 = convlogic_hip.full_convlogic_forward_logits(x, logits, sel, *geo, 3, 3, want_folded=True)
    assert torch.equal(y, y0) and torch.equal(am, am0) and torch.equal(folded, folded0)
    gy = torch.randn_like(y)
    gx0, gw0 = convlogic_hip.full_convlogic_backward_planned(gy, x, probs0, folded0, am0, sel, plan, sig, *geo)
    if cin == 3:
        assert padded is None
        return
    assert padded is not None
    # the copy itself: x inside, zeros in every halo
    rs, rows = w + 1, h + 1
    se = cin * rows * rs + rs + 1
    img = padded.view(n, se)[:, :cin * rows * rs].view(n, cin, rows, rs)
    assert torch.equal(img[:, :, 1:, 1:], x)
    assert not img[:, :, 0, :].any() and not img[:, :, :, 0].any() and not padded.view(n, se)[:, cin * rows * rs:].any()
    gx, gw = convlogic_hip.full_convlogic_backward_planned(gy, x, probs, folded, am, sel, plan, sig, *geo, padded=padded)
    assert torch.equal(gx, gx0) and torch.equal(gw, gw0)
    # and through the module: same gradients as the oracle route checks elsewhere, here against the plain call
    xg = x.clone().requires_grad_(True)
    layer(xg).backward(gy)
    assert torch.equal(xg.grad, gx0)


@pytest.mark.parametrize("n,cin,h,w,cout,dtype", [(5, 128, 8, 8, 512, torch.float32), (3, 16, 8, 8, 300, torch.float32),
                                                  (4, 24, 6, 6, 256, torch.float32), (2, 32, 8, 8, 256, torch.float64),
                                                  (3, 8, 8, 4, 260, torch.float32)])
def test_forward_with_one_kernel_per_lane_equals_the_position_major_kernel(n, cin, h, w, cout, dtype, monkeypatch):
    # deep blocks on small images (at least 256 kernels, at most 16 pooled cells): a lane keeps its kernel and walks the
    # positions; the same gate arithmetic, so y and the pooled positions equal those of the kernel with lanes along
    # positions bit for bit, and the oracle's to rounding
    torch.manual_seed(cin + cout)
    x = torch.rand(n, cin, h, w, device=DEV, dtype=dtype)
    layer = C.ConvLogicLayer(cin, cout, complete=True, implementation="cuda").to(DEV).to(dtype)
    w_prob = torch.softmax(layer.weights.detach(), -1)
    geo = (1, 1, 1, 1, 3, 3)
    set_knobs(monkeypatch, CLG_FWD_KPL=0)
    y0, am0 = convlogic_hip.full_convlogic_forward(x, w_prob, layer.selection, *geo)
    set_knobs(monkeypatch, CLG_FWD_KPL=None)
    y1, am1 = convlogic_hip.full_convlogic_forward(x, w_prob, layer.selection, *geo)
    assert torch.equal(y0, y1) and torch.equal(am0, am1)
    ref = O.conv_block_forward(x.cpu(), w_prob.cpu(), layer.selection.cpu(), (1, 1), (1, 1), (3, 3))
    assert (y1.cpu() - ref).abs().max().item() <= (1e-5 if dtype == torch.float32 else 1e-12)
    # from the logits, with the folded coefficients and the padded copy left for the backward pass
    res = convlogic_hip.full_convlogic_forward_logits(x, layer.weights.detach(), layer.selection, *geo, want_folded=True, want_padded=True)
    assert (res[0] - y1).abs().max().item() <= (2e-6 if dtype == torch.float32 else 1e-14)


def test_kernel_variants_behind_knobs_and_rare_shapes(monkeypatch):
    # instantiations that only a knob or an unusual shape selects, each against the default path or the split layers
    torch.manual_seed(12)
    # 1. the softmax of the logits as a launch of its own instead of inside the staged forward: same step bit for bit
    layer = C.ConvLogicLayer(4, 24, padding=1, complete=True, implementation="cuda").to(DEV)
    x = torch.rand(6, 4, 12, 12, device=DEV)
    gy = None
    results = []
    for knob in (None, "0", "1"):
        set_knobs(monkeypatch, CLG_FWD_SOFTMAX_IN_KERNEL=knob)
        xin = x.clone().requires_grad_(True)
        layer.weights.grad = None
        y = layer(xin)
        gy = torch.randn_like(y) if gy is None else gy
        y.backward(gy)
        results.append((y.detach().clone(), xin.grad.clone(), layer.weights.grad.clone()))
    set_knobs(monkeypatch, CLG_FWD_SOFTMAX_IN_KERNEL=None)
    for other in results[1:]:
        assert all(torch.equal(u, v) for u, v in zip(results[0], other))
    # 2. narrower histogram shares of the binary-input weight gradient: same sums in another order
    blayer = C.ConvLogicLayer(3, 10, padding=1, complete=True, implementation="cuda").to(DEV)
    blayer.binary_input = True
    xb = torch.randint(0, 2, (9, 3, 16, 16), device=DEV).float()
    grads = []
    for hl in (None, "32", "16"):
        set_knobs(monkeypatch, CLG_BIN_HL=hl)
        blayer.weights.grad = None
        yb = blayer(xb)
        yb.backward(torch.ones_like(yb) * 0.25)
        grads.append(blayer.weights.grad.clone())
    set_knobs(monkeypatch, CLG_BIN_HL=None)
    for g in grads[1:]:
        assert_grad_close(g, grads[0], rel=1e-5, name="grad_logits by histogram share")
    # 3. the intermediate tensors in float64 against the split layers
    full = C.ConvLogicLayer(3, 2, padding=1, kernel=3, implementation="cuda", complete=True, return_indices=True,
                            return_intermediate=True).double().to(DEV)
    conv = C.ConvLogicLayer(3, 2, padding=1, kernel=3, implementation="cuda").double().to(DEV)
    tree1, tree2 = C.TreeLogicLayer(2, 4, implementation="cuda").double().to(DEV), C.TreeLogicLayer(2, 2, implementation="cuda").double().to(DEV)
    conv.selection = full.selection
    conv.weights.data.copy_(full.weights[:, 0:4])
    tree1.weights.data.copy_(full.weights[:, 4:6])
    tree2.weights.data.copy_(full.weights[:, 6:7])
    xd = torch.randn(4, 3, 10, 10, device=DEV, dtype=torch.float64)
    with torch.no_grad():
        y_full, x1_full, x2_full, idx_full = full(xd)
        x1 = conv(xd)
        x2 = tree1(x1)
        y_split, idx_split = C.PoolLogicLayer(return_indices=True)(tree2(x2))
    assert torch.equal(idx_split.flatten(start_dim=2).to(torch.int32), idx_full)
    assert torch.allclose(x1, x1_full, atol=1e-13) and torch.allclose(x2, x2_full, atol=1e-13) and torch.allclose(y_split, y_full, atol=1e-13)
    # 4. the packed block with a window as large as the image (no staged or padded-copy plan): the float eval path's bits
    import numpy as np
    player = C.ConvLogicLayer(2, 5, padding=0, kernel=(120, 120), stride=2, complete=True, implementation="cuda").to(DEV).eval()
    bits = torch.randint(0, 2, (70, 2, 151, 151), device=DEV).bool()
    with torch.no_grad():
        yf = player(bits.float())
    p = player(C.PackBitsTensor(bits, 64))
    assert np.array_equal(O.unpack_image(p.t.cpu().numpy(), p.pad_len), yf.cpu().numpy() > 0.5)


@pytest.mark.parametrize("hw,pad", [(4, 1), (8, 1), (16, 1), (28, 1), (32, 1), (6, 0), (10, 0), (18, 0), (30, 0), (34, 0)])
def test_staged_forward_at_every_row_pitch_with_all_planes_and_with_a_plane_subset(hw, pad, monkeypatch):
    # the staged forward is compiled for the row pitches of the common image widths (5, 9, 17, 29, 33 and any other), with all
    # input planes of a sample in LDS or the two planes a kernel reads, for float and for packed words: every variant gives
    # the values of the default choice for the shape bit for bit, and the packed block the float eval path's bits
    import numpy as np
    torch.manual_seed(hw * 10 + pad)
    n, cin, cout = 70, 6, 10
    layer = C.ConvLogicLayer(cin, cout, padding=pad, kernel=3, complete=True, implementation="cuda", return_indices=True).to(DEV)
    x = torch.randn(n, cin, hw, hw, device=DEV)
    bits = torch.randint(0, 2, (n, cin, hw, hw), device=DEV).bool()
    with torch.no_grad():
        y0, idx0 = layer(x)
        layer.eval()
        yb0, _ = layer(bits.float())
        layer.train()
    routed, _, idx_ref, _, _, _, _, x4 = block_oracle(x, layer.weights, layer.selection, (1, 1), (pad, pad), (3, 3), idx0)
    check_pool_route(idx0, idx_ref, x4, tol=1e-5 * max(1.0, x4.abs().max().item()))
    assert (y0.cpu() - routed).abs().max().item() <= 1e-5 * max(1.0, x4.abs().max().item())
    for subset in ("0", "1"):
        set_knobs(monkeypatch, CLG_FWD_DIRECT="0", CLG_FWD_KPL="0", CLG_FWD_4X4="0", CLG_FWD_SUBSET=subset)
        with torch.no_grad():
            y, idx = layer(x)
            assert torch.equal(y, y0) and torch.equal(idx, idx0), (hw, pad, subset)
            layer.eval()
            p = layer(C.PackBitsTensor(bits, 64))
            layer.train()
        assert np.array_equal(O.unpack_image(p.t.cpu().numpy(), p.pad_len), yb0.cpu().numpy() > 0.5), (hw, pad, subset)
    set_knobs(monkeypatch, CLG_FWD_DIRECT=None, CLG_FWD_KPL=None, CLG_FWD_4X4=None, CLG_FWD_SUBSET=None)
