"""GPU parity of the fully connected LogicLayer (forward, both gradients) against the CPU oracle,
through the C ABI.  Tolerances: float32 forward 1e-5 absolute, gradients 1e-4 relative."""
import pytest
import torch

import convlogic_amd as C
from convlogic_amd.hip import difflogic_hip
from oracle import convlogic_oracle as O
from tests.gpu_util import DEV, assert_grad_close

pytestmark = pytest.mark.gpu


def _layer_with(idx0, idx1, in_dim, dtype):
    """A LogicLayer on the device with the given wiring (and the consumer lists that go with it)."""
    from convlogic_amd.difflogic.difflogic import _reverse_wiring
    layer = C.LogicLayer(in_dim, idx0.numel(), implementation="cuda")
    layer.indices_0.copy_(idx0)
    layer.indices_1.copy_(idx1)
    start, flat = _reverse_wiring(idx0.numpy(), idx1.numpy(), in_dim)
    layer.given_x_indices_of_y_start.copy_(start)
    layer.given_x_indices_of_y.copy_(flat)
    return layer.to(DEV).to(dtype)


def _oracle_grads(x, logits, idx0, idx1, gy):
    xl = x.detach().cpu().clone().requires_grad_(True)
    ll = logits.detach().cpu().clone().requires_grad_(True)
    y = O.logic_fc_forward(xl, idx0.cpu(), idx1.cpu(), torch.softmax(ll, -1))
    y.backward(gy.cpu())
    return y.detach(), xl.grad, ll.grad


@pytest.mark.parametrize("in_dim,out_dim,batch", [(8, 8, 32), (12, 16, 5), (100, 64, 256), (33, 40, 257), (1, 1, 1),
                                                  # 20 to 43 consumers per input (several groups of four in flight in the
                                                  # backward walk) at 16, 32 and 64 lanes per row and beyond one pass
                                                  (6, 60, 12), (10, 100, 100), (7, 150, 256), (6, 61, 300), (5, 43, 64)])
def test_fc_module_forward_backward(in_dim, out_dim, batch):
    # the feature-major kernels with transposed copies of x and grad_y (grad_x leaves its kernel sample-major)
    torch.manual_seed(in_dim * 1000 + batch)
    layer = C.LogicLayer(in_dim, out_dim, implementation="cuda").to(DEV)
    x = torch.rand(batch, in_dim, device=DEV, requires_grad=True)
    gy = torch.randn(batch, out_dim, device=DEV)
    y = layer(x)
    y.backward(gy)
    y_ref, gx_ref, gl_ref = _oracle_grads(x, layer.weights, layer.indices_0, layer.indices_1, gy)
    assert y.shape == (batch, out_dim)
    assert (y.detach().cpu() - y_ref).abs().max().item() <= 1e-5
    assert x.grad.is_contiguous()
    assert_grad_close(x.grad, gx_ref, name="grad_x")
    assert_grad_close(layer.weights.grad, gl_ref, name="grad_logits")


def test_fc_self_paired_neuron_follows_python_derivative():
    torch.manual_seed(5)
    layer = C.LogicLayer(6, 8, implementation="cuda")
    idx0, idx1 = layer.indices_0.clone(), layer.indices_1.clone()
    idx1[2] = idx0[2]
    idx1[5] = idx0[5]
    layer = C.LogicLayer(6, 8, implementation="cuda")
    layer.indices_0.copy_(idx0)
    layer.indices_1.copy_(idx1)
    from convlogic_amd.difflogic.difflogic import _reverse_wiring
    s, f = _reverse_wiring(idx0.numpy(), idx1.numpy(), 6)
    layer.given_x_indices_of_y_start.copy_(s)
    layer.given_x_indices_of_y.copy_(f)
    layer = layer.to(DEV)
    x = torch.rand(9, 6, device=DEV, requires_grad=True)
    gy = torch.randn(9, 8, device=DEV)
    layer(x).backward(gy)
    _, gx_ref, gl_ref = _oracle_grads(x, layer.weights, idx0, idx1, gy)
    assert_grad_close(x.grad, gx_ref, name="grad_x")
    assert_grad_close(layer.weights.grad, gl_ref, name="grad_logits")


def test_fc_all_logic_gates_exact():
    # reference KAT tests/difflogic/test_difflogic_forward.py:74-100
    layer = C.LogicLayer(in_dim=8, out_dim=64, implementation="cuda").to(DEV)
    layer.indices_0.copy_(torch.tensor([0, 2, 4, 6], device=DEV).repeat(16))
    layer.indices_1.copy_(torch.tensor([1, 3, 5, 7], device=DEV).repeat(16))
    logits = torch.full((64, 16), float("-inf"), device=DEV)
    for g in range(16):
        logits[g * 4: g * 4 + 4, g] = 0.0
    with torch.no_grad():
        layer.weights.copy_(logits)
    flat = [0.0, 0.0, 0.0, 1.0, 1.0, 0.0, 1.0, 1.0]
    y = layer(torch.tensor([flat], device=DEV))
    a, b = torch.tensor(flat[::2]), torch.tensor(flat[1::2])
    want = torch.stack([O.bin_op(a, b, g) for g in range(16)]).view(1, -1)
    assert torch.equal(y.cpu(), want)


def test_fc_eval_binary_and_deterministic():
    torch.manual_seed(7)
    layer = C.LogicLayer(50, 70, implementation="cuda").to(DEV).eval()
    x = torch.randint(0, 2, (33, 50), device=DEV).float()
    y1, y2 = layer(x), layer(x)
    assert torch.equal(y1, y2) and torch.all((y1 == 0) | (y1 == 1))
    want = O.logic_fc_forward(x.cpu(), layer.indices_0.cpu(), layer.indices_1.cpu(), O.gate_weights(layer.weights.detach().cpu(), False))
    assert torch.equal(y1.cpu(), want)


@pytest.mark.parametrize("in_dim,out_dim", [(8, 8), (12, 16)])
def test_fc_gradcheck_float64(in_dim, out_dim):
    # mirrors tests/difflogic/test_difflogic_autograd.py:31-54
    torch.manual_seed(11)
    layer = C.LogicLayer(in_dim, out_dim, implementation="cuda").double().to(DEV)
    x = torch.sigmoid(torch.randn(16, in_dim, dtype=torch.double, device=DEV)).requires_grad_(True)
    w = layer.weights.clone().detach().requires_grad_(True)
    a, b, gs, gl = layer.indices_0, layer.indices_1, layer.given_x_indices_of_y_start, layer.given_x_indices_of_y

    def fn(inp, logits):
        return C.LogicLayerCudaFunction.apply(inp.T.contiguous(), a, b, torch.softmax(logits, -1), gs, gl).T

    assert torch.autograd.gradcheck(fn, (x, w), eps=1e-6, atol=1e-4)


def test_fc_chained_layers_avoid_copies_and_match():
    torch.manual_seed(13)
    l1 = C.LogicLayer(20, 40, implementation="cuda").to(DEV)
    l2 = C.LogicLayer(40, 30, implementation="cuda").to(DEV)
    x = torch.rand(64, 20, device=DEV)
    y = l2(l1(x))
    h = O.logic_fc_forward(x.cpu(), l1.indices_0.cpu(), l1.indices_1.cpu(), torch.softmax(l1.weights.detach().cpu(), -1))
    want = O.logic_fc_forward(h, l2.indices_0.cpu(), l2.indices_1.cpu(), torch.softmax(l2.weights.detach().cpu(), -1))
    assert (y.detach().cpu() - want).abs().max().item() <= 1e-5


def test_fc_config1_shape_properties():
    # BASELINE config 1 at full size: oracle forward (cheap) + determinism and linearity of backward
    torch.manual_seed(17)
    layer = C.LogicLayer(8000, 8000, implementation="cuda").to(DEV)
    x = torch.rand(256, 8000, device=DEV, requires_grad=True)
    y = layer(x)
    want = O.logic_fc_forward(x.detach().cpu(), layer.indices_0.cpu(), layer.indices_1.cpu(),
                              torch.softmax(layer.weights.detach().cpu(), -1))
    assert (y.detach().cpu() - want).abs().max().item() <= 1e-5
    g1, g2 = torch.randn_like(y), torch.randn_like(y)

    def grads(g):
        gx, gw = torch.autograd.grad(y, (x, layer.weights), g, retain_graph=True)
        return gx, gw

    a, b, ab, a_again = grads(g1), grads(g2), grads(g1 + g2), grads(g1)
    assert torch.equal(a[0], a_again[0]) and torch.equal(a[1], a_again[1])          # bitwise reproducible
    assert_grad_close(ab[0], a[0] + b[0], rel=1e-4, name="linearity grad_x")
    assert_grad_close(ab[1], a[1] + b[1], rel=1e-4, name="linearity grad_w")


def test_transpose_kernel():
    # small matrices take 32 x 32 tiles, from 2048 tiles of 64 x 64 on those: all four element sizes on both
    for shape, dt in (((7, 130), torch.float32), ((129, 64), torch.float64), ((3, 5), torch.int16), ((65, 66), torch.uint8),
                      ((3000, 3001), torch.float32), ((2900, 3100), torch.float64), ((3333, 2800), torch.int16), ((2950, 3050), torch.uint8)):
        t = (torch.rand(shape, device=DEV) * 100).to(dt)
        assert torch.equal(difflogic_hip.transpose(t), t.T.contiguous())


@pytest.mark.parametrize("batch,dtype", [(21, torch.float32), (30, torch.float32), (19, torch.float64), (31, torch.float64),
                                         (37, torch.float16), (60, torch.float16), (27, torch.float16)])
def test_fc_weight_gradient_with_one_sample_per_lane_and_ragged_rows(batch, dtype):
    # batches that no vector width divides take one sample per lane; 17 to 32 of them are a row of 32 lanes, more a row of 64:
    # the reference-shaped weight-gradient call against the oracle
    torch.manual_seed(batch)
    in_dim, out_dim = 24, 40
    layer = C.LogicLayer(in_dim, out_dim, implementation="cuda").to(DEV)
    x = torch.rand(in_dim, batch, device=DEV).to(dtype)
    gy = torch.randn(out_dim, batch, device=DEV).to(dtype)
    gw = difflogic_hip.backward_w(x, layer.indices_0, layer.indices_1, gy)
    assert gw.dtype == dtype and gw.shape == (out_dim, 16)
    xl = x.float().cpu().double().t().contiguous()
    wl = torch.full((out_dim, 16), 1 / 16, dtype=torch.float64, requires_grad=True)
    y = O.logic_fc_forward(xl, layer.indices_0.cpu(), layer.indices_1.cpu(), wl)
    y.backward(gy.float().cpu().double().t())
    tol = {torch.float32: 1e-5, torch.float64: 1e-12, torch.float16: 2e-3}[dtype]
    scale = wl.grad.abs().max().item()
    assert (gw.double().cpu() - wl.grad).abs().max().item() <= tol * scale + (1e-3 if dtype == torch.float16 else 0.0)


def test_fc_rejects_bad_inputs():
    layer = C.LogicLayer(8, 8, implementation="cuda").to(DEV)
    with pytest.raises(RuntimeError):
        difflogic_hip.forward(torch.rand(8, 4), layer.indices_0, layer.indices_1, torch.rand(8, 16, device=DEV))
    with pytest.raises(RuntimeError):
        difflogic_hip.forward(torch.rand(8, 4, device=DEV).bfloat16(), layer.indices_0, layer.indices_1,
                              torch.rand(8, 16, device=DEV).bfloat16())
    with pytest.raises(RuntimeError):                                   # half is a format of the reference-shaped kernels only
        difflogic_hip.fold(torch.rand(8, 16, device=DEV).half(), from_logits=True)
    with pytest.raises(RuntimeError):                                   # ... and so are the logits-in forward and the one-pass backward
        difflogic_hip.forward_logits(torch.rand(8, 4, device=DEV).half(), layer.indices_0, layer.indices_1,
                                     torch.rand(8, 16, device=DEV).half())
    with pytest.raises(RuntimeError):
        difflogic_hip.forward_logits(torch.rand(8, 4, device=DEV), layer.indices_0, layer.indices_1, torch.rand(8, 16, device=DEV).double())
    with pytest.raises(AssertionError):
        layer(torch.rand(2, 3, 8, device=DEV))


def test_fused_softmax_backward_matches_softmax_plus_function():
    # training path of the module (logits in, softmax inside, its backward fused into the weight-gradient
    # kernel) against the reference-shaped route softmax -> LogicLayerCudaFunction, float32 and float64
    from convlogic_amd.difflogic.difflogic import _LogicLayerLogitsFunction
    for dtype, tol in ((torch.float32, 2e-5), (torch.float64, 1e-12)):
        torch.manual_seed(7)
        layer = C.LogicLayer(40, 96, implementation="cuda").to(DEV).to(dtype)
        x = torch.rand(40, 33, device=DEV, dtype=dtype)
        gy = torch.randn(96, 33, device=DEV, dtype=dtype)
        outs = []
        for fused in (True, False):
            xl = x.clone().requires_grad_(True)
            logits = layer.weights.detach().clone().requires_grad_(True)
            tabs = (layer.indices_0, layer.indices_1)
            csr = (layer.given_x_indices_of_y_start, layer.given_x_indices_of_y)
            if fused:
                y = _LogicLayerLogitsFunction.apply(xl, *tabs, logits, *csr)
            else:
                y = C.LogicLayerCudaFunction.apply(xl, *tabs, torch.softmax(logits, -1), *csr)
            y.backward(gy)
            outs.append((y.detach(), xl.grad, logits.grad))
        # the softmax of the fused route is computed by the fold kernel, not by torch: equal up to rounding
        for got, want in zip(outs[0], outs[1]):
            scale = max(want.abs().max().item(), 1.0)
            assert (got - want).abs().max().item() <= tol * scale


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("in_dim,out_dim,batch", [(24, 50, 8), (24, 50, 60), (40, 96, 64), (40, 97, 100), (64, 131, 128),
                                                  (64, 130, 132), (30, 75, 256), (30, 75, 300), (7, 9, 33), (3, 5, 1)])
def test_folded_kernels_equal_probability_kernels(in_dim, out_dim, batch, dtype):
    # same probabilities in, bit-identical forward and input gradient out: the folded kernels only move the
    # folding out of the wavefronts and pack 64/16, 64/32 or 1 rows into a wavefront by batch size
    torch.manual_seed(in_dim + out_dim + batch)
    layer = C.LogicLayer(in_dim, out_dim, implementation="cuda").to(DEV).to(dtype)
    tabs = (layer.indices_0, layer.indices_1)
    csr = (layer.given_x_indices_of_y_start, layer.given_x_indices_of_y)
    x = torch.rand(in_dim, batch, device=DEV, dtype=dtype)
    gy = torch.randn(out_dim, batch, device=DEV, dtype=dtype)
    w = torch.softmax(layer.weights.detach(), -1)
    none, folded = difflogic_hip.fold(w, from_logits=False, want_probs=False)
    assert none is None
    assert torch.equal(difflogic_hip.forward_folded(x, *tabs, folded), difflogic_hip.forward(x, *tabs, w))
    assert torch.equal(difflogic_hip.backward_x_folded(x, *tabs, folded, gy, *csr),
                       difflogic_hip.backward_x(x, *tabs, w, gy, *csr))
    # the probabilities of the fold kernel against torch's softmax, the coefficients against the oracle's fold
    probs, folded_l = difflogic_hip.fold(layer.weights.detach(), from_logits=True)
    eps = 1e-6 if dtype == torch.float32 else 1e-14
    assert (probs - w).abs().max().item() <= eps
    coef = O.fold_coefficients(w.cpu().double())
    assert (folded_l.cpu().double() - coef).abs().max().item() <= 16 * eps
    # weight gradient at this batch size (rows per wavefront differ) against the oracle
    gw = difflogic_hip.backward_w(x, *tabs, gy)
    xl, gl = x.cpu().double(), gy.cpu().double()
    xa, xb = xl[layer.indices_0.cpu()], xl[layer.indices_1.cpu()]
    sums = torch.stack([(gl * xa * xb).sum(1), (gl * xa).sum(1), (gl * xb).sum(1), gl.sum(1)], 1)      # [out, 4]
    assert_grad_close(gw, (sums @ O.COEF).to(dtype), name="grad_w")


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("in_dim,out_dim,batch", [(24, 50, 8), (24, 50, 60), (40, 97, 100), (64, 131, 128), (30, 75, 256),
                                                  (70, 40, 64), (7, 9, 33), (3, 5, 1), (8000, 8000, 256), (16, 8, 12),
                                                  (6, 60, 12), (10, 100, 100), (7, 150, 256)])   # lists of 20 to 43 consumers
def test_fused_backward_equals_the_two_kernels(in_dim, out_dim, batch, dtype):
    # one walk over the consumer lists gives both gradients: bit for bit what the input-gradient kernel and the
    # weight-gradient kernel give separately (w.r.t. the probabilities and w.r.t. the logits), for 16 / 32 / 64 lanes
    # per row, inputs without consumers, and neurons that read the same feature twice; either layout of grad_x
    torch.manual_seed(in_dim * 3 + out_dim + batch)
    layer = C.LogicLayer(in_dim, out_dim, implementation="cuda").to(DEV).to(dtype)
    a, b = layer.indices_0.clone(), layer.indices_1.clone()
    b[::5] = a[::5]                                                  # some neurons wired to one feature twice
    layer = _layer_with(a.cpu(), b.cpu(), in_dim, dtype)
    tabs = (layer.indices_0, layer.indices_1)
    csr = (layer.given_x_indices_of_y_start, layer.given_x_indices_of_y)
    x = torch.rand(in_dim, batch, device=DEV, dtype=dtype)
    gy = torch.randn(out_dim, batch, device=DEV, dtype=dtype)
    probs, folded = difflogic_hip.fold(layer.weights.detach(), from_logits=True)
    fits = difflogic_hip.backward_fused_fits(x)
    assert fits == (batch <= (256 if dtype == torch.float32 and batch % 4 == 0 else 128 if dtype == torch.float64 and batch % 2 == 0 else 64))
    if not fits:
        with pytest.raises(RuntimeError, match="exceeds what one pass covers"):
            difflogic_hip.backward_fused(x, *tabs, folded, probs, gy, *csr)
        return
    gx_ref = difflogic_hip.backward_x_folded(x, *tabs, folded, gy, *csr)
    for p_arg, gw_ref in ((None, difflogic_hip.backward_w(x, *tabs, gy)), (probs, difflogic_hip.backward_logits(x, *tabs, probs, gy))):
        gx, gw = difflogic_hip.backward_fused(x, *tabs, folded, p_arg, gy, *csr)
        assert torch.equal(gx, gx_ref) and torch.equal(gw, gw_ref)
        # the same sums with the input gradient written [batch, in] by the kernel itself
        gx_sm, gw_sm = difflogic_hip.backward_fused(x, *tabs, folded, p_arg, gy, *csr, sample_major_grad_x=True)
        assert gx_sm.shape == (batch, in_dim) and torch.equal(gx_sm, gx_ref.t()) and torch.equal(gw_sm, gw_ref)
        # ... and with grad_y handed over as [batch, out] (its feature-major copy made inside the call)
        gx_io, gw_io = difflogic_hip.backward_fused(x, *tabs, folded, p_arg, gy.t().contiguous(), *csr, sample_major_grad_x=True,
                                                    sample_major_grad_y=True)
        assert torch.equal(gx_io, gx_sm) and torch.equal(gw_io, gw_ref)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("in_dim,out_dim,batch", [(24, 50, 8), (40, 97, 100), (64, 131, 128), (30, 75, 256), (30, 75, 300),
                                                  (7, 9, 33), (3, 5, 1), (8000, 8000, 256)])
def test_forward_from_logits_folds_inside(in_dim, out_dim, batch, dtype):
    # one launch for softmax + fold + forward: probabilities against torch's softmax, coefficients against the oracle's
    # fold of those probabilities, and y bit for bit what the folded forward gives on the coefficients written out
    torch.manual_seed(in_dim + 2 * out_dim + batch)
    layer = C.LogicLayer(in_dim, out_dim, implementation="cuda").to(DEV).to(dtype)
    tabs = (layer.indices_0, layer.indices_1)
    x = torch.rand(in_dim, batch, device=DEV, dtype=dtype)
    logits = (torch.randn(out_dim, 16, device=DEV, dtype=dtype) * 3).contiguous()
    y, probs, folded = difflogic_hip.forward_logits(x, *tabs, logits)
    eps = 1e-6 if dtype == torch.float32 else 1e-14
    assert (probs - torch.softmax(logits, -1)).abs().max().item() <= eps
    assert (folded.cpu().double() - O.fold_coefficients(probs.cpu().double())).abs().max().item() <= 16 * eps
    assert torch.equal(y, difflogic_hip.forward_folded(x, *tabs, folded))
    want = O.logic_fc_forward(x.T.cpu(), layer.indices_0.cpu(), layer.indices_1.cpu(), torch.softmax(logits.cpu(), -1))
    assert (y.T.cpu() - want).abs().max().item() <= (1e-5 if dtype == torch.float32 else 1e-12)
    # handed a [batch, in] tensor, the same call makes the feature-major copy first: same outputs, and the copy comes back
    y2, probs2, folded2, x_fm = difflogic_hip.forward_logits(x.t().contiguous(), *tabs, logits, sample_major_x=True)
    assert torch.equal(x_fm, x) and torch.equal(y2, y) and torch.equal(probs2, probs) and torch.equal(folded2, folded)
    with pytest.raises(RuntimeError):
        difflogic_hip.forward_logits(x, *tabs, logits[:, :8].contiguous())


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("features,batch,k,once", [(10240, 256, 10, True), (640, 256, 10, True), (3200, 37, 50, True), (40960, 130, 10, True),
                                                   (40, 7, 4, False), (630, 256, 10, False), (640, 32, 10, False), (81920, 64, 10, False)])
def test_group_sum_in_one_launch(features, batch, k, once, dtype):
    # classes of 64 to 4096 rows with enough (class, 32 samples) pairs take the kernel without partial sums: same sums as
    # the sliced kernels up to rounding, exact on 0/1 activations, ragged batches, reproducible; other sizes are refused
    from convlogic_amd.hip import _lib
    lib = _lib.load()
    assert bool(lib.clg_group_sum_once_fits(features, batch, k)) == once
    torch.manual_seed(features + batch)
    x = torch.rand(features, batch, device=DEV, dtype=dtype)
    dt, st = _lib.dtype_code(x), _lib.stream_ptr(x)
    out = torch.full((batch, k), float("nan"), device=DEV, dtype=dtype)
    rc = lib.clg_group_sum_once(dt, x.data_ptr(), out.data_ptr(), features, batch, k, 6.5, st)
    if not once:
        assert rc != 0 and b"clg_group_sum_once_fits" in lib.clg_last_error()
        return
    assert rc == 0
    ref = x.double().reshape(k, features // k, batch).sum(1).t() / 6.5
    assert (out.double() - ref).abs().max().item() <= (1e-5 if dtype == torch.float32 else 1e-13) * ref.abs().max().item()
    scratch = torch.empty(lib.clg_group_sum_scratch_bytes(dt, features, batch, k), dtype=torch.uint8, device=DEV)
    sliced = torch.empty_like(out)
    _lib.check(lib.clg_group_sum(dt, x.data_ptr(), sliced.data_ptr(), scratch.data_ptr(), features, batch, k, 6.5, st))
    assert torch.allclose(out, sliced, rtol=1e-5 if dtype == torch.float32 else 1e-13, atol=0)
    again = torch.empty_like(out)
    _lib.check(lib.clg_group_sum_once(dt, x.data_ptr(), again.data_ptr(), features, batch, k, 6.5, st))
    assert torch.equal(out, again)
    bits = (x > 0.5).to(dtype)
    _lib.check(lib.clg_group_sum_once(dt, bits.data_ptr(), out.data_ptr(), features, batch, k, 1.0, st))
    assert torch.equal(out.cpu(), bits.cpu().reshape(k, features // k, batch).sum(1).t())


@pytest.mark.parametrize("features,batch,k", [(40, 7, 4), (640, 256, 10), (65536, 100, 8), (30, 1, 3), (10240, 256, 10)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_group_sum_on_feature_major_view(features, batch, k, dtype):
    # GroupSum behind a LogicLayer receives the transposed view of a feature-major tensor: summed by the HIP
    # kernels in that layout (fixed order), gradient handed back as a transposed view
    torch.manual_seed(features + batch)
    fm = torch.rand(features, batch, device=DEV, dtype=dtype)
    x = fm.transpose(0, 1).requires_grad_(True)
    gs = C.GroupSum(k, tau=6.5)
    y = gs(x)
    ref_in = fm.transpose(0, 1).contiguous().cpu().requires_grad_(True)
    ref = O.group_sum(ref_in, k, 6.5)
    assert y.shape == (batch, k)
    assert torch.allclose(y.detach().cpu(), ref.detach(), rtol=1e-5 if dtype == torch.float32 else 1e-12, atol=0)
    g = torch.randn(batch, k, device=DEV, dtype=dtype)
    y.backward(g)
    ref.backward(g.cpu())
    assert torch.allclose(x.grad.cpu(), ref_in.grad, rtol=1e-6 if dtype == torch.float32 else 1e-14, atol=0)
    # binary activations: integer sums are exact, so the packed counts still equal tau * y
    bits = (fm > 0.5).to(dtype)
    counts = C.GroupSum(k, tau=1.0)(bits.transpose(0, 1))
    assert torch.equal(counts.cpu(), bits.cpu().transpose(0, 1).reshape(batch, k, features // k).sum(-1))
    assert torch.equal(gs(x.detach()), gs(x.detach()))             # reproducible


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("out_dim,batch", [(16, 8), (50, 60), (64, 128), (33, 100), (200, 256), (75, 300), (9, 33), (1, 1)])
def test_halving_layer_gradients_come_from_one_pass(out_dim, batch, dtype):
    # 2*out == in with the reference's random wiring reads every input exactly once: the fused kernel must give
    # the gradients of the two separate kernels bit for bit, and the module must pick it by itself
    from convlogic_amd.difflogic.difflogic import _LogicLayerLogitsFunction
    torch.manual_seed(out_dim * 7 + batch)
    in_dim = 2 * out_dim
    layer = C.LogicLayer(in_dim, out_dim, implementation="cuda").to(DEV).to(dtype)
    assert layer._sole_consumers()
    tabs = (layer.indices_0, layer.indices_1)
    csr = (layer.given_x_indices_of_y_start, layer.given_x_indices_of_y)
    x = torch.rand(in_dim, batch, device=DEV, dtype=dtype)
    gy = torch.randn(out_dim, batch, device=DEV, dtype=dtype)
    probs, folded = difflogic_hip.fold(layer.weights.detach(), from_logits=True)
    gx, gl = difflogic_hip.backward_sole(x, *tabs, folded, probs, gy)
    assert torch.equal(gx, difflogic_hip.backward_x_folded(x, *tabs, folded, gy, *csr))
    assert torch.equal(gl, difflogic_hip.backward_logits(x, *tabs, probs, gy))
    gx2, gw = difflogic_hip.backward_sole(x, *tabs, folded, None, gy)
    assert torch.equal(gx2, gx) and torch.equal(gw, difflogic_hip.backward_w(x, *tabs, gy))
    # through the module, against the oracle
    xm = x.t().contiguous().requires_grad_(True)
    layer(xm).backward(gy.t().contiguous())
    _, gx_ref, gl_ref = _oracle_grads(xm, layer.weights, layer.indices_0, layer.indices_1, gy.t())
    assert_grad_close(xm.grad, gx_ref.to(dtype), name="grad_x")
    assert_grad_close(layer.weights.grad, gl_ref.to(dtype), name="grad_logits")


def test_halving_layer_with_shared_inputs_keeps_the_gather():
    # same sizes, but one input is wired twice and another never: the one-pass kernel would drop a term, so the
    # module has to notice (also after an in-place rewiring of a layer it had already classified)
    from convlogic_amd.difflogic.difflogic import _reverse_wiring
    torch.manual_seed(11)
    layer = C.LogicLayer(24, 12, implementation="cuda").to(DEV)
    assert layer._sole_consumers()
    idx0, idx1 = layer.indices_0.cpu().clone(), layer.indices_1.cpu().clone()
    idx1[5] = idx0[2]                                                # idx0[2] now read twice, old idx1[5] never
    layer.indices_1.copy_(idx1.to(DEV))
    s, f = _reverse_wiring(idx0.numpy(), idx1.numpy(), 24)
    layer.given_x_indices_of_y_start.copy_(s.to(DEV))
    layer.given_x_indices_of_y.copy_(f.to(DEV))
    assert not layer._sole_consumers()
    x = torch.rand(40, 24, device=DEV, requires_grad=True)
    gy = torch.randn(40, 12, device=DEV)
    layer(x).backward(gy)
    _, gx_ref, gl_ref = _oracle_grads(x, layer.weights, idx0, idx1, gy)
    assert_grad_close(x.grad, gx_ref, name="grad_x")
    assert_grad_close(layer.weights.grad, gl_ref, name="grad_logits")


@pytest.mark.parametrize("in_dim,out_dim,batch", [(12, 16, 5), (40, 96, 64), (100, 64, 256), (33, 40, 264)])
def test_fc_half_storage(in_dim, out_dim, batch):
    # float16 tensors through the module (the reference dispatches its LogicLayer kernels for half too,
    # src/difflogic/cuda/difflogic_kernel.cu:108,146,249): values are stored as half and computed in float32, so the
    # result equals the float32 oracle on the half-rounded inputs up to the rounding of the outputs.  The reference
    # has no test of this format: parity unpinned by the reference, pinned here by the float32 path.
    torch.manual_seed(batch + in_dim)
    layer = C.LogicLayer(in_dim, out_dim, implementation="cuda").to(DEV)
    x = torch.rand(batch, in_dim, device=DEV).half().requires_grad_(True)
    gy = torch.randn(batch, out_dim, device=DEV).half()
    y = layer(x)
    assert y.dtype == torch.float16 and y.shape == (batch, out_dim)
    y.backward(gy)
    w16 = torch.softmax(layer.weights.detach(), -1).half().float().cpu()
    xl = x.detach().float().cpu().requires_grad_(True)
    wl = w16.clone().requires_grad_(True)
    y_ref = O.logic_fc_forward(xl, layer.indices_0.cpu(), layer.indices_1.cpu(), wl)
    y_ref.backward(gy.float().cpu())
    assert (y.detach().float().cpu() - y_ref.detach()).abs().max().item() <= 1e-3
    scale = xl.grad.abs().max().item()
    assert (x.grad.float().cpu() - xl.grad).abs().max().item() <= 2e-3 * scale + 1e-3
    # weight gradient as the kernel returns it (w.r.t. the half probabilities), before the softmax's autograd node
    xt = x.detach().t().contiguous()
    gw = difflogic_hip.backward_w(xt, layer.indices_0, layer.indices_1, gy.t().contiguous())
    assert gw.dtype == torch.float16
    scale = wl.grad.abs().max().item()
    assert (gw.float().cpu() - wl.grad).abs().max().item() <= 2e-3 * scale + 1e-3
    assert torch.isfinite(layer.weights.grad).all()
    # eval mode: binary inputs give exactly 0/1 in half as well
    layer.eval()
    yb = layer(torch.randint(0, 2, (batch, in_dim), device=DEV).half())
    assert torch.all((yb == 0) | (yb == 1))


def test_fc_half_layer_trains_on_half_input():
    # layer.half() with a float16 batch (the reference dispatches forward / backward for half,
    # src/difflogic/cuda/difflogic_kernel.cu:108,146,249, with w = softmax(weights).to(x.dtype)): forward and both
    # gradients against the float32 oracle on the half-rounded tensors
    torch.manual_seed(21)
    layer = C.LogicLayer(48, 64, implementation="cuda").to(DEV).half()
    x = torch.rand(40, 48, device=DEV).half().requires_grad_(True)
    gy = torch.randn(40, 64, device=DEV).half()
    y = layer(x)
    assert y.dtype == torch.float16
    y.backward(gy)
    assert layer.weights.grad is not None and layer.weights.grad.dtype == torch.float16
    xl = x.detach().float().cpu().requires_grad_(True)
    ll = layer.weights.detach().float().cpu().requires_grad_(True)
    w = torch.softmax(ll, -1)
    y_ref = O.logic_fc_forward(xl, layer.indices_0.cpu(), layer.indices_1.cpu(), w)
    y_ref.backward(gy.float().cpu())
    assert (y.detach().float().cpu() - y_ref.detach()).abs().max().item() <= 2e-3
    assert (x.grad.float().cpu() - xl.grad).abs().max().item() <= 4e-3 * xl.grad.abs().max().item() + 1e-3
    assert (layer.weights.grad.float().cpu() - ll.grad).abs().max().item() <= 1e-2 * ll.grad.abs().max().item() + 1e-3


def test_fc_bindings_reject_mismatched_tensors():
    # the kernels read raw pointers: a tensor of another element type or shape must raise, as the reference's typed
    # accessors do, instead of being read out of bounds
    layer = C.LogicLayer(16, 24, implementation="cuda").to(DEV)
    xt = torch.rand(16, 8, device=DEV)
    a, b = layer.indices_0, layer.indices_1
    w = torch.softmax(layer.weights.detach(), -1)
    with pytest.raises(RuntimeError, match="dtype"):
        difflogic_hip.forward(xt.double(), a, b, w)                  # float32 probabilities with float64 x
    with pytest.raises(RuntimeError, match="dtype"):
        difflogic_hip.forward(xt, a.int(), b, w)                     # int32 wiring
    with pytest.raises(RuntimeError, match="shape"):
        difflogic_hip.forward(xt, a[:-1].contiguous(), b, w)
    with pytest.raises(RuntimeError, match="shape"):
        difflogic_hip.backward_w(xt, a, b, torch.rand(24, 9, device=DEV))
    with pytest.raises(RuntimeError, match="shape"):
        difflogic_hip.backward_x(xt, a, b, w, torch.rand(24, 8, device=DEV), layer.given_x_indices_of_y_start[:-1].contiguous(),
                                 layer.given_x_indices_of_y)
    with pytest.raises(RuntimeError):
        difflogic_hip.eval(torch.zeros(16, 4, dtype=torch.int64, device=DEV), a, b, torch.zeros(24, dtype=torch.int64, device=DEV))


def test_fc_rewired_out_of_range_raises_instead_of_launching():
    layer = C.LogicLayer(16, 24, implementation="cuda").to(DEV)
    x = torch.rand(8, 16, device=DEV)
    layer(x)
    layer.indices_0[5] = 16
    with pytest.raises(ValueError, match="indices_0"):
        layer(x)
    layer.eval()
    with pytest.raises(ValueError, match="indices_0"):
        layer(C.PackBitsTensor(x > 0.5, 64))


def test_fc_rewired_in_range_rebuilds_the_reverse_map():
    # an in-place rewiring (version counter) must reach the input gradient: the reverse map is rebuilt from the indices
    torch.manual_seed(31)
    layer = C.LogicLayer(20, 30, implementation="cuda").to(DEV)
    x = torch.rand(8, 20, device=DEV, requires_grad=True)
    layer(x).sum().backward()
    layer.indices_0[7] = 3
    layer.indices_1[11] = 19
    x.grad = None
    gy = torch.randn(8, 30, device=DEV)
    layer(x).backward(gy)
    xl = x.detach().cpu().requires_grad_(True)
    O.logic_fc_forward(xl, layer.indices_0.cpu(), layer.indices_1.cpu(), torch.softmax(layer.weights.detach().cpu(), -1)).backward(gy.cpu())
    assert_grad_close(x.grad, xl.grad, name="grad_x after rewiring")


def test_fc_index_corrupted_behind_the_host_check_is_clamped_not_faulting():
    # a write through `.data` is invisible to the cached host check: the kernels force every index into range, so the
    # call returns (reading a wrong row) instead of faulting the GPU -- forward, both gradients and the packed path
    torch.manual_seed(32)
    layer = C.LogicLayer(16, 24, implementation="cuda").to(DEV)
    x = torch.rand(8, 16, device=DEV, requires_grad=True)
    layer(x).sum().backward()                                        # host checks are now cached
    layer.eval()
    layer(C.PackBitsTensor(x.detach() > 0.5, 64))                    # ... and so is the walk plan of the packed path
    layer.train()
    layer.indices_0.data[5] = 1 << 40
    layer.indices_1.data[6] = -3
    y = layer(x)
    y.sum().backward()
    torch.cuda.synchronize()
    clamped = layer.indices_0.clamp(0, 15), layer.indices_1.clamp(0, 15)
    want = O.logic_fc_forward(x.detach().cpu(), clamped[0].cpu(), clamped[1].cpu(), torch.softmax(layer.weights.detach().cpu(), -1))
    assert (y.detach().cpu() - want).abs().max().item() <= 1e-5
    assert torch.isfinite(x.grad).all() and torch.isfinite(layer.weights.grad).all()
    layer.eval()
    bits = x.detach() > 0.5
    out = layer(C.PackBitsTensor(bits, 64)).t                        # packed path on the cached plan: clamped as well
    torch.cuda.synchronize()
    import numpy as np
    words, _ = O.pack_bits(bits.cpu().numpy().T, 64)
    want_words = O.eval_packed(words, clamped[0].cpu().numpy(), clamped[1].cpu().numpy(), layer.weights.argmax(-1).cpu().numpy().astype(np.uint8))
    assert np.array_equal(out.cpu().numpy(), want_words)
    # invalidate() brings the host check back
    layer.invalidate()
    with pytest.raises(ValueError, match="indices_0"):
        layer(x)


def test_packed_gates_follow_in_place_weight_updates():
    # the arg-max gates of the packed path are taken from the logits on every call: an update through `.data`
    # (EMA swap, legacy optimiser), which no version counter sees, must change the evaluated network
    torch.manual_seed(23)
    layer = C.LogicLayer(32, 48, implementation="cuda").to(DEV).eval()
    bits = torch.randint(0, 2, (100, 32), device=DEV).bool()
    before = layer(C.PackBitsTensor(bits, 64)).t.clone()
    new = torch.randn_like(layer.weights)
    layer.weights.data.copy_(new)
    after = layer(C.PackBitsTensor(bits, 64)).t
    words, _ = O.pack_bits(bits.cpu().numpy().T, 64)
    import numpy as np
    want = O.eval_packed(words, layer.indices_0.cpu().numpy(), layer.indices_1.cpu().numpy(),
                         new.argmax(-1).cpu().numpy().astype(np.uint8))
    assert np.array_equal(after.cpu().numpy(), want) and not torch.equal(before, after)
    # ties and the first-maximum rule of the arg-max kernel
    logits = torch.zeros(5, 16, device=DEV)
    logits[1, 7] = logits[1, 9] = 2.0
    logits[2, 15] = 1.0
    logits[3] = -1.0
    logits[4, 3] = float("nan")
    got = difflogic_hip.gate_argmax(logits)
    assert got.tolist() == [0, 7, 15, 0, 3] and got.dtype == torch.uint8
    assert torch.equal(difflogic_hip.gate_argmax(new).long(), new.argmax(-1))
    assert torch.equal(difflogic_hip.gate_argmax(new.double()).long(), new.argmax(-1))
    assert torch.equal(difflogic_hip.gate_argmax(new.half()).long(), new.half().argmax(-1))
