"""Oracle parity at the exact BASELINE shapes, batch 256: forward and BOTH gradients of the kernels and launch
plans that bench.py times (samples per workgroup, kernel-list splits, padded weight gradient and fused FC
backward are all chosen from the batch size, so a smaller batch checks other instantiations).

The oracle runs in float64 on the same float32 inputs: the reference value is then exact to ~1e-16 and the whole
difference is the float32 rounding of the HIP path.  Tolerances: forward 1e-5 absolute, gradients 1e-4 relative
(the three bounds of tests/gpu_util.assert_grad_close).  The pooled route of the GPU is followed (near ties
between different tap patterns are counted and bounded, tests/gpu_util.check_pool_route)."""
import pytest
import torch

import convlogic_amd as C
from convlogic_amd.hip import convlogic_hip
from oracle import convlogic_oracle as O
from tests.gpu_util import DEV, assert_grad_close, block_oracle, check_pool_route

pytestmark = pytest.mark.gpu


def _c4_input(n, seed):
    g = torch.Generator().manual_seed(seed)
    v = (torch.randn(n, 3, 32, 32, generator=g) * 0.25 + 0.5).clamp(0, 1)
    return torch.cat([(v > t).float() for t in (0.25, 0.5, 0.75)], dim=1)


def test_config1_fc_256x8000_forward_and_gradients_vs_oracle():
    torch.manual_seed(101)
    layer = C.LogicLayer(8000, 8000, implementation="cuda").to(DEV)
    x = torch.rand(256, 8000, device=DEV, requires_grad=True)
    gy = torch.randn(256, 8000, device=DEV)
    y = layer(x)
    y.backward(gy)
    xl = x.detach().cpu().double().requires_grad_(True)
    ll = layer.weights.detach().cpu().double().requires_grad_(True)
    want = O.logic_fc_forward(xl, layer.indices_0.cpu(), layer.indices_1.cpu(), torch.softmax(ll, -1))
    want.backward(gy.cpu().double())
    assert (y.detach().cpu().double() - want.detach()).abs().max().item() <= 1e-5
    assert_grad_close(x.grad, xl.grad, name="grad_x")
    assert_grad_close(layer.weights.grad, ll.grad, name="grad_logits")
    # and the reference-shaped Function (probabilities in, feature-major tensors) on the same data
    xt = x.detach().t().contiguous().requires_grad_(True)
    w = torch.softmax(layer.weights.detach(), -1).requires_grad_(True)
    yt = C.LogicLayerCudaFunction.apply(xt, layer.indices_0, layer.indices_1, w, layer.given_x_indices_of_y_start,
                                        layer.given_x_indices_of_y)
    yt.backward(gy.t().contiguous())
    wl = torch.softmax(ll.detach(), -1).requires_grad_(True)
    want2 = O.logic_fc_forward(xl.detach(), layer.indices_0.cpu(), layer.indices_1.cpu(), wl)
    want2.backward(gy.cpu().double())
    assert (yt.detach().t().cpu().double() - want2.detach()).abs().max().item() <= 1e-5
    assert_grad_close(xt.grad.t(), xl.grad, name="grad_x (Function)")
    assert_grad_close(w.grad, wl.grad, name="grad_w (Function)")


def _block_full_size(n, cin, cout, size, x, seed, chunk):
    """Fused block through the module at batch n against the float64 oracle evaluated in sample chunks."""
    torch.manual_seed(seed)
    layer = C.ConvLogicLayer(cin, cout, padding=1, complete=True, implementation="cuda").to(DEV)
    xg = x.to(DEV).requires_grad_(True)
    y = layer(xg)                                                   # training path: logits in, fused softmax backward
    gy = torch.randn_like(y)
    y.backward(gy)
    # the route the GPU took, from the same kernels on the same input (deterministic)
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
    return layer, xg, gy


def test_config3_block_256x1x28x28_forward_and_gradients_vs_oracle():
    g = torch.Generator().manual_seed(3)
    x = torch.randint(0, 2, (256, 1, 28, 28), generator=g).float()
    _block_full_size(256, 1, 32, 28, x, seed=33, chunk=256)


@pytest.mark.timeout(600)
def test_config4_block_256x9x32x32_forward_and_gradients_vs_oracle():
    _block_full_size(256, 9, 256, 32, _c4_input(256, 4), seed=44, chunk=32)


@pytest.mark.timeout(600)
def test_config4_reference_shaped_function_vs_oracle_along_its_own_route():
    # the reference-shaped pair of calls (probabilities from torch.softmax in, gradient w.r.t. the probabilities out) at
    # full C4: forward and both gradients against the float64 oracle evaluated along the route THIS call pooled
    torch.manual_seed(45)
    n, cin, cout, size, chunk = 256, 9, 256, 32, 32
    layer = C.ConvLogicLayer(cin, cout, complete=True, implementation="cuda").to(DEV)
    w = torch.softmax(layer.weights.detach(), -1).requires_grad_(True)
    x = _c4_input(n, 4).to(DEV).requires_grad_(True)
    y, idx = C.FullConvLogicFunction.apply(x, w, layer.selection, 1, 1, 1, 1, 3, 3, False, True)
    gy = torch.randn_like(y)
    y.backward(gy)
    gw_ref = torch.zeros(cout, 7, 16, dtype=torch.float64)
    flips = 0
    for s0 in range(0, n, chunk):
        sl = slice(s0, s0 + chunk)
        xl = x.detach()[sl].cpu().double().requires_grad_(True)
        wl = w.detach().cpu().double().requires_grad_(True)
        y_ref, _, x3, idx_ref = O.conv_block_forward(xl, wl, layer.selection.cpu(), (1, 1), (1, 1), (3, 3), return_all=True)
        x4 = O.tree_forward(x3, wl[:, 6:7]).squeeze(-1)
        flips += check_pool_route(idx[sl], idx_ref, x4)
        routed = x4.flatten(2).gather(2, idx[sl].cpu().long()).view_as(y_ref)
        assert (y.detach()[sl].cpu().double() - routed.detach()).abs().max().item() <= 1e-5, s0
        routed.backward(gy[sl].cpu().double())
        assert_grad_close(x.grad[sl], xl.grad, name=f"grad_x[{s0}:]")
        gw_ref += wl.grad
    assert flips <= 1e-4 * idx.numel(), flips
    assert_grad_close(w.grad, gw_ref, name="grad_w")


def _config5_network_step(residual_init, binary_first_block):
    """the k = 32 CIFAR topology (4 blocks, flatten, 3 LogicLayers, GroupSum(10, 6.5)), one cross-entropy training step in
    float32 at batch 256: scores, loss and every layer's logit gradient against the float64 oracle routed through the
    pooling choices of the GPU.  -> (pool-route flips per block, pooled cells per block, check(rel_elem))"""
    from tests.test_gpu_model import build
    torch.manual_seed(55)
    model = build(residual_init=residual_init).to(DEV)
    model[0].binary_input = binary_first_block
    n = 256
    x = _c4_input(n, 5)
    labels = torch.randint(0, 10, (n,), generator=torch.Generator().manual_seed(6))
    xg = x.to(DEV).requires_grad_(True)
    # forward layer by layer, keeping the pooling route of every block (same kernels as the module call: deterministic)
    routes, h = [], xg
    for m in model:
        if isinstance(m, C.ConvLogicLayer):
            _, argmax, _ = convlogic_hip.full_convlogic_forward_logits(h.detach().contiguous(), m.weights.detach(), m.selection,
                                                                       1, 1, 1, 1, 3, 3)
            routes.append(convlogic_hip.argmax_to_indices(argmax, h.shape[3]).cpu().long())
        h = m(h)
    scores = h
    loss = torch.nn.functional.cross_entropy(scores, labels.to(DEV))
    loss.backward()

    # the oracle in chunks of 64 samples (every sample is independent of the others; the chunk losses add up to the
    # batch mean and the leaves collect the summed gradients)
    params = [m for m in model if hasattr(m, "weights")]
    leaves = [m.weights.detach().cpu().double().requires_grad_(True) for m in params]
    flips, cells, ref_loss, ref_scores, ref_gx = [0] * 4, [0] * 4, 0.0, [], []
    for s0 in range(0, n, 64):
        sl = slice(s0, s0 + 64)
        xc = x[sl].double().requires_grad_(True)
        ref, k = xc, 0
        for m in model:
            if isinstance(m, C.ConvLogicLayer):
                w = torch.softmax(leaves[k], -1)
                y_ref, _, x3, idx_ref = O.conv_block_forward(ref, w, m.selection.cpu(), (1, 1), (1, 1), (3, 3), return_all=True)
                x4 = O.tree_forward(x3, w[:, 6:7]).squeeze(-1)
                flips[k] += check_pool_route(routes[k][sl], idx_ref, x4)    # asserts |gap| <= 1e-5 where the routes differ
                cells[k] += idx_ref.numel()
                ref = x4.flatten(2).gather(2, routes[k][sl]).view_as(y_ref)
                k += 1
            elif isinstance(m, torch.nn.Flatten):
                ref = ref.flatten(1)
            elif isinstance(m, C.LogicLayer):
                ref = O.logic_fc_forward(ref, m.indices_0.cpu(), m.indices_1.cpu(), torch.softmax(leaves[k], -1))
                k += 1
            else:
                ref = O.group_sum(ref, m.k, m.tau)
        chunk_loss = torch.nn.functional.cross_entropy(ref, labels[sl], reduction="sum") / n
        chunk_loss.backward()
        ref_loss += chunk_loss.item()
        ref_scores.append(ref.detach())
        ref_gx.append(xc.grad)
    # Where the GPU pooled another window position than the float64 oracle the two values are within 1e-5 (asserted
    # above).  On the binary input of the first block such near ties between different tap patterns are rare; deeper
    # into a random-init network the activations of neighbouring positions agree to float32 rounding in a sizeable
    # share of the windows (measured: several percent), which is why the oracle follows the GPU's route.
    print("pool route flips per block:", flips, "of", cells)
    # scores are sums of 1024 gate outputs / 6.5: 1e-5 per value allows 1.6e-3; measured differences are ~1e-5
    assert (scores.detach().cpu().double() - torch.cat(ref_scores)).abs().max().item() <= 1e-4
    assert abs(loss.item() - ref_loss) <= 1e-5

    def check(rel_elem):
        worst = []
        for i, (m, leaf) in enumerate(zip(params, leaves)):
            got, ref = m.weights.grad.detach().double().cpu(), leaf.grad
            worst.append(((got - ref).abs() / (ref.abs() + ref.abs().mean() + 1e-30)).max().item())
        print("worst per-element relative error of grad_logits per layer:", ["%.2e" % w for w in worst])
        for i, (m, leaf) in enumerate(zip(params, leaves)):
            assert_grad_close(m.weights.grad, leaf.grad, name=f"layer {i} grad_logits", rel_elem=rel_elem)
        assert_grad_close(xg.grad, torch.cat(ref_gx), name="grad_x", rel_elem=rel_elem)

    return flips, cells, check


@pytest.mark.timeout(900)
def test_config5_network_batch256_float32_vs_oracle():
    # random-init logits (BASELINE config 5).  Deep into a random-init network the activations of neighbouring positions
    # agree to float32 rounding in a sizeable share of the windows, so only the first block's route is bounded; the
    # per-element bound against the MEAN magnitude is 5e-4: the gradients of the early layers (~1e-11) have passed
    # through up to seven float32 layers, each within 1e-4 on its own (measured worst element: 1.4e-4 in the second block)
    flips, cells, check = _config5_network_step(residual_init=False, binary_first_block=False)
    assert flips[0] <= 1e-4 * cells[0], (flips, cells)
    check(5e-4)


@pytest.mark.timeout(900)
@pytest.mark.parametrize("binary_first_block", [True, False])
def test_config5_network_residual_init_vs_oracle(binary_first_block):
    # the reference's own initialisation (residual_init=True, src/convlogic/model.py:36,55), the first block on the
    # binary-input kernels as in the model topologies.  Every kernel starts as (almost) the pass-through gate A, so the
    # activations take few distinct levels and the four positions of a pooling window are often EQUAL up to rounding: which
    # of them wins is then decided by the last bit, in float32 here and in float64 in the oracle (measured: 8 %, 22 % and
    # 33 % of the windows of blocks 2-4 pick another position, every one of them within the 1e-5 value gap that
    # check_pool_route asserts; block 1, on binary inputs, has none).  The per-element bound against the mean magnitude is
    # 5e-4 as for the random-init network: measured worst element 2.4e-4 (first block) with the binary-input kernels and
    # with the any-input kernels alike -- float32 rounding through seven layers, not a property of either path.
    flips, cells, check = _config5_network_step(residual_init=True, binary_first_block=binary_first_block)
    assert flips[0] <= 1e-4 * cells[0], (flips, cells)
    check(5e-4)
