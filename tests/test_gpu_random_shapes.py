"""Seeded random shapes through the module interfaces, beyond the fixed matrices of the other files: the fused block, the
LogicLayer (+ GroupSum), the packed stack and whole networks, each against the CPU oracle or against the promise the
package makes about its own variants (the module's training path bit-equal in the forward to the reference-shaped Function,
reproducible steps, network-level shortcuts that change nothing).  Shapes are drawn from a fixed seed, so every run tests the same cases;
float32 forward within 1e-5 of the value scale, gradients within 1e-4 (L2 and per element against the largest magnitude),
float64 within 1e-12 / 1e-10, packed words and counts exact."""
import random

import numpy as np
import pytest
import torch

import convlogic_amd as C
from convlogic_amd.convlogic import binarize
from convlogic_amd.difflogic.difflogic import LogicLayerCudaFunction, logic_layer_group_sum
from oracle import convlogic_oracle as O
from tests.gpu_util import DEV, block_oracle, check_pool_route

pytestmark = pytest.mark.gpu


def _tolerances(dtype):
    return (1e-5, 1e-4) if dtype == torch.float32 else (1e-12, 1e-10)


def _grad_close(got, ref, rel, what):
    got, ref = got.detach().double().cpu(), ref.detach().double().cpu()
    assert got.shape == ref.shape, (what, got.shape, ref.shape)
    scale = ref.abs().max().item() + 1e-30
    err = (got - ref).abs()
    assert (err <= rel * (ref.abs() + scale)).all(), (what, err.max().item(), scale)
    assert (got - ref).norm().item() <= rel * (ref.norm().item() + 1e-30), (what, "L2")


def _grad_close_or_as_good_as_float32(got, ref32, ref64, rel, what):
    """_grad_close against the oracle in the tensors' own precision; where cancellation (the softmax backward of a peaked
    distribution, sums of terms of both signs) makes that oracle itself lose more than the bound, the kernel has to be within
    four times the float32 oracle's distance from the float64 oracle."""
    try:
        _grad_close(got, ref32, rel, what)
    except AssertionError:
        r64 = ref64().detach().double().cpu()
        lost = (ref32.detach().double().cpu() - r64).abs().max().item()
        mine = (got.detach().double().cpu() - r64).abs().max().item()
        assert got.dtype == torch.float32 and mine <= 4 * lost + 1e-12, (what, mine, lost)


def _block_cases(seed, count):
    rng = random.Random(seed)
    while count:
        stride, kernel, pad = rng.choice([1, 1, 1, 2]), rng.choice([2, 3, 3, 3, 4, 5]), rng.choice([0, 1, 1, 2])
        pad = min(pad, kernel - 1)
        sizes = [v for v in (4, 6, 8, 10, 12, 16, 20, 24, 28, 32, 34, 40)
                 if v + 2 * pad >= kernel and ((v + 2 * pad - kernel) // stride + 1) % 2 == 0]
        if not sizes:
            continue
        h, w = rng.choice(sizes), rng.choice(sizes)
        cells = ((h + 2 * pad - kernel) // stride + 1) * ((w + 2 * pad - kernel) // stride + 1)
        budget = 300000 // cells
        n = rng.choice([1, 2, 3, 5, 8, 16, 31, 32, 33, 64, 70])
        cout = max(1, min(rng.choice([1, 2, 3, 5, 8, 16, 32, 33, 64, 100, 128, 256, 300]), budget // n))
        n = max(1, min(n, budget // cout))
        binary = rng.random() < 0.4
        yield dict(n=n, cin=rng.choice([1, 1, 2, 3, 4, 7, 8, 9, 16, 31, 32, 40, 64]), cout=cout, h=h, w=w, stride=stride, pad=pad,
                   kernel=kernel, dtype=rng.choice([torch.float32, torch.float32, torch.float64]), binary=binary,
                   binary_input=binary and rng.random() < 0.7, feature_major=rng.random() < 0.3, scale=rng.choice([1.0, 3.0]),
                   seed=rng.randrange(1 << 30))
        count -= 1


def test_random_blocks_with_indices_against_the_oracle():
    # (a layer that returns its pooled positions takes the reference-shaped Function: probabilities in, generic kernels)
    for case in _block_cases(seed=11, count=160):
        torch.manual_seed(case["seed"])
        n, cin, cout, dtype, geo = case["n"], case["cin"], case["cout"], case["dtype"], (case["stride"], case["pad"], case["kernel"])
        layer = C.ConvLogicLayer(cin, cout, stride=geo[0], padding=geo[1], kernel=geo[2], complete=True, implementation="cuda",
                                 return_indices=True).to(DEV).to(dtype)
        with torch.no_grad():
            layer.weights.mul_(case["scale"])
        shape = (n, cin, case["h"], case["w"])
        x = torch.randint(0, 2, shape, device=DEV).to(dtype) if case["binary"] else torch.randn(shape, device=DEV, dtype=dtype)
        x.requires_grad_(True)
        y, idx = layer(x)
        gy = torch.randn_like(y)
        y.backward(gy)
        pairs = tuple((v, v) for v in geo)
        routed, y_ref, idx_ref, _, _, ll, xl, x4 = block_oracle(x, layer.weights, layer.selection, *pairs, idx)
        tol, rel = _tolerances(dtype)
        size = max(1.0, x4.detach().abs().max().item())
        assert y.shape == y_ref.shape and idx.shape == idx_ref.shape, case
        check_pool_route(idx, idx_ref, x4, tol=tol * size)
        assert (y.detach().cpu() - routed.detach()).abs().max().item() <= tol * size, case
        routed.backward(gy.cpu())
        _grad_close(x.grad, xl.grad, rel, ("grad_x", case))
        _grad_close(layer.weights.grad, ll.grad, rel, ("grad_logits", case))
        # eval mode: arg-max gates; exact on 0/1 inputs
        layer.eval()
        with torch.no_grad():
            ye, idxe = layer(x.detach())
        _, ye_ref, idxe_ref, _, _, _, _, x4e = block_oracle(x, layer.weights, layer.selection, *pairs, idxe, training=False)
        check_pool_route(idxe, idxe_ref, x4e, tol=tol * max(1.0, x4e.detach().abs().max().item()))
        routed_e = x4e.flatten(2).gather(2, idxe.cpu().long()).view_as(ye_ref)
        assert (ye.cpu() - routed_e).abs().max().item() <= tol * max(1.0, routed_e.abs().max().item()), case
        if case["binary"]:
            assert torch.equal(ye.cpu(), ye_ref) and torch.equal(idxe.cpu(), idxe_ref), case


def test_random_blocks_on_the_training_path_of_the_module():
    # logits in, planned backward, the binary-input kernels where the layer promises 0/1 inputs, feature-major output, with and
    # without an input gradient: the forward is bit for bit the reference-shaped Function's on the probabilities this
    # library's softmax gives, whose pooled positions then route the oracle for the gradients.  (Strides that do not divide
    # the padded image are among the cases: the planned backward once rebuilt its geometry from the output size there.)
    from convlogic_amd.hip import difflogic_hip
    for case in _block_cases(seed=16, count=200):
        torch.manual_seed(case["seed"])
        n, cin, cout, dtype, geo = case["n"], case["cin"], case["cout"], case["dtype"], (case["stride"], case["pad"], case["kernel"])
        layer = C.ConvLogicLayer(cin, cout, stride=geo[0], padding=geo[1], kernel=geo[2], complete=True, implementation="cuda").to(DEV).to(dtype)
        layer.binary_input, layer.feature_major_output = case["binary_input"], case["feature_major"]
        with torch.no_grad():
            layer.weights.mul_(case["scale"])
        shape = (n, cin, case["h"], case["w"])
        x = torch.randint(0, 2, shape, device=DEV).to(dtype) if case["binary"] else torch.randn(shape, device=DEV, dtype=dtype)
        need_gx = case["seed"] % 7 != 0
        x.requires_grad_(need_gx)
        y = layer(x)
        gy = torch.randn_like(y)
        y.backward(gy)
        probs = difflogic_hip.fold(layer.weights.detach().reshape(-1, 16), from_logits=True)[0].reshape(cout, 7, 16)
        with torch.no_grad():
            y_fn, idx = C.FullConvLogicFunction.apply(x.detach(), probs, layer.selection, geo[0], geo[0], geo[1], geo[1], geo[2], geo[2], False, True)
        assert torch.equal(y, y_fn), case
        pairs = tuple((v, v) for v in geo)
        routed, _, idx_ref, _, _, ll, xl, x4 = block_oracle(x, layer.weights, layer.selection, *pairs, idx)
        tol, rel = _tolerances(dtype)
        size = max(1.0, x4.detach().abs().max().item())
        check_pool_route(idx, idx_ref, x4, tol=tol * size)
        assert (y.detach().cpu() - routed.detach()).abs().max().item() <= tol * size, case
        routed.backward(gy.cpu())
        if need_gx:
            _grad_close(x.grad, xl.grad, rel, ("grad_x", case))

        def in_float64():
            r64, _, _, _, _, l64, _, _ = block_oracle(x.detach().double(), layer.weights.detach().double(), layer.selection, *pairs, idx)
            r64.backward(gy.cpu().double())
            return l64.grad

        _grad_close_or_as_good_as_float32(layer.weights.grad, ll.grad, in_float64, rel, ("grad_logits", case))
        layer.check_binary_input()


def _fc_cases(seed, count):
    rng = random.Random(seed)
    for _ in range(count):
        batch = rng.choice([1, 2, 3, 4, 7, 16, 31, 32, 33, 37, 64, 100, 127, 128, 129, 200, 255, 256, 257, 300, 513])
        kind = rng.choice(["fan", "halving", "halving", "any"])
        if kind == "halving":
            out_dim = rng.choice([1, 2, 3, 5, 10, 30, 63, 64, 100, 250, 640, 1000, 4096])
            in_dim = 2 * out_dim
        elif kind == "fan":
            in_dim = rng.choice([1, 2, 5, 6, 10, 33, 64, 100, 512])
            out_dim = in_dim * rng.choice([1, 2, 5, 10, 20, 43])
        else:
            in_dim = rng.choice([1, 3, 8, 50, 99, 128, 1000])
            out_dim = max((in_dim + 1) // 2, rng.choice([1, 4, 17, 64, 300, 999]))
        while in_dim * batch > 600000 or out_dim * batch > 1500000:
            batch = max(1, batch // 2)
        yield dict(in_dim=in_dim, out_dim=out_dim, batch=batch, dtype=rng.choice([torch.float32, torch.float32, torch.float64]),
                   connections=rng.choice(["random", "random", "unique"]), grad_factor=rng.choice([1.0, 1.0, 1.0, 2.5]),
                   k=rng.choice([d for d in (1, 2, 3, 5, 7, 10, out_dim) if out_dim % d == 0]), tau=rng.choice([1.0, 6.5, 20.0]),
                   feature_major_view=rng.random() < 0.5, tail=rng.choice(["none", "group_sum", "one_node"]), scale=rng.choice([1.0, 4.0]),
                   seed=rng.randrange(1 << 30))


def test_random_logic_layers_and_group_sums_against_the_oracle():
    for case in _fc_cases(seed=12, count=400):
        torch.manual_seed(case["seed"])
        in_dim, out_dim, batch, dtype, gf = case["in_dim"], case["out_dim"], case["batch"], case["dtype"], case["grad_factor"]
        try:
            layer = C.LogicLayer(in_dim, out_dim, grad_factor=gf, connections=case["connections"], implementation="cuda")
        except AssertionError:                                       # "unique" wiring has no solution for this pair of widths
            assert case["connections"] == "unique", case
            continue
        layer = layer.to(DEV).to(dtype)
        with torch.no_grad():
            layer.weights.mul_(case["scale"])
        if case["feature_major_view"]:                               # what a LogicLayer hands to the next one
            x = torch.rand(in_dim, batch, device=DEV, dtype=dtype).requires_grad_(True)
            xin = x.transpose(0, 1)
        else:
            x = torch.rand(batch, in_dim, device=DEV, dtype=dtype).requires_grad_(True)
            xin = x
        gs = C.GroupSum(case["k"], tau=case["tau"])
        y = {"none": lambda: layer(xin), "group_sum": lambda: gs(layer(xin)), "one_node": lambda: logic_layer_group_sum(layer, gs, xin)}[case["tail"]]()
        gy = torch.randn_like(y)
        y.backward(gy)
        xl = x.detach().cpu().clone().requires_grad_(True)
        ll = layer.weights.detach().cpu().clone().requires_grad_(True)
        xr = xl.transpose(0, 1) if case["feature_major_view"] else xl
        idx0, idx1 = layer.indices_0.cpu(), layer.indices_1.cpu()
        y_ref = O.logic_fc_forward(xr, idx0, idx1, torch.softmax(ll, -1))
        if case["tail"] != "none":
            y_ref = O.group_sum(y_ref, case["k"], case["tau"])
        y_ref.backward(gy.cpu())
        tol, rel = _tolerances(dtype)
        assert (y.detach().cpu() - y_ref.detach()).abs().max().item() <= tol * max(1.0, y_ref.detach().abs().max().item()), case
        _grad_close(x.grad, xl.grad * gf, rel, ("grad_x", case))

        def in_float64():
            x64, l64 = x.detach().cpu().double(), layer.weights.detach().cpu().double().requires_grad_(True)
            y64 = O.logic_fc_forward(x64.transpose(0, 1) if case["feature_major_view"] else x64, idx0, idx1, torch.softmax(l64, -1))
            if case["tail"] != "none":
                y64 = O.group_sum(y64, case["k"], case["tau"])
            y64.backward(gy.cpu().double())
            return l64.grad

        _grad_close_or_as_good_as_float32(layer.weights.grad, ll.grad, in_float64, rel, ("grad_logits", case))
        layer.eval()
        with torch.no_grad():
            ye = layer(xin.detach())
        one_hot = torch.nn.functional.one_hot(layer.weights.detach().cpu().argmax(-1), 16).to(dtype)
        assert (ye.cpu() - O.logic_fc_forward(xr.detach(), idx0, idx1, one_hot)).abs().max().item() <= tol, case


def test_random_packed_stacks_against_the_oracle_and_the_float_eval_path():
    rng = random.Random(13)
    for _ in range(250):
        bits = rng.choice([8, 16, 32, 64, 64, 64])
        batch = rng.choice([1, 5, 8, 31, 63, 64, 65, 100, 128, 200, 255, 256, 257, 511, 512, 1000, 1030, 2049, 4096, 4133, 8192])
        dims = [rng.choice([1, 2, 6, 10, 33, 48, 64, 100, 160, 528, 1000, 2000])]
        for _ in range(rng.choice([1, 2, 3])):
            dims.append(max((dims[-1] + 1) // 2, rng.choice([1, 3, 10, 16, 40, 64, 120, 500, 1024, 3000])))
        while max(dims) * batch > 8_000_000:
            batch = max(1, batch // 2)
        k = rng.choice([d for d in (1, 2, 3, 4, 5, 8, 10, dims[-1]) if dims[-1] % d == 0])
        case = (bits, batch, dims, k)
        torch.manual_seed(rng.randrange(1 << 30))
        layers = [C.LogicLayer(a, b, implementation="cuda") for a, b in zip(dims[:-1], dims[1:])]
        model = torch.nn.Sequential(*layers, C.GroupSum(k, tau=6.5)).to(DEV).eval()
        x = torch.randint(0, 2, (batch, dims[0]), device=DEV).bool()
        with torch.no_grad():
            y_bits = model(C.PackBitsTensor(x, bits))
            y_float = model(x.float())
        assert y_bits.dtype == torch.int32 and y_bits.shape == (batch, k), case
        assert torch.equal(y_bits.float() / 6.5, y_float), case
        words, pad = O.pack_bits(x.cpu().numpy().T, bits)
        for layer in layers:
            words = O.eval_packed(words, layer.indices_0.cpu().numpy(), layer.indices_1.cpu().numpy(),
                                  layer.weights.argmax(-1).cpu().numpy().astype(np.uint8))
        assert np.array_equal(O.group_bit_sum(words, pad, k), y_bits.cpu().numpy()), case


def test_random_networks_keep_their_promises():
    # a training step is reproducible bit for bit; the last LogicLayer and GroupSum as one autograd node change nothing
    # (bit for bit; a batch of one hands the GroupSum module a contiguous [1, F] tensor, which torch sums in another order);
    # the network-wide fold changes values by rounding only; packed inference equals the float eval path exactly
    rng = random.Random(14)
    for _ in range(40):
        topology = rng.choice(["cifar", "cifar", "mnist"])
        k, n, tau = rng.choice([1, 2, 3, 4, 6, 8]), rng.choice([1, 2, 5, 31, 64, 65, 100, 128, 200]), rng.choice([1.0, 6.5, 20.0])
        cin = rng.choice([1, 3, 6, 9]) if topology == "cifar" else 1
        case = (topology, k, n, cin, tau)
        torch.manual_seed(rng.randrange(1 << 30))
        if topology == "cifar":
            model, size = C.ConvLogicCifarModel(k_param=k, input_channels=cin, input_size=32, tau=tau).to(DEV), 32
        else:
            model, size = C.ConvLogicMnistModel(k_param=k, tau=tau).to(DEV), 28
        x = torch.randint(0, 2, (n, cin, size, size), device=DEV)
        labels = torch.randint(0, 10, (n,), device=DEV)
        xf = x.float()

        def step(prefold, fused_tail):
            model.train()
            model.prefold, model.fused_tail = prefold, fused_tail
            for p in model.parameters():
                p.grad = None
            out = model(xf)
            torch.nn.functional.cross_entropy(out, labels).backward()
            return out.detach().clone(), [p.grad.clone() for p in model.parameters()]

        out_a, grads_a = step(False, False)
        out_b, grads_b = step(False, False)
        assert torch.equal(out_a, out_b) and all(torch.equal(u, v) for u, v in zip(grads_a, grads_b)), case
        out_c, grads_c = step(False, True)
        if n > 1:
            assert torch.equal(out_a, out_c) and all(torch.equal(u, v) for u, v in zip(grads_a, grads_c)), case
        out_d, grads_d = step("always", True)
        for out, grads in ((out_c, grads_c), (out_d, grads_d)):
            assert (out_a - out).abs().max().item() <= 1e-5 * max(1.0, out_a.abs().max().item()), case
            for u, v in zip(grads_a, grads):
                assert (u - v).norm().item() <= 1e-4 * (u.norm().item() + 1e-30), case
        model.eval()
        with torch.no_grad():
            y_float = model(xf)
            y_bits = model(C.PackBitsTensor(x.bool(), 64))
        assert y_bits.dtype == torch.int32 and torch.equal(y_bits.float() / tau, y_float), case


def _window(rng):
    """A random (stride, padding, kernel, h, w) with non-square members; windows of one element are left out (the
    constructor refuses them)."""
    while True:
        st = (rng.choice([1, 1, 2, 3]), rng.choice([1, 1, 2]))
        kn = (rng.choice([1, 2, 3, 3, 4, 5]), rng.choice([2, 3, 3, 5]))
        pd = (min(rng.choice([0, 1, 2]), kn[0] - 1), min(rng.choice([0, 1, 2]), kn[1] - 1))
        h, w = rng.choice([1, 2, 3, 5, 8, 9, 12, 17, 28, 33]), rng.choice([1, 2, 4, 7, 10, 16, 31, 40])
        if h + 2 * pd[0] >= kn[0] and w + 2 * pd[1] >= kn[1]:
            return st, pd, kn, h, w


def test_random_split_layers_tree_levels_packed_blocks_thresholds_and_the_reference_shaped_function():
    rng = random.Random(15)
    for _ in range(400):
        what = rng.choice(["conv4", "tree", "packed", "thresholds", "function"])
        torch.manual_seed(rng.randrange(1 << 30))
        dtype = rng.choice([torch.float32, torch.float32, torch.float64])
        tol, rel = _tolerances(dtype)
        if what == "conv4":                                          # split layer, any stride / padding / window
            st, pd, kn, h, w = _window(rng)
            n, cin, cout = rng.choice([1, 2, 4, 17, 64]), rng.choice([1, 2, 3, 8, 20]), rng.choice([1, 2, 5, 16, 40])
            case = (what, n, cin, cout, h, w, st, pd, kn, dtype)
            layer = C.ConvLogicLayer(cin, cout, stride=st, padding=pd, kernel=kn, implementation="cuda").to(DEV).to(dtype)
            x = torch.randn(n, cin, h, w, device=DEV, dtype=dtype, requires_grad=True)
            y = layer(x)
            gy = torch.randn_like(y)
            y.backward(gy)
            xl, ll = x.detach().cpu().requires_grad_(True), layer.weights.detach().cpu().requires_grad_(True)
            want = O.conv4_forward(xl, torch.softmax(ll, -1), layer.selection.cpu(), st, pd, kn)
            want.backward(gy.cpu())
            assert y.shape == want.shape, case
            assert (y.detach().cpu() - want.detach()).abs().max().item() <= tol * max(1.0, want.detach().abs().max().item()), case
            _grad_close(x.grad, xl.grad, rel, ("grad_x", case))
            _grad_close(layer.weights.grad, ll.grad, rel, ("grad_logits", case))
        elif what == "tree":
            bits = rng.choice([2, 4, 6, 8])
            n, c, h, w = rng.choice([1, 3, 16, 70]), rng.choice([1, 2, 5, 33]), rng.choice([1, 2, 4, 9, 16]), rng.choice([1, 3, 6, 16])
            case = (what, n, c, h, w, bits, dtype)
            layer = C.TreeLogicLayer(c, bits, implementation="cuda").to(DEV).to(dtype)
            x = torch.rand(n, c, h, w, bits, device=DEV, dtype=dtype, requires_grad=True)
            y = layer(x)
            gy = torch.randn_like(y)
            y.backward(gy)
            xl, ll = x.detach().cpu().requires_grad_(True), layer.weights.detach().cpu().requires_grad_(True)
            want = O.tree_forward(xl, torch.softmax(ll, -1))
            want.backward(gy.cpu())
            assert (y.detach().cpu() - want.detach()).abs().max().item() <= tol, case
            _grad_close(x.grad, xl.grad, rel, ("grad_x", case))
            _grad_close(layer.weights.grad, ll.grad, rel, ("grad_logits", case))
        elif what == "packed":                                       # packed block: numpy oracle and the float eval path
            while True:
                st, pd, kn, h, w = _window(rng)
                ho, wo = O.conv_out_size(h, w, st, pd, kn)
                if ho >= 2 and wo >= 2 and ho % 2 == 0 and wo % 2 == 0:
                    break
            n, cin, cout = rng.choice([1, 5, 64, 65, 130, 300]), rng.choice([1, 2, 3, 9, 32, 100]), rng.choice([1, 2, 6, 32, 96, 200])
            case = (what, n, cin, cout, h, w, st, pd, kn)
            layer = C.ConvLogicLayer(cin, cout, stride=st, padding=pd, kernel=kn, complete=True, implementation="cuda").to(DEV)
            with torch.no_grad():
                layer.weights.copy_(torch.randn_like(layer.weights))
            layer.eval()
            bits = torch.randint(0, 2, (n, cin, h, w), device=DEV).bool()
            with torch.no_grad():
                y_float = layer(bits.float())
            p = C.PackBitsTensor(bits, 64)
            words, pad = O.pack_image(bits.cpu().numpy())
            assert p.pad_len == pad and np.array_equal(p.t.cpu().numpy(), words), case
            out = layer(p)
            gates = layer.weights.argmax(-1).to(torch.uint8).cpu().numpy()
            want = O.conv_block_eval_packed(words, gates, layer.selection.cpu().numpy(), st, pd, kn)
            assert np.array_equal(out.t.cpu().numpy(), want), case
            assert np.array_equal(O.unpack_image(out.t.cpu().numpy(), pad), y_float.cpu().numpy() > 0.5), case
        elif what == "thresholds":
            n, c0, levels = rng.choice([1, 33, 64, 70, 200]), rng.choice([1, 2, 3]), rng.choice([1, 2, 3, 9])
            h, w = rng.choice([1, 4, 5, 28, 32]), rng.choice([1, 4, 7, 28, 32])
            case = (what, n, c0, h, w, levels)
            x = torch.rand(n, c0, h, w)
            thr = O.thresholds_uniform(levels)
            want = O.apply_thresholds(x, thr)
            assert torch.equal(binarize.apply_thresholds(x.to(DEV), thr).cpu(), want), case
            p = binarize.pack_thresholds(x.to(DEV), thr)
            words, pad = O.pack_image(want.numpy() > 0.5)
            assert p.pad_len == pad and np.array_equal(p.t.cpu().numpy(), words), case
        else:                                                        # probabilities in, their gradient out (the reference's Function)
            in_dim = rng.choice([1, 2, 7, 64, 100, 999])
            out_dim, batch = max((in_dim + 1) // 2, rng.choice([1, 5, 64, 300, 2000])), rng.choice([1, 3, 32, 100, 256, 300])
            case = (what, in_dim, out_dim, batch, dtype)
            layer = C.LogicLayer(in_dim, out_dim, implementation="cuda").to(DEV).to(dtype)
            x = torch.rand(in_dim, batch, device=DEV, dtype=dtype, requires_grad=True)
            w = torch.softmax(layer.weights.detach(), -1).requires_grad_(True)
            y = LogicLayerCudaFunction.apply(x, layer.indices_0, layer.indices_1, w, layer.given_x_indices_of_y_start,
                                             layer.given_x_indices_of_y)
            gy = torch.randn_like(y)
            y.backward(gy)
            xl, wl = x.detach().cpu().requires_grad_(True), w.detach().cpu().requires_grad_(True)
            want = O.logic_fc_forward(xl.transpose(0, 1), layer.indices_0.cpu(), layer.indices_1.cpu(), wl).transpose(0, 1)
            want.backward(gy.cpu())
            assert (y.detach().cpu() - want.detach()).abs().max().item() <= tol, case
            _grad_close(x.grad, xl.grad, rel, ("grad_x", case))
            _grad_close(w.grad, wl.grad, rel, ("grad_w", case))
