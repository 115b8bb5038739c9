"""BASELINE config 5 as a parity case: the conv-logic network topology (4 fused blocks, flatten, 3
LogicLayers, GroupSum; src/convlogic/model.py:16-58 with k=32, 9 input channels) built from this
package's layers, one training step and the packed-bit evaluation of the fully connected tail against
the CPU oracle at a reduced batch."""
import copy

import numpy as np
import pytest
import torch

import convlogic_amd as C
from oracle import convlogic_oracle as O
from tests.gpu_util import DEV, assert_grad_close

pytestmark = pytest.mark.gpu


def build(k=32, cin=9, size=32, tau=6.5, residual_init=False):
    chans = [cin, k, 4 * k, 16 * k, 32 * k]
    layers = [C.ConvLogicLayer(a, b, padding=1, complete=True, implementation="cuda", residual_init=residual_init)
              for a, b in zip(chans[:-1], chans[1:])]
    flat = chans[-1] * (size // 16) ** 2
    dims = [flat, flat * 10, flat * 5, (flat * 10) // 4]
    layers.append(torch.nn.Flatten())
    layers += [C.LogicLayer(a, b, implementation="cuda", residual_init=residual_init) for a, b in zip(dims[:-1], dims[1:])]
    layers.append(C.GroupSum(10, tau))
    return torch.nn.Sequential(*layers)


def oracle_forward(model, x, training=True):
    h = x
    for m in model:
        if isinstance(m, C.ConvLogicLayer):
            h = O.conv_block_forward(h, O.gate_weights(m.weights.detach().cpu() if not training else m._w, training, h.dtype),
                                     m.selection.cpu(), tuple(m.stride), tuple(m.padding), tuple(m.kernel))
        elif isinstance(m, torch.nn.Flatten):
            h = h.flatten(1)
        elif isinstance(m, C.LogicLayer):
            h = O.logic_fc_forward(h, m.indices_0.cpu(), m.indices_1.cpu(),
                                   O.gate_weights(m.weights.detach().cpu() if not training else m._w, training, h.dtype))
        else:
            h = O.group_sum(h, m.k, m.tau)
    return h


def test_config5_training_step_matches_oracle():
    # float64 on both sides: through 7 layers of random-init gates the first-layer gradient is ~1e-10 of
    # the last one, and in float32 a single near-tie in a pooling window decides its leading digits
    torch.manual_seed(0)
    model = build().double().to(DEV)
    n = 4
    v = (torch.randn(n, 3, 32, 32, dtype=torch.float64) * 0.25 + 0.5).clamp(0, 1)
    x = torch.cat([(v > t).double() for t in (0.25, 0.5, 0.75)], dim=1)
    labels = torch.randint(0, 10, (n,))
    xg = x.to(DEV).requires_grad_(True)
    logits = model(xg)
    assert logits.shape == (n, 10)
    loss = torch.nn.functional.cross_entropy(logits, labels.to(DEV))
    loss.backward()

    params = [m for m in model if hasattr(m, "weights")]
    for m in params:
        m._w = m.weights.detach().cpu().clone().requires_grad_(True)
    xc = x.clone().requires_grad_(True)
    ref = oracle_forward(model, xc)
    ref_loss = torch.nn.functional.cross_entropy(ref, labels)
    ref_loss.backward()
    assert (logits.detach().cpu() - ref.detach()).abs().max().item() <= 1e-9
    assert abs(loss.item() - ref_loss.item()) <= 1e-10
    for i, m in enumerate(params):
        assert_grad_close(m.weights.grad, m._w.grad, rel=1e-6, name=f"layer {i} grad_logits")
    assert_grad_close(xg.grad, xc.grad, rel=1e-6, name="grad_x")


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_fold_many_equals_the_folds_of_the_layers(dtype):
    # one launch for the logits of several layers: row by row what the LogicLayer's fold and the set-up launch of the
    # fused block give, the pair of a tensor in one buffer (probabilities first)
    from convlogic_amd.hip import convlogic_hip, difflogic_hip
    torch.manual_seed(3)
    tensors = [torch.randn(300, 16, device=DEV, dtype=dtype) * 3, torch.randn(24, 7, 16, device=DEV, dtype=dtype) * 3,
               torch.randn(1, 16, device=DEV, dtype=dtype), torch.randn(513, 7, 16, device=DEV, dtype=dtype) * 5]
    pairs = difflogic_hip.fold_many(tensors)
    for t, (probs, folded) in zip(tensors, pairs):
        want_p, want_f = difflogic_hip.fold(t.reshape(-1, 16), from_logits=True)
        assert probs.shape == t.shape and folded.shape == (*t.shape[:-1], 4)
        assert torch.equal(probs.reshape(-1, 16), want_p) and torch.equal(folded.reshape(-1, 4), want_f)
        assert torch.equal(folded.reshape(-1, 4), difflogic_hip.fold(probs.reshape(-1, 16), from_logits=False)[1])   # = the fold of the stored values
        assert folded.data_ptr() == probs.data_ptr() + probs.numel() * probs.element_size()
    # the block's forward takes such a pair instead of folding itself: same outputs, bit for bit, on every forward path
    for (n, cin, h, c) in ((40, 16, 4, 24), (6, 8, 8, 24), (3, 4, 16, 24)):
        layer = C.ConvLogicLayer(cin, c, padding=1, complete=True, implementation="cuda").to(DEV).to(dtype)
        x = torch.rand(n, cin, h, h, device=DEV, dtype=dtype)
        lg = layer.weights.detach()
        pair = difflogic_hip.fold_many([lg, tensors[0]])[0]
        geo = (*layer.stride, *layer.padding, *layer.kernel)
        a = convlogic_hip.full_convlogic_forward_logits(x, lg, layer.selection, *geo, want_folded=True)
        b = convlogic_hip.full_convlogic_forward_logits(x, lg, layer.selection, *geo, want_folded=True, prefolded=pair)
        for u, v, name in zip(a, b, ("y", "argmax", "probs", "folded")):
            assert torch.equal(u, v), (name, n, cin, h)
    with pytest.raises(RuntimeError):
        difflogic_hip.fold_many([])


def test_network_folds_all_layers_in_one_launch():
    # the CIFAR topology folds its layers' logits once per training step (model.prefold): logits, loss and
    # every gradient against the same network with the per-layer folds (the blocks bit for bit up to the first
    # LogicLayer, whose in-kernel softmax sums in another order: 1e-6).  (Against the oracle: the C5 case of
    # test_gpu_baseline_shapes.py, which runs this model as it is.)
    torch.manual_seed(5)
    model = C.ConvLogicCifarModel(k_param=4, input_channels=9, input_size=32, tau=6.5).to(DEV)
    x = torch.randint(0, 2, (40, 9, 32, 32), device=DEV).float()
    labels = torch.randint(0, 10, (40,), device=DEV)

    def step(prefold):
        model.prefold = prefold
        for p in model.parameters():
            p.grad = None
        out = model(x)
        torch.nn.functional.cross_entropy(out, labels).backward()
        return out.detach().clone(), [p.grad.clone() for p in model.parameters()]

    out_a, grads_a = step("always")                                      # (True: only where it pays -- big networks, graph capture)
    assert all("_prefold" not in m.__dict__ for m in model.network)        # every pair was taken by its layer
    out_b, grads_b = step(False)
    assert (out_a - out_b).abs().max().item() <= 1e-5
    for i, (ga, gb) in enumerate(zip(grads_a, grads_b)):
        assert_grad_close(ga, gb, rel=1e-4, name=f"parameter {i}")
    out_c, grads_c = step("always")
    assert torch.equal(out_a, out_c) and all(torch.equal(u, v) for u, v in zip(grads_a, grads_c))   # reproducible
    # a stale pair (weights changed in place after it was made) is not used
    first_fc = next(m for m in model.network if isinstance(m, C.LogicLayer))
    from convlogic_amd.hip import difflogic_hip
    first_fc.set_prefold(*difflogic_hip.fold_many([first_fc.weights.detach(), first_fc.weights.detach()])[0])
    with torch.no_grad():
        first_fc.weights.add_(1.0)
    assert first_fc._take_prefold(first_fc.weights) is None
    with torch.no_grad():
        first_fc.weights.sub_(1.0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_last_layer_and_group_sum_as_one_autograd_node(dtype):
    # the networks run their last LogicLayer and the GroupSum behind it as one node whose backward hands the gradient of
    # the class sums straight to the layer's kernel: outputs and every gradient bit for bit those of the two modules, for
    # both topologies, ragged batches and a class count that the kernel's lanes do not divide
    from convlogic_amd.hip import difflogic_hip
    torch.manual_seed(11)
    # (batch 200 at 4 samples per lane: the shape on which the compiler once fused the division by tau into the sums)
    for model, shape in ((C.ConvLogicCifarModel(k_param=2, input_channels=3, input_size=32, tau=6.5), (37, 3, 32, 32)),
                         (C.ConvLogicCifarModel(k_param=1, input_channels=1, input_size=32, tau=6.5), (200, 1, 32, 32)),
                         (C.ConvLogicMnistModel(k_param=2, tau=3.0), (64, 1, 28, 28))):
        model = model.to(DEV).to(dtype)
        x = torch.randint(0, 2, shape, device=DEV).to(dtype)
        labels = torch.randint(0, 10, (shape[0],), device=DEV)

        def step(fused):
            model.fused_tail = fused
            for p in model.parameters():
                p.grad = None
            xin = x.clone().requires_grad_(True)
            out = model(xin)
            torch.nn.functional.cross_entropy(out, labels).backward()
            return out.detach().clone(), [xin.grad.clone()] + [p.grad.clone() for p in model.parameters()]

        out_a, grads_a = step(True)
        out_b, grads_b = step(False)
        assert torch.equal(out_a, out_b)
        for i, (u, v) in enumerate(zip(grads_a, grads_b)):
            assert torch.equal(u, v), (type(model).__name__, i, (u - v).abs().max().item())
    # a forward hook on the last layer is a reason to call the module itself: the hook still fires
    seen = []
    handle = model.network[-2].register_forward_hook(lambda m, i, o: seen.append(tuple(o.shape)))
    model.fused_tail = True
    model(x)
    handle.remove()
    assert seen == [(shape[0], model.network[-2].out_dim)]
    # the entry point against its two-launch equivalent, k = 7 classes of 9 rows
    layer = C.LogicLayer(126, 63, implementation="cuda").to(DEV).to(dtype)
    xf = torch.rand(126, 52, device=DEV, dtype=dtype)
    go = torch.randn(52, 7, device=DEV, dtype=dtype)
    probs, folded = difflogic_hip.fold(layer.weights.detach(), from_logits=True)
    gy = difflogic_hip.group_sum_backward(go, 63, 2.5)
    want = difflogic_hip.backward_sole(xf, layer.indices_0, layer.indices_1, folded, probs, gy)
    got = difflogic_hip.backward_sole_classes(xf, layer.indices_0, layer.indices_1, folded, probs, go, 7, 2.5)
    assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])
    with pytest.raises(RuntimeError):
        difflogic_hip.backward_sole_classes(xf, layer.indices_0, layer.indices_1, folded, probs, go[:, :5].contiguous(), 5, 2.5)


def test_config5_training_step_float32_runs_and_is_deterministic():
    torch.manual_seed(2)
    model = build().to(DEV)
    x = torch.randint(0, 2, (8, 9, 32, 32), device=DEV).float()
    labels = torch.randint(0, 10, (8,), device=DEV)

    def step():
        for m in model:
            if hasattr(m, "weights"):
                m.weights.grad = None
        loss = torch.nn.functional.cross_entropy(model(x), labels)
        loss.backward()
        return loss.detach().clone(), [m.weights.grad.clone() for m in model if hasattr(m, "weights")]

    l1, g1 = step()
    l2, g2 = step()
    assert torch.equal(l1, l2) and all(torch.equal(a, b) for a, b in zip(g1, g2))
    assert all(torch.isfinite(g).all() for g in g1)


def test_config5_eval_float_and_packed_tail():
    torch.manual_seed(1)
    model = build().to(DEV).eval()
    n = 96
    x = torch.randint(0, 2, (n, 9, 32, 32), device=DEV).float()
    with torch.no_grad():
        feats = x
        for m in list(model)[:5]:
            feats = m(feats)                       # 4 blocks + flatten, float eval path: exactly binary
        assert torch.all((feats == 0) | (feats == 1))
        y_float = feats
        for m in list(model)[5:]:
            y_float = m(y_float)
        p = C.PackBitsTensor(feats.bool(), 64)
        for m in list(model)[5:]:
            p = m(p)
    assert p.dtype == torch.int32 and p.shape == (n, 10)
    assert torch.equal(p.float() / 6.5, y_float)
    assert torch.equal(p.float(), torch.round(y_float * 6.5))
    # against the oracle: float eval of the whole network on the CPU
    ref = oracle_forward(model, x.cpu(), training=False)
    # identical counts; torch divides by tau with a reciprocal on the GPU (1 ulp from the CPU division)
    assert torch.equal(torch.round(y_float.cpu() * 6.5), torch.round(ref * 6.5))
    assert torch.allclose(y_float.cpu(), ref, rtol=3e-7, atol=0)
    words, pad = O.pack_bits(feats.cpu().numpy().T.astype(bool), 64)
    for m in list(model)[5:8]:
        words = O.eval_packed(words, m.indices_0.cpu().numpy(), m.indices_1.cpu().numpy(),
                              m.weights.argmax(-1).cpu().numpy().astype(np.uint8))
    assert np.array_equal(O.group_bit_sum(words, pad, 10), p.cpu().numpy())


def test_config5_eval_fully_packed_from_the_input():
    # the whole network on packed bits: group-major image words through the four blocks, nn.Flatten turns
    # them feature-major, three packed LogicLayers, per-class bit counts == the float eval path's scores
    torch.manual_seed(4)
    model = build().to(DEV).eval()
    n = 200
    bits = torch.randint(0, 2, (n, 9, 32, 32), device=DEV).bool()
    with torch.no_grad():
        y_float = model(bits.float())
        p = model(C.PackBitsTensor(bits, 64))
    assert p.dtype == torch.int32 and p.shape == (n, 10)
    assert torch.equal(p.float(), torch.round(y_float * 6.5))
    ref = oracle_forward(model, bits[:48].float().cpu(), training=False)
    assert torch.equal(p[:48].cpu().float(), torch.round(ref * 6.5))


def test_mnist_topology_training_step_and_packed_eval():
    # ConvLogicMnistModel (5x5 / padding 0 first block; src/convlogic/model.py:63-108) at k = 4: one float64
    # training step against the oracle, an optimizer step, then eval: float path == packed path == oracle
    torch.manual_seed(6)
    model = C.ConvLogicMnistModel(k_param=4).double().to(DEV)
    net = model.network
    with torch.no_grad():
        for m in net:
            if hasattr(m, "weights"):
                m.weights.copy_(torch.randn_like(m.weights))      # off the residual init, so every gate matters
    n = 6
    x = torch.randint(0, 2, (n, 1, 28, 28)).double()
    labels = torch.randint(0, 10, (n,))
    opt = torch.optim.AdamW(model.parameters(), lr=0.01)
    logits = model(x.to(DEV))
    loss = torch.nn.functional.cross_entropy(logits, labels.to(DEV))
    loss.backward()
    params = [m for m in net if hasattr(m, "weights")]
    for m in params:
        m._w = m.weights.detach().cpu().clone().requires_grad_(True)
    ref = oracle_forward(net, x.clone())
    torch.nn.functional.cross_entropy(ref, labels).backward()
    assert (logits.detach().cpu() - ref.detach()).abs().max().item() <= 1e-9
    for i, m in enumerate(params):
        assert_grad_close(m.weights.grad, m._w.grad, rel=1e-6, name=f"layer {i} grad_logits")
    before = [m.weights.detach().clone() for m in params]
    opt.step()
    assert all(not torch.equal(b, m.weights) for b, m in zip(before, params))

    model = model.float().eval()
    bits = torch.randint(0, 2, (150, 1, 28, 28), device=DEV).bool()
    with torch.no_grad():
        y_float = model(bits.float())
        counts = model(C.PackBitsTensor(bits, 64))
    assert counts.dtype == torch.int32 and torch.equal(counts.float(), torch.round(y_float * 6.5))
    ref = oracle_forward(net, bits[:40].float().cpu(), training=False)
    assert torch.equal(counts[:40].cpu().float(), torch.round(ref * 6.5))


def test_cifar_topology_state_dict_round_trip():
    torch.manual_seed(8)
    a = C.ConvLogicCifarModel(k_param=4, input_channels=9, tau=6.5).to(DEV).eval()
    b = C.ConvLogicCifarModel(k_param=4, input_channels=9, tau=6.5).to(DEV).eval()
    x = torch.randint(0, 2, (70, 9, 32, 32), device=DEV).bool()
    with torch.no_grad():
        ya = a(x.float())
        assert not torch.equal(ya, b(x.float()))                  # different wiring and taps
        b.load_state_dict(a.state_dict())
        assert torch.equal(ya, b(x.float()))
        assert torch.equal(b(C.PackBitsTensor(x, 64)).float(), torch.round(ya * 6.5))


def test_compiled_netlist_runs_the_packed_kernels(tmp_path):
    # CompiledLogicNet(device="cuda"): the frozen netlist (conv blocks + LogicLayers) evaluated by the packed
    # kernels equals the module path, before and after a trip through the .npz file
    from convlogic_amd.difflogic import CompiledLogicNet
    torch.manual_seed(10)
    model = C.ConvLogicMnistModel(k_param=4).to(DEV).eval()
    with torch.no_grad():
        for m in model.network:
            if hasattr(m, "weights"):
                m.weights.copy_(torch.randn_like(m.weights))
    bits = torch.randint(0, 2, (130, 1, 28, 28), device=DEV).bool()
    with torch.no_grad():
        want = model(C.PackBitsTensor(bits, 64))
    net = CompiledLogicNet(model, device="cuda")
    assert torch.equal(net(bits), want)
    net.save(str(tmp_path / "mnist.npz"))
    back = CompiledLogicNet.load_netlist(str(tmp_path / "mnist.npz"))
    assert torch.equal(back(bits.cpu()), want) and torch.equal(back(C.PackBitsTensor(bits, 64)), want)
    # fully connected only, flat input
    fc = torch.nn.Sequential(C.LogicLayer(64, 128), C.LogicLayer(128, 80), C.GroupSum(10)).to(DEV).eval()
    x = torch.randint(0, 2, (200, 64), device=DEV).bool()
    with torch.no_grad():
        assert torch.equal(CompiledLogicNet(fc)(x), fc(C.PackBitsTensor(x, 64)))


def test_small_network_learns_a_synthetic_task():
    # end to end: a small CIFAR-topology network trained with Adam on a task its first block can see (which image
    # half holds more ones) -- the loss has to fall, in eager steps and in HIP-graph replays alike
    torch.manual_seed(0)
    n = 256
    x = (torch.rand(n, 3, 32, 32, device=DEV) < 0.5).float()
    boost = torch.randint(0, 2, (n,), device=DEV)
    x[boost == 1, :, :16] = (torch.rand(int((boost == 1).sum()), 3, 16, 32, device=DEV) < 0.8).float()
    x[boost == 0, :, 16:] = (torch.rand(int((boost == 0).sum()), 3, 16, 32, device=DEV) < 0.8).float()
    labels = boost * 5                                               # classes 0 and 5 of 10
    ce = torch.nn.functional.cross_entropy
    for graphed in (False, True):
        torch.manual_seed(1)
        model = C.ConvLogicCifarModel(k_param=4, input_channels=3, input_size=32, tau=4).to(DEV)
        opt = torch.optim.Adam(model.parameters(), lr=0.05)
        step = C.GraphedStep(lambda a, b: ce(model(a), b), (x, labels), model.parameters()) if graphed else None
        losses = []
        for _ in range(40):
            if graphed:
                loss = step(x, labels)
            else:
                opt.zero_grad(set_to_none=True)
                loss = ce(model(x), labels)
                loss.backward()
            opt.step()
            losses.append(loss.item())
        assert all(torch.isfinite(torch.tensor(losses)))
        assert losses[-1] < 0.6 * losses[0], (graphed, losses[0], losses[-1])


def test_networks_stepping_on_four_host_threads_equal_their_serial_runs():
    # calls may come from any host thread and are ordered by the caller's stream only: four networks, each on its own
    # thread and stream at the same time, give bit for bit what each gives alone (no state shared between calls)
    import threading
    torch.manual_seed(0)
    specs = [("cifar", 2, 3, 40), ("mnist", 2, 1, 64), ("cifar", 4, 9, 17), ("cifar", 1, 1, 200)]
    nets, data = [], []
    for kind, k, cin, n in specs:
        model = (C.ConvLogicCifarModel(k_param=k, input_channels=cin, input_size=32, tau=6.5) if kind == "cifar"
                 else C.ConvLogicMnistModel(k_param=k, tau=6.5)).to(DEV)
        size = 32 if kind == "cifar" else 28
        nets.append(model)
        data.append([(torch.randint(0, 2, (n, cin, size, size), device=DEV).float(), torch.randint(0, 10, (n,), device=DEV)) for _ in range(5)])

    def run(model, batches, out):
        for _ in range(4):
            for x, labels in batches:
                for p in model.parameters():
                    p.grad = None
                logits = model(x)
                torch.nn.functional.cross_entropy(logits, labels).backward()
                out.append((logits.detach().clone(), [p.grad.clone() for p in model.parameters()]))

    serial = []
    for model, batches in zip(nets, data):
        serial.append([])
        run(copy.deepcopy(model), batches, serial[-1])
    torch.cuda.synchronize()
    results, errors = [[] for _ in nets], []
    multithreaded = torch.autograd.is_multithreading_enabled()
    torch.autograd.set_multithreading_enabled(False)              # backward on the thread that calls it

    def worker(i):
        try:
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                run(nets[i], data[i], results[i])
            stream.synchronize()
        except Exception as e:                                       # noqa: BLE001 - reported by the assert below
            errors.append((i, repr(e)))

    try:
        threads = [threading.Thread(target=worker, args=(i,)) for i in range(len(nets))]
        for t in threads:
            t.start()
        for t in threads:
            t.join()
        torch.cuda.synchronize()
    finally:
        torch.autograd.set_multithreading_enabled(multithreaded)
    assert not errors, errors
    for i, (alone, together) in enumerate(zip(serial, results)):
        assert len(alone) == len(together) == 20
        for step, ((oa, ga), (ob, gb)) in enumerate(zip(alone, together)):
            assert torch.equal(oa, ob), (i, step)
            assert all(torch.equal(u, v) for u, v in zip(ga, gb)), (i, step)


def test_python_implementation_of_a_network_trains_on_the_gpu_next_to_the_hip_one():
    # implementation="python" (torch ops) with device tensors: nothing of the network-level shortcuts applies, and a second
    # step must find that out as the first did (the fold cache of a network with nothing to fold once broke it);
    # the HIP network follows the same trajectory
    torch.manual_seed(6)
    a = C.ConvLogicMnistModel(k_param=2, tau=6.5, implementation="cuda").to(DEV)
    b = C.ConvLogicMnistModel(k_param=2, tau=6.5, implementation="python").to(DEV)
    b.load_state_dict(a.state_dict(), strict=False)
    opt_a, opt_b = torch.optim.SGD(a.parameters(), lr=0.5), torch.optim.SGD(b.parameters(), lr=0.5)
    for _ in range(3):
        x = torch.randint(0, 2, (32, 1, 28, 28), device=DEV).float()
        labels = torch.randint(0, 10, (32,), device=DEV)
        loss_a = torch.nn.functional.cross_entropy(a(x), labels)
        loss_b = torch.nn.functional.cross_entropy(b(x), labels)
        opt_a.zero_grad()
        opt_b.zero_grad()
        loss_a.backward()
        loss_b.backward()
        # (the losses, not the gradients: on 0/1 inputs the pooling windows are full of ties and near ties, which the two
        # implementations may route to different positions -- both valid, but not the same gradient element by element)
        assert abs(loss_a.item() - loss_b.item()) <= 1e-4 * max(1.0, abs(loss_b.item()))
        assert all(torch.isfinite(q.grad).all() for q in b.parameters())
        opt_a.step()
        opt_b.step()
