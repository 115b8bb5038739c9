"""HIP-graph capture of training steps (torch.cuda.CUDAGraph): the library launches on the current stream,
never synchronises and never allocates, so a forward+backward step can be captured once and replayed.
Every replay is checked against an eager step on copies of the same data, with eager work and
synchronisations between the replays."""
import copy

import pytest
import torch

import convlogic_amd as C
from tests.gpu_util import DEV

pytestmark = pytest.mark.gpu


def _capture(run):
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            run()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    return graph


@pytest.mark.parametrize("kind", ["fc", "block", "block_wide", "mnist_net", "mnist_net_prefold"])
def test_training_step_replays_equal_eager(kind):
    torch.manual_seed(3)
    if kind == "fc":
        model = C.LogicLayer(300, 400, implementation="cuda").to(DEV)
        x = torch.rand(64, 300, device=DEV)
        loss_of = lambda out: (out * out).sum()
    elif kind == "block":
        model = C.ConvLogicLayer(3, 16, padding=1, complete=True).to(DEV)
        x = torch.rand(16, 3, 16, 16, device=DEV)
        loss_of = lambda out: (out * out).sum()
    elif kind == "block_wide":
        model = C.ConvLogicLayer(96, 64, padding=1, complete=True).to(DEV)      # direct forward / input gradient
        x = torch.rand(8, 96, 8, 8, device=DEV)
        loss_of = lambda out: (out * out).sum()
    else:
        model = C.ConvLogicMnistModel(k_param=2).to(DEV)
        if kind == "mnist_net_prefold":
            model.prefold = "always"                               # the launch that folds all layers' logits is part of the graph
        x = torch.randint(0, 2, (32, 1, 28, 28), device=DEV).float()
        labels = torch.randint(0, 10, (32,), device=DEV)
        loss_of = lambda out: torch.nn.functional.cross_entropy(out, labels)
    with torch.no_grad():
        for p in model.parameters():
            p.copy_(torch.randn_like(p))
    static_x = x.clone().requires_grad_(True)
    params = list(model.parameters())

    def run():
        for p in params:
            p.grad = None
        static_x.grad = None
        loss_of(model(static_x)).backward()

    graph = _capture(run)
    for p in params:
        p.grad = None
    static_x.grad = None
    with torch.cuda.graph(graph):
        loss_of(model(static_x)).backward()
    static_grads = [static_x.grad] + [p.grad for p in params]
    assert all(g is not None for g in static_grads)

    eager = copy.deepcopy(model)
    for trial in range(3):
        new_x = torch.rand_like(x) if not kind.startswith("mnist_net") else torch.randint(0, 2, x.shape, device=DEV).float()
        with torch.no_grad():
            static_x.copy_(new_x)
        for g in static_grads:
            g.fill_(float("nan"))                        # a replay has to rewrite every gradient
        graph.replay()
        torch.cuda.synchronize()
        # eager work of the program between replays
        ex = new_x.clone().requires_grad_(True)
        for p in eager.parameters():
            p.grad = None
        loss_of(eager(ex)).backward()
        torch.cuda.synchronize()
        want = [ex.grad] + [p.grad for p in eager.parameters()]
        for i, (got, ref) in enumerate(zip(static_grads, want)):
            assert torch.equal(got, ref), (kind, trial, i, (got - ref).abs().max().item())


def test_graphed_step_helper_trains_like_eager_steps():
    # GraphedStep on the CIFAR topology with an optimizer outside the graph: three steps on different batches
    # give the same losses and parameters as three eager steps from the same start
    torch.manual_seed(5)
    model = C.ConvLogicCifarModel(k_param=2, input_channels=3, input_size=32, tau=10).to(DEV)
    twin = copy.deepcopy(model)
    batches = [(torch.randint(0, 2, (64, 3, 32, 32), device=DEV).float(), torch.randint(0, 10, (64,), device=DEV)) for _ in range(3)]
    ce = torch.nn.functional.cross_entropy
    step = C.GraphedStep(lambda x, y: ce(model(x), y), batches[0], model.parameters())
    opt_g = torch.optim.SGD(model.parameters(), lr=0.1)
    opt_e = torch.optim.SGD(twin.parameters(), lr=0.1)
    for x, y in batches:
        loss_g = step(x, y).clone()
        opt_g.step()
        torch.cuda.synchronize()
        opt_e.zero_grad(set_to_none=True)
        loss_e = ce(twin(x), y)
        loss_e.backward()
        opt_e.step()
        assert torch.equal(loss_g, loss_e.detach())
        for pg, pe in zip(model.parameters(), twin.parameters()):
            assert torch.equal(pg, pe)
    with pytest.raises(ValueError):
        step(batches[0][0][:32], batches[0][1][:32])
