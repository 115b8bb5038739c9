"""HIP-graph replay of a training step.

The kernels of this package launch on the current stream, never synchronise and never allocate, so the
forward + loss + backward of a model built from its modules can be recorded once into a HIP graph
(torch.cuda.CUDAGraph) and replayed with one launch call per step.  For the small and medium layers the step
is then bound by the GPU instead of by Python and the autograd engine.
"""
import torch


class GraphedStep:
    """Records ``loss = loss_fn(*inputs); loss.backward()`` and replays it.

        step = GraphedStep(lambda x, y: F.cross_entropy(model(x), y), (x0, y0), model.parameters())
        for x, y in batches:            # same shapes and dtypes as x0, y0
            loss = step(x, y)           # gradients are in p.grad of the parameters
            optimizer.step()

    The inputs are copied into buffers owned by the step; the returned loss and the parameters' ``.grad`` tensors
    are overwritten by every call.  Shapes, dtypes, training/eval mode, wiring buffers and environment knobs are
    those of the recording.  ``input_grads=True`` also keeps the gradients of floating-point inputs
    (``step.input_grads``).
    """

    def __init__(self, loss_fn, example_inputs, parameters, warmup=3, input_grads=False):
        self.loss_fn = loss_fn
        self.parameters = [p for p in parameters if p.requires_grad]
        self.inputs = [t.detach().clone() for t in example_inputs]
        if input_grads:
            for t in self.inputs:
                if t.is_floating_point():
                    t.requires_grad_(True)
        if not all(t.is_cuda for t in self.inputs) or not all(p.is_cuda for p in self.parameters):
            raise RuntimeError("GraphedStep needs inputs and parameters on the GPU")
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):                     # lets lazy initialisation and plan caches settle
            for _ in range(warmup):
                self._eager()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        self._clear_grads()                               # the recording allocates the gradient tensors it will refill
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self.loss = self._eager(clear=False)

    def _clear_grads(self):
        for t in self.parameters + self.inputs:
            t.grad = None

    def _eager(self, clear=True):
        if clear:
            self._clear_grads()
        loss = self.loss_fn(*self.inputs)
        loss.backward()
        return loss.detach()

    @property
    def input_grads(self):
        return [t.grad for t in self.inputs]

    def __call__(self, *inputs):
        if len(inputs) != len(self.inputs):
            raise ValueError(f"expected {len(self.inputs)} inputs, got {len(inputs)}")
        with torch.no_grad():
            for dst, src in zip(self.inputs, inputs):
                if dst.shape != src.shape or dst.dtype != src.dtype:
                    raise ValueError(f"input of shape {tuple(src.shape)} / {src.dtype} does not match the recorded "
                                     f"{tuple(dst.shape)} / {dst.dtype}")
                dst.copy_(src)
        self.graph.replay()
        return self.loss
