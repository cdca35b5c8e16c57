"""HIP-graph replay of a whole training step, and of packed inference.

A logic-gate net's step is dozens of short kernels (per layer: softmax, forward, backward_x,
backward_w, softmax backward; each tens of microseconds at the reference's batch sizes), so an
eager step is bound by host launch overhead rather than by the GPU.  ``GraphedTrainStep``
captures forward + loss + backward (and optionally the optimizer step) once into a HIP graph on
static buffers and replays it per step.
"""
import torch


class GraphedTrainStep:
    """Captures ``loss = loss_fn(model(x), y); loss.backward()[; optimizer.step()]``.

    ``step(x, y)`` copies the batch into the static input buffers, replays the graph and returns
    the static loss tensor (valid until the next replay).  Parameter gradients are the
    ``.grad`` tensors of the parameters, rewritten by every replay.  Shapes and dtypes are fixed
    at construction.  With ``optimizer`` given it must be constructed with ``capturable=True``.
    """

    def __init__(self, model, loss_fn, example_x, example_y, optimizer=None, warmup=3):
        self.model, self.loss_fn, self.optimizer = model, loss_fn, optimizer
        self.x = example_x.detach().clone()
        self.y = example_y.detach().clone()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(warmup):
                self._eager()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        self.graph = torch.cuda.CUDAGraph()
        self._zero_grad()
        with torch.cuda.graph(self.graph):
            self.loss = self._eager(zero=False)

    def _zero_grad(self):
        if self.optimizer is not None:
            self.optimizer.zero_grad(set_to_none=True)
        else:
            self.model.zero_grad(set_to_none=True)

    def _eager(self, zero=True):
        if zero:
            self._zero_grad()
        loss = self.loss_fn(self.model(self.x), self.y)
        loss.backward()
        if self.optimizer is not None:
            self.optimizer.step()
        return loss

    def step(self, x=None, y=None):
        if x is not None:
            self.x.copy_(x, non_blocking=True)
        if y is not None:
            self.y.copy_(y, non_blocking=True)
        self.graph.replay()
        return self.loss


class GraphedPackedInference:
    """Captures ``model(PackBitsTensor(x, bit_count))`` -- packing, every gate layer, the count -- for a
    model in eval mode and a fixed input shape, and replays it per batch: one graph launch instead of
    a dozen kernel launches and their Python.  ``__call__(x)`` copies the bool batch ``[B, F]`` into
    the static input buffer, replays and returns the static ``[B, k]`` int32 counts (valid until the
    next call).  The gate ids are taken from the weights inside the graph, so weights updated in
    place between calls are seen; a model whose wiring tensors are replaced needs a new capture.
    """

    def __init__(self, model, example_x, bit_count=64, warmup=2):
        from .packbitstensor import PackBitsTensor
        assert not model.training, "packed inference runs the discretised net: call model.eval() first"
        assert example_x.dtype == torch.bool and example_x.dim() == 2 and example_x.is_cuda, (
            example_x.dtype, tuple(example_x.shape), example_x.device)
        self.model, self.bit_count = model, bit_count
        self.x = example_x.detach().clone()

        def run():
            with torch.no_grad():
                return model(PackBitsTensor(self.x, bit_count=bit_count))

        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(warmup):              # also builds and caches the wiring's schedules on the host
                run()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self.out = run()

    def __call__(self, x=None):
        if x is not None:
            self.x.copy_(x, non_blocking=True)
        self.graph.replay()
        return self.out
