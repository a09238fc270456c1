"""Forward (and backward) of a layer at fixed shapes, recorded once in a HIP graph.

At small batch a butterfly layer's kernels take a few microseconds each and the step is bound
by the host: every operator call costs dispatch, output allocation and a kernel launch, and a
layer with folded diagonals or a bias issues several.  Recording the step once and replaying
it removes all of that; the replay is one graph launch.  The native library neither allocates
nor synchronises inside its calls, and the operators' workspaces come from PyTorch's
allocator, which keeps a private pool for a recorded graph, so both record cleanly.

No counterpart in the reference (it predates graph capture in PyTorch).
"""
import torch


class GraphedStep:
    """``y = fn(x)`` and, when ``example_grad`` is given, the gradients of ``y`` with respect to
    ``x`` and ``params`` for the output gradient ``grad``: recorded for the shapes, dtypes and
    device of the example tensors, then replayed by each call.

    ``step(x, grad)`` copies its arguments into the recorded input buffers, replays, and
    returns ``(y, (d_x, *d_params))`` (``(y, ())`` without a backward).  The returned tensors
    are the graph's own output buffers: the next call overwrites them, so copy what must
    outlive it.  ``params`` are read in place by every replay, so in-place updates (an
    optimiser step) are seen; replacing a parameter's storage is not.  Callers that can write
    straight into ``step.input`` / ``step.grad_output`` skip the copies with ``step.replay()``.
    """

    def __init__(self, fn, example_input, example_grad=None, params=(), warmup=2):
        if not example_input.is_cuda:
            raise ValueError("GraphedStep records device work: the example input must be a device tensor")
        self._fn = fn
        self._params = tuple(params)
        self._backward = example_grad is not None
        self.input = example_input.detach().clone().requires_grad_(self._backward)
        self.grad_output = example_grad.detach().clone() if self._backward else None
        # Warm-up on a side stream, as recording requires: lazy initialisation (library handles,
        # the allocator's pools) must not happen while the stream is being recorded.
        side = torch.cuda.Stream(device=example_input.device)
        side.wait_stream(torch.cuda.current_stream(example_input.device))
        with torch.cuda.stream(side):
            for _ in range(max(1, warmup)):
                self._run()
        torch.cuda.current_stream(example_input.device).wait_stream(side)
        torch.cuda.synchronize(example_input.device)
        self._graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self._graph):
            self.output, self.grads = self._run()

    def _run(self):
        y = self._fn(self.input)
        if not self._backward:
            return y.detach(), ()
        grads = torch.autograd.grad(y, (self.input,) + self._params, self.grad_output)
        return y.detach(), grads

    def replay(self):
        """Run the recorded step on whatever ``input`` / ``grad_output`` hold now."""
        self._graph.replay()
        return self.output, self.grads

    def __call__(self, x, grad=None):
        if x.shape != self.input.shape or x.dtype != self.input.dtype:
            raise ValueError(f"recorded for input {tuple(self.input.shape)} {self.input.dtype}, "
                             f"got {tuple(x.shape)} {x.dtype}")
        if self._backward != (grad is not None):
            raise ValueError("recorded with a backward pass: pass the output gradient" if self._backward
                             else "recorded without a backward pass: pass no output gradient")
        with torch.no_grad():
            self.input.copy_(x)
            if self._backward:
                if grad.shape != self.grad_output.shape or grad.dtype != self.grad_output.dtype:
                    raise ValueError(f"recorded for output gradient {tuple(self.grad_output.shape)} "
                                     f"{self.grad_output.dtype}, got {tuple(grad.shape)} {grad.dtype}")
                self.grad_output.copy_(grad)
        return self.replay()
