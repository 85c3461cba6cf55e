"""Activation recomputation that keeps no output: the helper ``GmmExpertsImpl.forward`` wraps its activation in.

Behaves like ``CheckpointWithoutOutput`` of mindspeed/core/tensor_parallel/random.py:94-192: ``checkpoint`` runs the
function without recording a graph and remembers its inputs; ``discard_output`` releases the storage of what it
returned once the consumer (the second grouped matmul) has run; ``recompute``, registered as a gradient hook on the
consumer's output, runs the function again with a graph, puts the values back into the very tensors the consumer
saved, and the checkpoint node's backward then differentiates through the recomputed graph.  Random-number state is
restored around the second run, as in the reference, so a function that draws random numbers repeats them.
"""
from __future__ import annotations

import torch

__all__ = ["CheckpointWithoutOutput"]


class _Node(torch.autograd.Function):
    @staticmethod
    def forward(ctx, run_function, manager, *args):
        with torch.no_grad():
            outputs = run_function(*args)
        ctx.save_for_backward(*[a.detach().requires_grad_(a.requires_grad) if isinstance(a, torch.Tensor) else a
                                for a in args])
        ctx.recomputed = None
        manager.ctx = ctx
        return outputs

    @staticmethod
    def backward(ctx, *grads):
        if ctx.recomputed is None:
            raise RuntimeError("CheckpointWithoutOutput: backward reached the checkpoint before recompute() ran "
                               "(register manager.recompute as a hook on the consumer's output)")
        inputs = ctx.saved_tensors
        pairs = [(o, g) for o, g in zip(ctx.recomputed, grads) if torch.is_tensor(o) and o.grad_fn is not None]
        if pairs:
            torch.autograd.backward([o for o, _ in pairs], [g for _, g in pairs])
        ctx.recomputed = None
        return (None, None) + tuple(inp.grad if isinstance(inp, torch.Tensor) else None for inp in inputs)


class CheckpointWithoutOutput:
    def __init__(self):
        self.run_function = None
        self.outputs = None
        self.ctx = None
        self._cpu_rng = None
        self._dev_rng = None

    def checkpoint(self, run_function, distribute_saved_activations, *args):
        if distribute_saved_activations:
            raise RuntimeError("CheckpointFunctionWithoutOutput does not support distribute_saved_activations")
        self.run_function = run_function
        self._cpu_rng = torch.get_rng_state()
        self._dev_rng = torch.cuda.get_rng_state() if torch.cuda.is_available() else None
        outputs = _Node.apply(run_function, self, *args)
        self.outputs = (outputs,) if isinstance(outputs, torch.Tensor) else tuple(outputs)
        return outputs

    def discard_output(self):
        for out in self.outputs:
            out.untyped_storage().resize_(0)

    def recompute(self, _):
        if not torch.autograd._is_checkpoint_valid():
            raise RuntimeError("Checkpointing is not compatible with .grad(), please use .backward() if possible")
        cpu_now = torch.get_rng_state()
        dev_now = torch.cuda.get_rng_state() if self._dev_rng is not None else None
        torch.set_rng_state(self._cpu_rng)
        if self._dev_rng is not None:
            torch.cuda.set_rng_state(self._dev_rng)
        with torch.enable_grad():
            again = self.run_function(*self.ctx.saved_tensors)
        torch.set_rng_state(cpu_now)
        if dev_now is not None:
            torch.cuda.set_rng_state(dev_now)
        again = (again,) if isinstance(again, torch.Tensor) else tuple(again)
        for out, new in zip(self.outputs, again):
            out.untyped_storage().resize_(new.untyped_storage().size())
            with torch.no_grad():
                out.untyped_storage().copy_(new.untyped_storage())
        self.ctx.recomputed = again
        self.run_function = None
        self.outputs = None
        self.ctx = None
