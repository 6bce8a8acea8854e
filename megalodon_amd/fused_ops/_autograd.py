"""One generic bridge from the library's forward / backward entry points to
`torch.autograd.Function`.

An operator is described by two plain functions:

* ``run(*args) -> (outputs, saved, consts)``: `outputs` is what the caller
  receives (a tensor or a tuple), `saved` the tensors (or None) the backward
  pass needs, `consts` any non-tensor state, and
* ``grad(consts, saved, *output_grads) -> tuple`` with one entry per argument
  of ``run`` (None for non-tensor arguments; entries for arguments the caller
  left at their defaults are dropped).

`fused_op` turns the pair into a Function class with the given name; outputs
listed in `non_differentiable` are marked as such."""
from typing import Callable, Sequence

import torch


def fused_op(name: str, run: Callable, grad: Callable, non_differentiable: Sequence[int] = (), doc: str = ""):
    def forward(ctx, *args):
        outputs, saved, consts = run(*args)
        ctx.consts = consts
        ctx.n_args = len(args)  # trailing arguments may have been left at their defaults
        ctx.save_for_backward(*saved)
        if non_differentiable:
            ctx.mark_non_differentiable(*(outputs[i] for i in non_differentiable))
        return outputs

    def backward(ctx, *output_grads):
        grads = tuple(grad(ctx.consts, ctx.saved_tensors, *output_grads))
        return (grads + (None,) * ctx.n_args)[:ctx.n_args]

    return type(name, (torch.autograd.Function,),
                {"forward": staticmethod(forward), "backward": staticmethod(backward), "__doc__": doc or name})
