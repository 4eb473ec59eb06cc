"""One autograd node for every forward / backward operator pair of the extension.

An operator pair is described by a `KernelPair`: `launch` runs the forward operator and says what the backward needs
(tensors to keep, plain values to remember), `grads` runs the backward operator and returns one gradient per tensor
argument. `KernelPair.__call__` records a single `torch.autograd.Function` node whichever pair it is, so the wiring
(saved tensors, non-differentiable outputs, once-differentiable backward, contiguous upstream gradients, float32 under
autocast) is written once.
"""
from __future__ import annotations

from typing import Any, Callable, Optional, Sequence, Tuple

import torch
from torch import Tensor
from torch.autograd.function import once_differentiable

from fast_sp_gs_amd._C import get_C_function


def _contiguous(t):
    return t.contiguous() if isinstance(t, Tensor) else t


class KernelPair:
    """forward_name / backward_name: operator names resolved through `get_C_function` when the pair is created (the
    extension must be loadable by then, as for the reference's class-level bindings).
    launch(fwd, needs, *args) -> (outputs, keep, remember): `outputs` a tensor or tuple of tensors, `keep` the tensors
    the backward reads, `remember` any plain values. grads(bwd, needs, keep, remember, *upstream) -> one entry per
    element of *args (None for non-tensors and for inputs without a gradient).
    non_differentiable: indices of outputs that carry no gradient (index lists, detached statistics).
    autocast_float32: run in float32 under autocast (the reference's custom_fwd(cast_inputs=float32) operators)."""

    def __init__(self, forward_name: str, backward_name: Optional[str], launch: Callable, grads: Optional[Callable],
                 non_differentiable: Sequence[int] = (), autocast_float32: bool = False):
        self.fwd = get_C_function(forward_name)
        self.bwd = get_C_function(backward_name) if backward_name else None
        self.launch, self.grads = launch, grads
        self.non_differentiable = tuple(non_differentiable)
        self.autocast_float32 = autocast_float32

    def __call__(self, *args):
        return _KernelNode.apply(self, *args)


class _KernelNode(torch.autograd.Function):
    @staticmethod
    def forward(ctx, pair: KernelPair, *args):
        if pair.autocast_float32 and torch.is_autocast_enabled():
            args = tuple(a.float() if isinstance(a, Tensor) and a.is_floating_point() else a for a in args)
            with torch.autocast('cuda', enabled=False):
                return _KernelNode._run(ctx, pair, args)
        return _KernelNode._run(ctx, pair, args)

    @staticmethod
    def _run(ctx, pair: KernelPair, args: Tuple[Any, ...]):
        needs = ctx.needs_input_grad[1:]
        outputs, keep, remember = pair.launch(pair.fwd, needs, *[_contiguous(a) for a in args])
        ctx.pair, ctx.remember = pair, remember
        # the backward gets its saved tensors with the Nones where launch put them
        ctx.keep_mask = tuple(k is not None for k in keep)
        ctx.save_for_backward(*[k for k in keep if k is not None])
        many = isinstance(outputs, (tuple, list))
        for i in pair.non_differentiable:
            ctx.mark_non_differentiable(outputs[i] if many else outputs)
        return tuple(outputs) if many else outputs

    @staticmethod
    @once_differentiable
    def backward(ctx, *upstream):
        pair = ctx.pair
        saved = iter(ctx.saved_tensors)
        keep = tuple(next(saved) if present else None for present in ctx.keep_mask)
        with torch.autocast('cuda', enabled=False):
            g = pair.grads(pair.bwd, ctx.needs_input_grad[1:], keep, ctx.remember, *[_contiguous(u) for u in upstream])
        return (None, *g)
