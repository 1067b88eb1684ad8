"""Forward-only guard of the module layer.

The kernels compute the inference forward pass: no dropout mask is drawn (the reference's
DropoutRowwise / DropoutColumnwise are the identity only in eval mode, dropout.py:57-58) and no
autograd graph is recorded.  A call that expects either must fail instead of silently returning
an un-dropped, non-differentiable result.
"""
from __future__ import annotations

import functools

import torch


def _tensors(values):
    for v in values:
        if isinstance(v, torch.Tensor):
            yield v
        elif isinstance(v, (list, tuple)):
            yield from _tensors(v)


def refuse_training(module, args=(), kwargs=None):
    """Raises RuntimeError when `module` is in training mode, or when autograd is recording and an
    input tensor asks for a gradient."""
    name = type(module).__name__
    if module.training:
        raise RuntimeError(
            "%s is forward-only (inference): call .eval() first.  In training mode the reference applies "
            "dropout and records gradients; these kernels do neither." % name)
    if torch.is_grad_enabled():
        for t in _tensors(list(args) + list((kwargs or {}).values())):
            if t.requires_grad:
                raise RuntimeError(
                    "%s is forward-only (inference): an input requires a gradient, and the kernels record no "
                    "autograd graph.  Detach the input or call under torch.no_grad()." % name)


def forward_only(fn):
    """Method decorator: refuse_training(self, inputs), then run under torch.no_grad()."""

    @functools.wraps(fn)
    def wrapper(self, *args, **kwargs):
        refuse_training(self, args, kwargs)
        with torch.no_grad():
            return fn(self, *args, **kwargs)

    return wrapper
