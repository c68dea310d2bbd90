"""Whether a convolution's forward pass has to keep its projection for a backward pass.

Inside ``Function.forward`` autograd has gradient mode switched off and ``ctx.needs_input_grad`` only says which
inputs are marked as requiring a gradient (parameters always are), so a forward pass under ``torch.no_grad()`` cannot
tell from there that nothing will ever ask it for gradients.  ``ConvFunction.apply`` notes the caller's gradient mode
on the way in; ``keeps_projection(ctx)`` is then true only if a backward pass can follow.  A forward pass that keeps
nothing lets the library run the gather and the contraction as one kernel."""
import threading

import torch

_state = threading.local()


class ConvFunction(torch.autograd.Function):
    @classmethod
    def apply(cls, *args, **kwargs):
        stack = _state.__dict__.setdefault("grad_mode", [])
        stack.append(torch.is_grad_enabled())
        try:
            return super().apply(*args, **kwargs)
        finally:
            stack.pop()


def keeps_projection(ctx):
    stack = _state.__dict__.get("grad_mode")
    outer = stack[-1] if stack else True
    return outer and any(ctx.needs_input_grad)
