"""Decorators of the operator boundary, mirroring HRDPLR/utils.py:7-25."""
import functools

import torch

# torch.amp.custom_fwd/custom_bwd keep the autocast state of the forward call for the backward call
# (HRDPLR/utils.py:7-12); ROCm builds of torch use the "cuda" device type too.
autocast_custom_fwd = functools.partial(torch.amp.custom_fwd, device_type="cuda")
autocast_custom_bwd = functools.partial(torch.amp.custom_bwd, device_type="cuda")


def contiguous(fn):
    """Make every tensor argument contiguous before the wrapped autograd method runs (HRDPLR/utils.py:14-25)."""
    @functools.wraps(fn)
    def wrapper(ctx, *args, **kwargs):
        return fn(ctx,
                  *(x.contiguous() if isinstance(x, torch.Tensor) else x for x in args),
                  **{k: (x.contiguous() if isinstance(x, torch.Tensor) else x) for k, x in kwargs.items()})
    return wrapper
