"""Tensor helpers of the public package (reference src/trifast/utils.py)."""

from __future__ import annotations

from functools import wraps

import torch


def gen_tensors(
    n: int,
    d: int,
    h: int,
    use_mask: bool,
    device: torch.device,
    dtype: torch.dtype,
    batch: int = 1,
    std: float = 1.0,
):
    """Random q, k, v [batch,h,n,n,d], bias [batch,h,n,n] (all requiring grad) and a
    bool mask [batch,n,n] that is 50 % True when ``use_mask`` else all False
    (reference src/trifast/utils.py:5-33)."""
    def normal(*shape):
        return torch.normal(0, std, shape, device=device, dtype=dtype, requires_grad=True)

    q = normal(batch, h, n, n, d)
    k = normal(batch, h, n, n, d)
    v = normal(batch, h, n, n, d)
    b = normal(batch, h, n, n)
    if use_mask:
        m = torch.randint(0, 2, (batch, n, n), device=device, dtype=torch.bool)
    else:
        m = torch.zeros((batch, n, n), device=device, dtype=torch.bool)
    return q, k, v, b, m


def clone_and_clear_grad(*tensors):
    """Clone the gradients of ``tensors`` and reset them (reference utils.py:36-44)."""
    grads = tuple(t.grad.clone() if t.grad is not None else None for t in tensors)
    for t in tensors:
        t.grad = None
    return grads


def _with_tf32(enabled: bool):
    def deco(fn):
        @wraps(fn)
        def wrapped(*args, **kwargs):
            old = (torch.backends.cuda.matmul.allow_tf32, torch.backends.cudnn.allow_tf32)
            torch.backends.cuda.matmul.allow_tf32 = enabled
            torch.backends.cudnn.allow_tf32 = enabled
            try:
                return fn(*args, **kwargs)
            finally:
                torch.backends.cuda.matmul.allow_tf32, torch.backends.cudnn.allow_tf32 = old

        return wrapped

    return deco


# reference src/trifast/utils.py:47-88; the flags only affect torch's own matmuls
disable_tf32 = _with_tf32(False)
enable_tf32 = _with_tf32(True)
