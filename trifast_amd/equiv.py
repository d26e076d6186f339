"""Pure-PyTorch triangle attention, for users who compare against it.

The reference ships these two functions as ``trifast.equiv`` (reference
src/trifast/equiv.py:12-69) and its tests and benchmark scripts import them from
there, so the drop-in package offers them under the same names.  They run on any
device PyTorch supports and materialise the b*h*n^3 logits; the fused operator
never calls them.
"""

from __future__ import annotations

import torch


def neg_inf(dtype: torch.dtype) -> float:
    return torch.finfo(dtype).min


def triangle_attention_simple(q, k, v, bias, mask):
    """einsum formulation with a filled mask (reference src/trifast/equiv.py:16-39).

    q, k, v: [..., h, n, n, d]; bias: [..., h, n, n]; mask: [..., n, n] bool, True = masked
    out; any number of leading batch dims, as in the reference.
    """
    scale = q.shape[-1] ** -0.5
    logits = torch.einsum("...hijd,...hikd->...hijk", q * scale, k) + bias[..., None, :, :]
    logits = logits.masked_fill(mask[..., None, :, None, :], neg_inf(q.dtype))
    return torch.einsum("...hijk,...hikd->...hijd", logits.softmax(dim=-1), v)


def attention_reference(q, k, v, bias, mask):
    """matmul formulation with an additive ``finfo.min`` mask (reference
    src/trifast/equiv.py:42-69): the ground truth of the reference's tests.  A row
    whose keys are all masked attends uniformly and carries gradient."""
    scale = q.shape[-1] ** -0.5
    # rows i become a batch dim: [b, i, h, j|k, d]
    qr, kr, vr = (t.transpose(1, 2) for t in (q, k, v))
    logits = (qr @ kr.transpose(-1, -2)) * scale
    logits = logits + (neg_inf(q.dtype) * mask.to(q.dtype))[:, :, None, None, :]
    logits = logits + bias[:, None]
    return (logits.softmax(dim=-1) @ vr).transpose(1, 2)
