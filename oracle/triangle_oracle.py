"""CPU oracle for fused triangle self-attention.  TEST INFRASTRUCTURE ONLY.

This module is a checker: it is imported by the tests, by the smoke check and by
the CPU-baseline leg of the benchmark, and by nothing else.  The shipped operator
never calls into it and has no CPU fallback.

It restates, in plain PyTorch / numpy, the pure-PyTorch triangle attention that
the reference uses as ground truth for its Triton kernels:

  * ``neg_inf``                   follows reference src/trifast/equiv.py:12-13
  * ``attention_reference``       follows reference src/trifast/equiv.py:42-69
    (matmul, additive ``finfo.min`` key mask, bias broadcast over rows, softmax,
    matmul) -- THE ground truth of reference tests/unit/test_trifast.py:50,111
  * ``triangle_attention_simple`` follows reference src/trifast/equiv.py:16-39
    (einsum + ``masked_fill_``) -- an independent second formulation
  * ``gen_tensors``               follows reference src/trifast/utils.py:5-33
  * ``compare_values`` & friends  follow reference tests/utils.py:31-83 and
    tests/unit/test_trifast.py:19-23,73-89

Tensor layout (reference src/trifast/torch.py:220-226):
  q, k, v : [b, h, n, n, d]   q[b,h,i,j,:] attends over k[b,h,i,k,:], v[b,h,i,k,:]
  bias    : [b, h, n, n]      indexed [j, k], shared by every row i
  mask    : [b, n, n] bool    indexed [i, k], True = key k of row i is masked OUT
  o       : [b, h, n, n, d]

How the restatement is pinned (tests/test_oracle.py), since the reference holds
no stored vectors for this path: forward against
``torch.nn.functional.scaled_dot_product_attention``, against a float64
brute-force loop nest and against the second formulation; log-sum-exp against
``torch.logsumexp``; gradients against float64 closed forms written with explicit
loops, against ``torch.autograd.gradcheck`` and against invariants of softmax
attention (rows of P sum to one, db sums to zero over keys, masked keys get zero
gradient in partially masked rows, rows/heads/batches are independent).
"""

from __future__ import annotations

import math

import numpy as np
import torch


def neg_inf(dtype: torch.dtype) -> float:
    # reference src/trifast/equiv.py:12-13
    return torch.finfo(dtype).min


def attention_reference(q, k, v, bias, mask):
    """Ground-truth forward.  Follows reference src/trifast/equiv.py:42-69.

    The mask is ADDITIVE (finfo.min * mask), not a fill: in a row whose keys are
    all masked every logit saturates to the same value and the softmax is
    uniform over all n keys, and autograd sends gradient through such rows.
    """
    mask_bias = neg_inf(q.dtype) * mask.to(q.dtype)  # [b, i, k]
    sm_scale = q.shape[-1] ** -0.5

    qp = q.permute(0, 2, 1, 3, 4)  # b i h j d
    kp = k.permute(0, 2, 1, 4, 3)  # b i h d k
    vp = v.permute(0, 2, 1, 3, 4)  # b i h k d

    a = torch.matmul(qp, kp) * sm_scale  # b i h j k
    a += mask_bias[:, :, None, None, :]
    a += bias[:, None, :, :, :]
    a = torch.softmax(a, dim=-1)
    o = torch.matmul(a, vp)  # b i h j d
    return o.permute(0, 2, 1, 3, 4)


def triangle_attention_simple(q, k, v, bias, mask):
    """Second formulation.  Follows reference src/trifast/equiv.py:16-39."""
    q = q * (q.shape[-1] ** -0.5)
    s = torch.einsum("bhijd,bhikd->bhijk", q, k)
    s = s + bias[:, :, None, :, :]
    s = s.masked_fill(mask[:, None, :, None, :], neg_inf(q.dtype))
    a = torch.softmax(s, dim=-1)
    return torch.einsum("bhijk,bhikd->bhijd", a, v)


def logits_reference(q, k, bias, mask):
    """The pre-softmax logits of ``attention_reference`` as [b, h, i, j, k]."""
    sm_scale = q.shape[-1] ** -0.5
    a = torch.matmul(q, k.transpose(-1, -2)) * sm_scale  # b h i j k
    a = a + (neg_inf(q.dtype) * mask.to(q.dtype))[:, None, :, None, :]
    a = a + bias[:, :, None, :, :]
    return a


def lse_reference(q, k, bias, mask):
    """Natural-log log-sum-exp of the logits, [b, h, i, j] float32.

    The operator returns this as its second output (reference
    src/trifast/torch.py:43,65; kernel epilogue src/trifast/triton.py:130-132).
    """
    return torch.logsumexp(logits_reference(q, k, bias, mask).float(), dim=-1)


def forward_backward(q, k, v, bias, mask, do, fn=attention_reference):
    """o, dq, dk, dv, db of ``fn`` by autograd, on detached copies."""
    q, k, v, bias = (t.detach().clone().requires_grad_(True) for t in (q, k, v, bias))
    o = fn(q, k, v, bias, mask)
    o.backward(do)
    return o.detach(), q.grad, k.grad, v.grad, bias.grad


def forward_backward_chunked(q, k, v, bias, mask, do, chunk: int = 32, want_grads: bool = True):
    """Same numbers as ``forward_backward(attention_reference)``, row-chunked.

    Rows i are independent except for db = sum_i dS, so the b*h*n^3 logits are
    only ever live for ``chunk`` rows at a time; db is accumulated across chunks
    in the input dtype's float32 upcast.  Used where n^3 does not fit.
    """
    b, h, n, _, d = q.shape
    o = torch.empty_like(q)
    dq = torch.empty_like(q) if want_grads else None
    dk = torch.empty_like(k) if want_grads else None
    dv = torch.empty_like(v) if want_grads else None
    db = torch.zeros(bias.shape, dtype=torch.float32, device=bias.device) if want_grads else None
    for i0 in range(0, n, chunk):
        sl = slice(i0, min(n, i0 + chunk))
        qc, kc, vc = (t[:, :, sl].detach().clone().requires_grad_(want_grads) for t in (q, k, v))
        bc = bias.detach().clone().requires_grad_(want_grads)
        oc = attention_reference(qc, kc, vc, bc, mask[:, sl])
        o[:, :, sl] = oc.detach()
        if want_grads:
            oc.backward(do[:, :, sl])
            dq[:, :, sl], dk[:, :, sl], dv[:, :, sl] = qc.grad, kc.grad, vc.grad
            db += bc.grad.float()
    if want_grads:
        db = db.to(bias.dtype)
    return o, dq, dk, dv, db


# --------------------------------------------------------------------------
# float64 loop-nest restatements: slow, tiny inputs only.  They share no code
# with the tensor formulations above, which is what makes them a pin.
# --------------------------------------------------------------------------
def brute_force_f64(q, k, v, bias, mask, do=None, mask_min=None):
    """Explicit loops in float64 numpy.

    Returns o, lse (and dq, dk, dv, db when ``do`` is given).  ``mask_min`` is the
    additive mask value (defaults to float32's finfo.min, the value the fp32
    ground truth uses).
    """
    q, k, v, bias = (np.asarray(t.detach().double().numpy()) for t in (q, k, v, bias))
    m = np.asarray(mask.numpy()).astype(bool)
    b, h, n, _, d = q.shape
    scale = 1.0 / math.sqrt(d)
    if mask_min is None:
        mask_min = float(np.finfo(np.float32).min)
    o = np.zeros_like(q)
    lse = np.zeros((b, h, n, n))
    grads = do is not None
    if grads:
        do = np.asarray(do.detach().double().numpy())
        dq, dk, dv, db = np.zeros_like(q), np.zeros_like(k), np.zeros_like(v), np.zeros_like(bias)
    for bi in range(b):
        for hi in range(h):
            for i in range(n):
                for j in range(n):
                    s = np.empty(n)
                    for kk in range(n):
                        dot = 0.0
                        for c in range(d):
                            dot += q[bi, hi, i, j, c] * k[bi, hi, i, kk, c]
                        s[kk] = dot * scale
                        # float32 saturation of (finfo.min + x) is what makes a
                        # fully masked row uniform; reproduce it by rounding.
                        if m[bi, i, kk]:
                            s[kk] = float(np.float32(s[kk]) + np.float32(mask_min))
                        s[kk] = s[kk] + bias[bi, hi, j, kk]
                        if m[bi, i, kk]:
                            s[kk] = float(np.float32(s[kk]))
                    mx = s.max()
                    e = np.exp(s - mx)
                    den = e.sum()
                    p = e / den
                    lse[bi, hi, i, j] = mx + math.log(den)
                    for c in range(d):
                        acc = 0.0
                        for kk in range(n):
                            acc += p[kk] * v[bi, hi, i, kk, c]
                        o[bi, hi, i, j, c] = acc
                    if grads:
                        dp = np.empty(n)
                        for kk in range(n):
                            acc = 0.0
                            for c in range(d):
                                acc += do[bi, hi, i, j, c] * v[bi, hi, i, kk, c]
                            dp[kk] = acc
                        delta = float((p * dp).sum())
                        ds = p * (dp - delta)
                        for kk in range(n):
                            db[bi, hi, j, kk] += ds[kk]
                            for c in range(d):
                                dv[bi, hi, i, kk, c] += p[kk] * do[bi, hi, i, j, c]
                                dq[bi, hi, i, j, c] += scale * ds[kk] * k[bi, hi, i, kk, c]
                                dk[bi, hi, i, kk, c] += scale * ds[kk] * q[bi, hi, i, j, c]
    if grads:
        return o, lse, dq, dk, dv, db
    return o, lse


# --------------------------------------------------------------------------
# Input generators
# --------------------------------------------------------------------------
def gen_tensors(n, d, h, use_mask, device="cpu", dtype=torch.float32, batch=1, std=1.0, generator=None):
    """Follows reference src/trifast/utils.py:5-33: draw order q, k, v, bias, mask;
    mask is randint(0, 2) i.e. 50 % masked."""
    kw = dict(device=device, dtype=dtype, generator=generator)
    q = torch.normal(0, std, (batch, h, n, n, d), **kw).requires_grad_(True)
    k = torch.normal(0, std, (batch, h, n, n, d), **kw).requires_grad_(True)
    v = torch.normal(0, std, (batch, h, n, n, d), **kw).requires_grad_(True)
    b = torch.normal(0, std, (batch, h, n, n), **kw).requires_grad_(True)
    if use_mask:
        m = torch.randint(0, 2, (batch, n, n), device=device, generator=generator).bool()
    else:
        m = torch.zeros((batch, n, n), device=device, dtype=torch.bool)
    return q, k, v, b, m


# --------------------------------------------------------------------------
# Acceptance rules of the reference's tests
# --------------------------------------------------------------------------
DTYPE_EPS = {  # reference tests/unit/test_trifast.py:19-23
    torch.float16: 1e-3,
    torch.bfloat16: 1e-3,
    torch.float32: 1e-4,
}


def max_abs_err(a, ref):
    return (a.float() - ref.float()).abs().max().item()


def compare_values(kernel, pt, ref, msg="", eps=1e-4):
    """reference tests/utils.py:31-36: max|kernel-ref| <= 3 * (max|pt-ref| + eps)."""
    a = max_abs_err(kernel, ref)
    b = max_abs_err(pt, ref) + eps
    assert a <= 3 * b, f"{msg} value mismatch, kernel: {a:.3e}, pt: {b:.3e}"
    return a, b


def cosine_similarity(a, b, eps=1e-8):
    # reference tests/utils.py:43-53
    a = a.float().flatten()
    b = b.float().flatten()
    return (torch.dot(a, b) / (torch.norm(a) * torch.norm(b) + eps)).item()


def compare_directions(kernel, pt, ref, msg="", threshold=0.99):
    # reference tests/utils.py:56-67
    ck, cp = cosine_similarity(kernel, ref), cosine_similarity(pt, ref)
    assert ck > threshold, f"{msg} kernel->ref direction mismatch: {ck:.4f}"
    assert cp > threshold, f"{msg} pt->ref direction mismatch: {cp:.4f}"


def compare_relative_direction(kernel, pt, ref, msg="", ratio=0.99):
    # reference tests/utils.py:70-83
    ck, cp = cosine_similarity(kernel, ref), cosine_similarity(pt, ref)
    assert ck >= ratio * cp, f"{msg} relative direction mismatch: {ck:.4f} vs {ratio * cp:.4f}"


def compare_dot(kernel, pt, ref, msg="", threshold=0.01):
    # reference tests/unit/test_trifast.py:73-89
    def dot(x, y):
        return torch.dot(x.float().flatten(), y.float().flatten())

    mag = dot(ref, ref)
    err = (dot(kernel, ref) / mag - dot(pt, ref) / mag).item()
    assert err >= -threshold, f"{msg} dot product mismatch: {err:.4f}"
