"""Callers of the operator: the gated triangle-attention block of AlphaFold-style models.

The reference ships the operator only; its tests hint at the surrounding module
(reference tests/unit/test_trifast.py:152-169: linear layers for q, k, v and the bias over
a pair representation ``x [*, n, n, c]``).  This module is that block written so that no
tensor is copied to change its layout:

* q, k, v are written by their projection heads-outermost, ``[h, *, n, n, d]``, and go to the
  operator as ``[*, h, n, n, d]`` views: its fastest layout (interleaved heads, which is what
  separate linear layers produce, share every 128-byte line between two heads); the bias as a
  ``[*, h, n, n]`` view of ``[*, n, n, h]``.  The operator reads them through their strides
  and writes dq, dk, dv, db with the same strides, so autograd needs no re-layout copy on the
  way back either, and the projections' backward reads the heads-outermost gradients as
  they are.
* The weight gradients of the six linear layers come from ``trifast_linear_dw``: for rows in
  the millions and a few hundred channels the BLAS library runs that product (a contraction
  over all rows into a tiny matrix) on one or two workgroups, ten times slower than the
  layer's other two products.  The five projections of x are one pass over x
  (``trifast_linear_fwd``) and their input gradient is one pass (``trifast_linear_dx``)
  instead of five products and four additions.
* The output gate ``o * sigmoid(g)`` and the layout change from the operator's
  ``[*, h, n, n, d]`` to the ``[*, n, n, h*d]`` that the output projection consumes are one
  streaming HIP kernel (``trifast_gate_fwd`` / ``trifast_gate_bwd``).
"""

from __future__ import annotations

from typing import Optional, Sequence

import torch

from trifast_amd import _lib
from trifast_amd.torch import _dtype_code, triangle_attention, triangle_attention_ending_node


def _gate_shapes(o: torch.Tensor, g: torch.Tensor) -> tuple[int, int, int, int]:
    if o.dim() < 4:
        raise ValueError(f"o must be [*, h, n, n, d], got shape {tuple(o.shape)}")
    *lead, h, n, n2, d = o.shape
    if n != n2:
        raise ValueError(f"o must be square in its pair dims, got shape {tuple(o.shape)}")
    if tuple(g.shape) != (*lead, n, n, h * d):
        raise ValueError(f"g must be [*, n, n, h*d] = {(*lead, n, n, h * d)}, got {tuple(g.shape)}")
    if g.dtype != o.dtype:
        raise TypeError("o and g must share one dtype")
    if not (o.is_cuda and g.is_cuda and o.device == g.device):
        raise RuntimeError("gated_output runs on the GPU only (o and g on one device)")
    b = 1
    for s in lead:
        b *= s
    return b, h, n, d


def _dims4(o: torch.Tensor) -> tuple[int, int, int, int]:
    *lead, h, n, _, d = o.shape
    b = 1
    for s in lead:
        b *= s
    return b, h, n, d


# The kernels are torch.library custom ops, like the operator itself: opaque to a tracing
# compiler (torch.compile sees one node each), with shape-only implementations for it.
@torch.library.custom_op("trifast::gated_output", mutates_args=())
def _gated_output(o: torch.Tensor, g: torch.Tensor) -> torch.Tensor:
    b, h, n, d = _dims4(o)
    o, g = o.contiguous(), g.contiguous()
    y = torch.empty_like(g)
    if y.numel():
        with torch.cuda.device(o.device):
            rc = _lib.load().trifast_gate_fwd(y.data_ptr(), o.data_ptr(), g.data_ptr(), b, h, n, d, _dtype_code(o),
                                              torch.cuda.current_stream(o.device).cuda_stream)
        _lib.check(rc, "trifast_gate_fwd")
    return y


@_gated_output.register_fake
def _(o, g):
    return g.new_empty(g.shape)


@torch.library.custom_op("trifast::gated_output_backward", mutates_args=())
def _gated_output_bwd(dy: torch.Tensor, o: torch.Tensor, g: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    b, h, n, d = _dims4(o)
    dy, o, g = dy.contiguous(), o.contiguous(), g.contiguous()
    do, dg = torch.empty_like(o), torch.empty_like(g)
    if dy.numel():
        with torch.cuda.device(o.device):
            rc = _lib.load().trifast_gate_bwd(do.data_ptr(), dg.data_ptr(), dy.data_ptr(), o.data_ptr(), g.data_ptr(),
                                              b, h, n, d, _dtype_code(o), torch.cuda.current_stream(o.device).cuda_stream)
        _lib.check(rc, "trifast_gate_bwd")
    return do, dg


@_gated_output_bwd.register_fake
def _(dy, o, g):
    return o.new_empty(o.shape), g.new_empty(g.shape)


def _gate_setup(ctx, inputs, output) -> None:
    ctx.save_for_backward(*inputs)


def _gate_backward(ctx, dy):
    o, g = ctx.saved_tensors
    return _gated_output_bwd(dy, o, g)


_gated_output.register_autograd(_gate_backward, setup_context=_gate_setup)


def gated_output(o: torch.Tensor, g: torch.Tensor) -> torch.Tensor:
    """``y[*, i, j, h*d] = o[*, h, i, j, d] * sigmoid(g[*, i, j, h*d])``: the operator's output
    gated and handed to the output projection in one pass."""
    _gate_shapes(o, g)
    return _gated_output(o, g)


_DW_K = (32, 64, 128, 256)


def _dw_ready(x: torch.Tensor, weight: torch.Tensor) -> bool:
    """Shapes and types the weight-gradient kernel takes; anything else is torch's product."""
    return x.is_cuda and x.dtype in (torch.bfloat16, torch.float16) and weight.dtype == x.dtype and x.shape[-1] in _DW_K and x.numel() > 0


def _rows_n(dy: torch.Tensor, head_dim: int) -> tuple[int, int]:
    """rows and outputs of a layer's output gradient: ``[rows, n]``, or ``[n / head_dim, rows,
    head_dim]`` for a layer kept heads-outermost."""
    return (dy.shape[1], dy.shape[0] * dy.shape[2]) if head_dim else (dy.shape[0], dy.shape[1])


@torch.library.custom_op("trifast::linear_weight_grad", mutates_args=())
def _linear_weight_grad(dy: torch.Tensor, x: torch.Tensor, head_dim: int, with_bias: bool) -> tuple[torch.Tensor, torch.Tensor]:
    dy, x = dy.contiguous(), x.contiguous()
    rows, n = _rows_n(dy, head_dim)
    k = x.shape[1]
    lib = _lib.load()
    dw = torch.empty(n, k, dtype=x.dtype, device=x.device)
    db = torch.empty(n if with_bias else 0, dtype=x.dtype, device=x.device)
    ws = torch.empty(lib.trifast_linear_dw_workspace_bytes(rows, k, n), dtype=torch.uint8, device=x.device)
    with torch.cuda.device(x.device):
        rc = lib.trifast_linear_dw(dw.data_ptr(), db.data_ptr() if with_bias else None, dy.data_ptr(), x.data_ptr(), rows, k, n, head_dim,
                                   _dtype_code(x), ws.data_ptr(), ws.numel(), torch.cuda.current_stream(x.device).cuda_stream)
    _lib.check(rc, "trifast_linear_dw")
    return dw, db


@_linear_weight_grad.register_fake
def _(dy, x, head_dim, with_bias):
    n = _rows_n(dy, head_dim)[1]
    return x.new_empty((n, x.shape[1])), x.new_empty((n if with_bias else 0,))


def linear_weight_grad(dy: torch.Tensor, x: torch.Tensor, head_dim: int = 0, with_bias: bool = False):
    """``dy^T x`` for ``dy [rows, n]``, ``x [rows, k]``: the weight gradient of a linear layer, with
    the long contraction over the rows split over the whole GPU (``trifast_linear_dw``).  With
    ``head_dim = d``, dy is ``[n / d, rows, d]`` (heads outermost).  ``with_bias``: also the bias
    gradient ``dy.sum(0)`` from the same pass; the result is then the pair (dw, db)."""
    dw, db = _linear_weight_grad(dy, x, head_dim, with_bias)
    return (dw, db) if with_bias else dw


class _Linear(torch.autograd.Function):
    """``linear(x, weight, bias)`` whose weight gradient comes from ``trifast_linear_dw``; the
    forward and the input gradient are the BLAS library's products, which run at memory speed
    for these shapes."""

    @staticmethod
    def forward(ctx, x, weight, bias):
        ctx.save_for_backward(x, weight)
        ctx.has_bias = bias is not None
        return torch.nn.functional.linear(x, weight, bias)

    @staticmethod
    def backward(ctx, dy):
        x, weight = ctx.saved_tensors
        dy2 = dy.reshape(-1, dy.shape[-1])
        dx = (dy2 @ weight).view(x.shape) if ctx.needs_input_grad[0] else None
        dw, db = linear_weight_grad(dy2, x.reshape(-1, x.shape[-1]), 0, True) if ctx.has_bias else (linear_weight_grad(dy2, x.reshape(-1, x.shape[-1])), None)
        return dx, dw, db


_DX_K = (32, 64, 128)
_DX_LAYERS = 6


@torch.library.custom_op("trifast::linear_input_grad", mutates_args=())
def _linear_input_grad(dys: Sequence[torch.Tensor], weights: Sequence[torch.Tensor], head_dims: Sequence[int]) -> torch.Tensor:
    dys = [dy.contiguous() for dy in dys]
    wts = [w.t().contiguous() for w in weights]  # [k, n_p]: a few tens of KiB each
    rows, k = _rows_n(dys[0], head_dims[0])[0], weights[0].shape[1]
    dx = torch.empty(rows, k, dtype=dys[0].dtype, device=dys[0].device)
    ptrs = lambda ts: (_lib.c_void_p * len(ts))(*[t.data_ptr() for t in ts])
    with torch.cuda.device(dx.device):
        rc = _lib.load().trifast_linear_dx(dx.data_ptr(), rows, k, len(dys), ptrs(dys), ptrs(wts), _lib.i64_array([w.shape[0] for w in weights]),
                                           _lib.i64_array(list(head_dims)), _dtype_code(dx), torch.cuda.current_stream(dx.device).cuda_stream)
    _lib.check(rc, "trifast_linear_dx")
    return dx


@_linear_input_grad.register_fake
def _(dys, weights, head_dims):
    return dys[0].new_empty((_rows_n(dys[0], head_dims[0])[0], weights[0].shape[1]))


def linear_input_grad(dys, weights, head_dims=None) -> torch.Tensor:
    """``sum_p dys[p] @ weights[p]`` for ``dys[p] [rows, n_p]``, ``weights[p] [n_p, k]``: the input
    gradient of several linear layers over one input, every ``dys[p]`` read once and the sum
    written once (``trifast_linear_dx``).  ``head_dims[p] = d``: ``dys[p]`` is ``[n_p / d, rows, d]``."""
    return _linear_input_grad(list(dys), list(weights), list(head_dims) if head_dims is not None else [0] * len(dys))


def _output_shape(rows: int, n: int, d: int) -> tuple[int, ...]:
    return (n // d, rows, d) if d else (rows, n)


@torch.library.custom_op("trifast::linear_outputs", mutates_args=())
def _linear_outputs(x: torch.Tensor, weights: Sequence[torch.Tensor], biases: Sequence[Optional[torch.Tensor]],
                    head_dims: Sequence[int]) -> list[torch.Tensor]:
    x = x.contiguous()
    rows, k = x.shape
    ws = [w.contiguous() for w in weights]
    bs = [None if b is None else b.contiguous() for b in biases]
    ys = [torch.empty(_output_shape(rows, w.shape[0], d), dtype=x.dtype, device=x.device) for w, d in zip(ws, head_dims)]
    ptrs = lambda ts: (_lib.c_void_p * len(ts))(*[None if t is None else t.data_ptr() for t in ts])
    with torch.cuda.device(x.device):
        rc = _lib.load().trifast_linear_fwd(x.data_ptr(), rows, k, len(ws), ptrs(ws), ptrs(bs), ptrs(ys), _lib.i64_array([w.shape[0] for w in ws]),
                                            _lib.i64_array(list(head_dims)), _dtype_code(x), torch.cuda.current_stream(x.device).cuda_stream)
    _lib.check(rc, "trifast_linear_fwd")
    return ys


@_linear_outputs.register_fake
def _(x, weights, biases, head_dims):
    return [x.new_empty(_output_shape(x.shape[0], w.shape[0], d)) for w, d in zip(weights, head_dims)]


def linear_outputs(x: torch.Tensor, weights, biases, head_dims=None) -> list[torch.Tensor]:
    """``[x @ w.T + b for w, b in zip(weights, biases)]`` for ``x [rows, k]`` in one pass that reads
    x once (``trifast_linear_fwd``); a bias may be None.  ``head_dims[p] = d``: output p comes
    heads-outermost, ``[n_p / d, rows, d]``."""
    return _linear_outputs(x, list(weights), list(biases), list(head_dims) if head_dims is not None else [0] * len(weights))


class _Project(torch.autograd.Function):
    """Several linear layers over one input.  Forward: one pass over x for all layers
    (``trifast_linear_fwd``).  Backward: one pass for the input gradient of all layers
    (``trifast_linear_dx``), this library's kernel for each weight gradient
    (``trifast_linear_dw``).  Layers with a head dim give their output heads-outermost,
    ``[n / d, *x.shape[:-1], d]``.  For 256 input channels the forward and the input gradient
    are the BLAS library's products (and every output is plain)."""

    @staticmethod
    def forward(ctx, x, head_dims, *params):
        n_layers = len(head_dims)
        weights, biases = params[:n_layers], params[n_layers:]
        ctx.save_for_backward(x, *weights)
        ctx.has_bias = [b is not None for b in biases]
        ctx.head_dims = head_dims
        ctx.set_materialize_grads(False)  # an unused output gives None, not a tensor of zeros to multiply
        lead = x.shape[:-1]
        if x.shape[-1] in _DX_K:
            ys = linear_outputs(x.reshape(-1, x.shape[-1]), weights, biases, head_dims)
            return tuple(y.view(y.shape[0], *lead, d) if d else y.view(*lead, y.shape[1]) for y, d in zip(ys, head_dims))
        return tuple(torch.nn.functional.linear(x, w, b) for w, b in zip(weights, biases))

    @staticmethod
    def backward(ctx, *dys):
        x, *weights = ctx.saved_tensors
        x2 = x.reshape(-1, x.shape[-1])
        # two dims per layer ([rows, n], or [n / d, rows, d] for a heads-outermost layer); a layer
        # whose output took no part in the loss has no gradient to give
        flat = [None if dy is None else (dy.reshape(dy.shape[0], -1, d) if d else dy.reshape(-1, dy.shape[-1])) for dy, d in zip(dys, ctx.head_dims)]
        live = [(dy, w, d) for dy, w, d in zip(flat, weights, ctx.head_dims) if dy is not None]
        dx = None
        if ctx.needs_input_grad[0] and live:
            if x.shape[-1] in _DX_K:
                dx = linear_input_grad([t[0] for t in live], [t[1] for t in live], [t[2] for t in live]).view(x.shape)
            else:
                dx = sum(dy @ w for dy, w, _ in live).view(x.shape)
        dws, dbs = [], []
        for dy, d, has in zip(flat, ctx.head_dims, ctx.has_bias):
            if dy is None:
                dw, db = None, None
            elif has:
                dw, db = linear_weight_grad(dy, x2, d, True)
            else:
                dw, db = linear_weight_grad(dy, x2, d), None
            dws.append(dw)
            dbs.append(db)
        return (dx, None, *dws, *dbs)


def project(x: torch.Tensor, layers, head_dims=None) -> tuple[torch.Tensor, ...]:
    """``tuple(layer(x) for layer in layers)`` for up to 6 ``torch.nn.Linear`` layers over the
    same pair representation ``x [*, k]``: one pass over x, and a backward that reads every
    output gradient once for the input gradient and computes the weight gradients with this
    library's kernel (GPU, 16-bit, k in (32, 64, 128); k = 256: the weight gradients only);
    anything else is the layers themselves.

    ``head_dims[p] = d`` (a layer of ``h * d`` outputs) returns output p as
    ``[h, *x.shape[:-1], d]``, heads outermost, which is how the attention operator reads q, k, v
    fastest; the kernels write and read that layout directly (elsewhere it is a copy)."""
    layers = list(layers)
    head_dims = tuple(head_dims) if head_dims is not None else (0,) * len(layers)
    fused = 0 < len(layers) <= _DX_LAYERS and all(_dw_ready(x, m.weight) for m in layers)
    if not fused or x.shape[-1] not in _DX_K:
        ys = _Project.apply(x, (0,) * len(layers), *[m.weight for m in layers], *[m.bias for m in layers]) if fused else tuple(m(x) for m in layers)
        return tuple(y.unflatten(-1, (-1, d)).movedim(-2, 0).contiguous() if d else y for y, d in zip(ys, head_dims))
    return _Project.apply(x, head_dims, *[m.weight for m in layers], *[m.bias for m in layers])


def linear(x: torch.Tensor, layer: torch.nn.Linear) -> torch.Tensor:
    """``layer(x)`` for a linear layer over a pair representation ``x [*, k]``; on the GPU, for
    16-bit tensors with k in (32, 64, 128, 256), its weight gradient is computed by this
    library's kernel (the BLAS library runs that one product, a contraction over millions of
    rows into a tiny result, on one or two workgroups)."""
    if not _dw_ready(x, layer.weight):
        return layer(x)
    return _Linear.apply(x, layer.weight, layer.bias)


class TriangleAttention(torch.nn.Module):
    """Gated triangle self-attention around the starting node (``ending_node=False``) or the
    ending node of a pair representation ``x [*, n, n, c_in]``; ``mask [*, n, n]`` is True
    where a pair is masked out (the operator's polarity)."""

    def __init__(self, c_in: int, h: int, d: int, ending_node: bool = False):
        super().__init__()
        self.h, self.d, self.ending_node = h, d, ending_node
        self.q = torch.nn.Linear(c_in, h * d, bias=False)
        self.k = torch.nn.Linear(c_in, h * d, bias=False)
        self.v = torch.nn.Linear(c_in, h * d, bias=False)
        self.b = torch.nn.Linear(c_in, h, bias=False)
        self.g = torch.nn.Linear(c_in, h * d)
        self.out = torch.nn.Linear(h * d, c_in)

    def heads(self, t: torch.Tensor) -> torch.Tensor:
        """``[*, n, n, h*d] -> [*, h, n, n, d]`` as a view."""
        return t.unflatten(-1, (self.h, self.d)).movedim(-2, -4)

    def forward(self, x: torch.Tensor, mask: torch.Tensor) -> torch.Tensor:
        # q, k, v come heads-outermost, [h, *, n, n, d]: the operator's fastest input layout
        q, k, v, bias, g = project(x, (self.q, self.k, self.v, self.b, self.g), (self.d, self.d, self.d, 0, 0))
        attend = triangle_attention_ending_node if self.ending_node else triangle_attention
        o = attend(q.movedim(0, -4), k.movedim(0, -4), v.movedim(0, -4), bias.movedim(-1, -3), mask)
        return linear(gated_output(o, g), self.out)
