"""PyTorch operator boundary of the MI355X triangle attention.

Mirrors the public surface of reference src/trifast/torch.py: two ``torch.library``
operators, ``trifast::triangle_attention`` (-> o, lse; reference :17-65) and
``trifast::triangle_attention_backward`` (-> dq, dk, dv, db, dmask; reference
:68-182), glued by ``register_autograd`` (reference :185-217), and the
``triangle_attention`` wrapper that drops lse (reference :220-228).  The device
work is done by hand-written HIP kernels behind the C ABI of
``libtrifast_hip.so``; PyTorch only owns the memory and the stream.
"""

from __future__ import annotations

import torch

from trifast_amd import _lib, tuner

_DTYPE_CODE = {torch.float32: _lib.F32, torch.bfloat16: _lib.BF16, torch.float16: _lib.F16}


def _dtype_code(t: torch.Tensor) -> int:
    try:
        return _DTYPE_CODE[t.dtype]
    except KeyError:
        raise TypeError(f"triangle_attention supports float32, bfloat16 and float16, got {t.dtype}") from None


def _check_inputs(q, k, v, b, mask) -> tuple[int, int, int, int]:
    if q.dim() != 5:
        raise ValueError(f"q must be [b, h, n, n, d], got shape {tuple(q.shape)}")
    bs, h, n, n2, d = q.shape
    if n != n2:
        raise ValueError(f"q must be square in its pair dims, got shape {tuple(q.shape)}")
    if k.shape != q.shape or v.shape != q.shape:
        raise ValueError("q, k, v must have the same shape")
    if tuple(b.shape) != (bs, h, n, n):
        raise ValueError(f"bias must be [b, h, n, n] = {(bs, h, n, n)}, got {tuple(b.shape)}")
    if tuple(mask.shape) != (bs, n, n):
        raise ValueError(f"mask must be [b, n, n] = {(bs, n, n)}, got {tuple(mask.shape)}")
    if mask.dtype != torch.bool:
        raise TypeError(f"mask must be bool, got {mask.dtype}")
    if not (k.dtype == q.dtype and v.dtype == q.dtype and b.dtype == q.dtype):
        raise TypeError("q, k, v and bias must share one dtype")
    for name, t in (("q", q), ("k", k), ("v", v), ("bias", b), ("mask", mask)):
        if not t.is_cuda:
            raise RuntimeError(f"{name} is on {t.device}: triangle_attention runs on the GPU only")
        if t.device != q.device:
            raise RuntimeError("all inputs must be on the same device")
    return bs, h, n, d


def _strides(t: torch.Tensor) -> list[int]:
    # the stride of a size-1 dim is never used for addressing; report 0
    return [0 if sz == 1 else st for sz, st in zip(t.shape, t.stride())]


def _vector_ready(t: torch.Tensor) -> torch.Tensor:
    """q-like tensors are read with 16-byte vector loads along d: the last stride
    must be 1, the base 16-byte aligned and the other strides multiples of the
    vector width.  Transposed (i<->j) views qualify and are read in place; anything
    else is copied, as the reference forward copies every non-contiguous input
    (src/trifast/torch.py:30-34)."""
    vec = 16 // t.element_size()
    st = _strides(t)
    if st[-1] == 1 and t.data_ptr() % 16 == 0 and all(s % vec == 0 for s in st[:-1]) and _j_stride_ok(t, st):
        return t
    return t.contiguous()


def _j_stride_ok(t: torch.Tensor, st: list[int]) -> bool:
    """The kernels address the rows of a tile through 32-bit offsets from a per-tile base:
    the stride between consecutive j, in bytes, must lie in [0, 2^24) (the library returns
    TRIFAST_EUNSUPPORTED otherwise)."""
    return t.dim() != 5 or 0 <= st[3] * t.element_size() < (1 << 24)


def _broadcast_rows(t: torch.Tensor) -> torch.Tensor:
    """An upstream gradient that is one value or one [d] row expanded over b, h, i, j
    (``o.sum().backward()`` gives such a tensor, all strides 0) becomes a single
    16-byte-aligned row read through zero strides: nothing of q's size is
    materialised."""
    st = _strides(t)
    if any(st[:-1]) or t.dim() != 5:
        return t
    row = t[(0,) * 4].contiguous()  # [d] elements
    return row.expand(t.shape)


def _grad_like(t: torch.Tensor) -> torch.Tensor:
    """Empty gradient buffer for input ``t``: laid out like ``t`` when ``t`` is dense
    and the kernels can write that layout (d contiguous, 16-byte rows), so that a
    leaf that is a transposed view takes its gradient without a re-layout copy;
    contiguous otherwise."""
    vec = 16 // t.element_size()
    st = _strides(t)
    if t.dim() == 5 and st[-1] == 1 and all(s % vec == 0 for s in st[:-1]) and _j_stride_ok(t, st):
        out = torch.empty_like(t)  # preserves the strides of a dense tensor
        if out.stride() == t.stride():
            return out
    elif t.dim() == 4:
        out = torch.empty_like(t)
        if out.stride() == t.stride():
            return out
    return torch.empty(t.shape, dtype=t.dtype, device=t.device)


def _workspace(nbytes: int, device) -> torch.Tensor:
    return torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=device)


# What a call needs besides the pointers, per (operator, shapes and strides of its tensors):
# the stride arrays the C ABI takes and the workspace size.  At small sizes a step is bound
# by the host (n = 256: 0.13 ms of kernels), and marshalling ten stride arrays and asking
# the library for sizes on every call is a good part of that.
_PLANS: dict = {}
_MAX_PLANS = 256


def _plan(kind: str, tensors, bs: int, h: int, n: int, d: int, code: int):
    key = (kind, code, tuple((t.shape, t.stride()) for t in tensors))
    plan = _PLANS.get(key)
    if plan is None:
        lib = _lib.load()
        size = lib.trifast_fwd_workspace_bytes if kind == "fwd" else lib.trifast_bwd_workspace_bytes
        plan = ([_lib.i64_array(_strides(t)) for t in tensors], size(bs, h, n, d, code))
        if len(_PLANS) >= _MAX_PLANS:
            _PLANS.clear()
        _PLANS[key] = plan
    return plan


def _ptr(t):
    return t.data_ptr()


@torch.library.custom_op("trifast::triangle_attention", mutates_args=())
def _triangle_attention(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    b: torch.Tensor,
    mask: torch.Tensor,
) -> tuple[torch.Tensor, torch.Tensor]:
    lib = _lib.load()
    bs, h, n, d = _check_inputs(q, k, v, b, mask)
    code = _dtype_code(q)
    o = torch.empty((bs, h, n, n, d), dtype=q.dtype, device=q.device)
    lse = torch.empty((bs, h, n, n), dtype=torch.float32, device=q.device)
    if o.numel() == 0 and d > 0:  # an empty batch (or no heads, or no tokens): nothing to launch
        return o, lse
    # bias and mask are re-tiled by the library's pre-passes, so any strides go
    q, k, v = _vector_ready(q), _vector_ready(k), _vector_ready(v)
    mask_u8 = mask.view(torch.uint8)

    with torch.cuda.device(q.device):
        strides, ws_bytes = _plan("fwd", (q, k, v, b, mask_u8), bs, h, n, d, code)
        ws = _workspace(ws_bytes, q.device)
        stream = torch.cuda.current_stream(q.device).cuda_stream

        def launch(tile: int) -> None:
            rc = lib.trifast_fwd(
                _ptr(o), _ptr(lse), _ptr(q), _ptr(k), _ptr(v), _ptr(b), _ptr(mask_u8),
                bs, h, n, d, code, *strides,
                tile, _ptr(ws), ws.numel(), stream,
            )
            _lib.check(rc, "trifast_fwd")

        tile = tuner.pick(_lib.KERNEL_FWD, n, h, d, q.dtype, launch)
        launch(tile)
    return o, lse


@_triangle_attention.register_fake
def _(q, k, v, b, mask):
    bs, h, n, _, d = q.shape
    o = q.new_empty((bs, h, n, n, d))
    lse = q.new_empty((bs, h, n, n), dtype=torch.float32)
    return o, lse


@torch.library.custom_op("trifast::triangle_attention_backward", mutates_args=())
def triangle_attention_bwd(
    do: torch.Tensor,
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    b: torch.Tensor,
    o: torch.Tensor,
    l: torch.Tensor,
    mask: torch.Tensor,
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    lib = _lib.load()
    bs, h, n, d = _check_inputs(q, k, v, b, mask)
    code = _dtype_code(q)
    if q.numel() == 0 and d > 0:  # an empty batch: empty gradients
        return _grad_like(q), _grad_like(k), _grad_like(v), _grad_like(b), torch.zeros_like(mask)
    if do.dtype != q.dtype:
        do = do.to(q.dtype)
    # the upstream gradient is often an expanded (stride-0) tensor, e.g. from
    # o.sum().backward(): it is read through its zero strides
    do = _vector_ready(_broadcast_rows(do))
    # bias and mask are re-tiled by the library's pre-passes, so any strides go
    q_in, k_in, v_in = q, k, v
    q, k, v = _vector_ready(q), _vector_ready(k), _vector_ready(v)
    o = o.contiguous()
    l = l.contiguous()
    mask_u8 = mask.view(torch.uint8)

    # gradients in the layout of the inputs they belong to (the layout of the
    # caller's tensors, not of a vector-ready copy)
    dq, dk, dv, db = _grad_like(q_in), _grad_like(k_in), _grad_like(v_in), _grad_like(b)
    with torch.cuda.device(q.device):
        strides, ws_bytes = _plan("bwd", (do, q, k, v, b, mask_u8, dq, dk, dv, db), bs, h, n, d, code)
        ws = _workspace(ws_bytes, q.device)
        stream = torch.cuda.current_stream(q.device).cuda_stream

        def launch_one(kernel: int, tile: int) -> None:
            rc = lib.trifast_bwd_one(
                kernel, _ptr(dq), _ptr(dk), _ptr(dv), _ptr(db),
                _ptr(do), _ptr(q), _ptr(k), _ptr(v), _ptr(b), _ptr(mask_u8), _ptr(o), _ptr(l),
                bs, h, n, d, code, *strides, tile, _ptr(ws), ws.numel(), stream,
            )
            _lib.check(rc, "trifast_bwd_one")

        # fixed launch order; _bwd_q also produces delta for the other two
        # (reference src/trifast/torch.py:110).  When a later kernel has to be timed
        # but _bwd_q's tile comes from the cache, _bwd_q runs once first so that the
        # timed kernels read a valid workspace.
        tiles = []
        primed = False
        for kernel in (_lib.KERNEL_BWD_Q, _lib.KERNEL_BWD_KV, _lib.KERNEL_BWD_B):
            def timed(t, kern=kernel):
                nonlocal primed
                if kern != _lib.KERNEL_BWD_Q and not primed:
                    launch_one(_lib.KERNEL_BWD_Q, tiles[0])
                primed = True
                launch_one(kern, t)

            # a dk/dv tile that also produces dq saves the dq kernel's launch: the other
            # dk/dv tiles are charged with it
            extra = None
            if kernel == _lib.KERNEL_BWD_KV:
                dq_ms: list[float] = []

                def extra(t):
                    if lib.trifast_bwd_kv_tile_writes_dq(t):
                        return 0.0
                    if not dq_ms:
                        dq_ms.append(tuner._time_launch(lambda tile: launch_one(_lib.KERNEL_BWD_Q, tile), tiles[0]))
                    return dq_ms[0]

            tiles.append(tuner.pick(kernel, n, h, d, q.dtype, timed, extra))
        rc = lib.trifast_bwd(
            _ptr(dq), _ptr(dk), _ptr(dv), _ptr(db),
            _ptr(do), _ptr(q), _ptr(k), _ptr(v), _ptr(b), _ptr(mask_u8), _ptr(o), _ptr(l),
            bs, h, n, d, code, *strides,
            (_lib.c_int * 3)(*tiles), _ptr(ws), ws.numel(), stream,
        )
        _lib.check(rc, "trifast_bwd")
    # the mask takes no gradient; autograd still wants a tensor in this slot
    # (reference src/trifast/torch.py:102)
    dmask = torch.zeros_like(mask)
    return dq, dk, dv, db, dmask


@triangle_attention_bwd.register_fake
def _(do, q, k, v, b, o, l, mask):
    return (_grad_like(q), _grad_like(k), _grad_like(v), _grad_like(b), torch.zeros_like(mask))


def backwards(ctx, *grad):
    # reference src/trifast/torch.py:185-207
    do = grad[0]
    q, k, v, b, mask, o, l = ctx.saved_tensors
    if do is None:  # only lse was used downstream: nothing flows back through o
        do = torch.zeros_like(o)
    dq, dk, dv, db, _ = triangle_attention_bwd(do, q, k, v, b, o, l, mask)
    return dq, dk, dv, db, None


def setup_context(ctx, inputs, output) -> None:
    # reference src/trifast/torch.py:210-214
    q, k, v, b, mask, *_ = inputs
    o, l = output
    ctx.save_for_backward(q, k, v, b, mask, o, l)
    # lse takes no gradient: without this autograd fills a zero tensor of its size for every backward
    ctx.set_materialize_grads(False)


_triangle_attention.register_autograd(backwards, setup_context=setup_context)


class _EagerTriangleAttention(torch.autograd.Function):
    """The two operators glued by a plain autograd function: what ``triangle_attention``
    runs in ordinary eager mode on plain tensors.  Same kernels, same saved tensors, same
    gradients as the registered operators; it only skips the dispatcher passes of a Python
    custom operator (forward, autograd wrapper and backward operator: about 50 us of host time
    per step, which at n = 256 is a third of what the kernels take)."""

    @staticmethod
    def forward(ctx, q, k, v, b, mask):
        o, l = _triangle_attention._init_fn(q, k, v, b, mask)
        ctx.save_for_backward(q, k, v, b, mask, o, l)
        ctx.set_materialize_grads(False)
        return o

    @staticmethod
    def backward(ctx, do):
        q, k, v, b, mask, o, l = ctx.saved_tensors
        if do is None:
            return None, None, None, None, None
        dq, dk, dv, db, _ = triangle_attention_bwd._init_fn(do, q, k, v, b, o, l, mask)
        return dq, dk, dv, db, None


def _plain_eager(*tensors) -> bool:
    """Ordinary eager execution on plain tensors: no compilation or tracing, no function
    transforms, no autocast, no tensor subclasses or dispatch modes; everything else goes
    through the registered operators."""
    if torch.compiler.is_compiling() or torch.is_autocast_enabled() or torch._C._are_functorch_transforms_active():
        return False
    if torch._C._dispatch_tls_local_include_set().has(torch._C.DispatchKey.Python) or torch._C._len_torch_dispatch_stack() > 0:
        return False
    return all(type(t) is torch.Tensor for t in tensors)


def triangle_attention(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    b: torch.Tensor,
    mask: torch.Tensor,
) -> torch.Tensor:
    """Fused triangle self-attention (starting node).

    q, k, v: [b, h, n, n, d]; b (bias): [b, h, n, n]; mask: [b, n, n] bool with
    True = key masked out.  Returns o: [b, h, n, n, d].  Reference
    src/trifast/torch.py:220-228.

    Beyond the reference (its own TODO, src/trifast/torch.py:29,84): any number of
    leading batch dims, q [*batch, h, n, n, d] with bias [*batch, h, n, n] and mask
    [*batch, n, n], including none at all; they are folded into one batch dim (views
    where the layout allows it) and restored on the output.
    """
    if q.dim() == 5:
        if _plain_eager(q, k, v, b, mask):
            return _EagerTriangleAttention.apply(q, k, v, b, mask)
        o, _ = _triangle_attention(q, k, v, b, mask)
        return o
    if q.dim() < 4:
        raise ValueError(f"q must be [*batch, h, n, n, d], got shape {tuple(q.shape)}")
    lead = q.shape[:-4]
    if b.shape[:-3] != lead or mask.shape[:-2] != lead or k.shape != q.shape or v.shape != q.shape:
        raise ValueError(
            f"leading batch dims must agree: q {tuple(q.shape)}, k {tuple(k.shape)}, v {tuple(v.shape)}, "
            f"bias {tuple(b.shape)}, mask {tuple(mask.shape)}"
        )
    fold = lambda t, keep: t.reshape(-1, *t.shape[-keep:])
    o, _ = _triangle_attention(fold(q, 4), fold(k, 4), fold(v, 4), fold(b, 3), fold(mask, 2))
    return o.reshape(*lead, *o.shape[1:])


def triangle_attention_ending_node(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    b: torch.Tensor,
    mask: torch.Tensor,
) -> torch.Tensor:
    """Triangle self-attention around the ending node, on tensors in the ordinary
    (untransposed) pair layout:

        a[i, j, k] = softmax_k(q[i, j] . k[k, j] / sqrt(d) + b[k, i] + mask[k, j] * finfo.min)
        o[i, j]    = sum_k a[i, j, k] v[k, j]

    with q, k, v: [*batch, h, n, n, d] indexed [.., i, j, :], b: [*batch, h, n, n],
    mask: [*batch, n, n] (True = masked out).  This is the starting-node operator on
    the pair-transposed problem; the transposes are views (q, k, v are read in place
    through their strides, bias and mask are re-tiled by the pre-passes anyway), so
    nothing is copied.  The result is a transposed view of a contiguous tensor.
    The reference has no such entry: its callers transpose and copy by hand.
    """
    t = lambda x: x.transpose(-3, -2)
    return t(triangle_attention(t(q), t(k), t(v), b.transpose(-1, -2), mask.transpose(-1, -2)))
