"""Callers either side of the operator: leading batch dims and the ending-node entry.

Both are thin host-side layers over the starting-node operator; they are checked
against the oracle (leading dims: one call per batch element) and against the
ending-node formula written out with einsum (AlphaFold 2 supplement, algorithm 14),
values and gradients, with the reference's tolerance rule (tests/utils.py:31-36).
"""

import math

import pytest
import torch

import trifast_amd
from oracle import triangle_oracle as orc

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _inputs(lead, h, n, d, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    q, k, v = (torch.randn(*lead, h, n, n, d, generator=g) for _ in range(3))
    b = torch.randn(*lead, h, n, n, generator=g)
    mask = torch.rand(*lead, n, n, generator=g) < 0.25
    do = torch.randn(*lead, h, n, n, d, generator=g)
    return [t.to(DEV).to(dtype) for t in (q, k, v, b)] + [mask.to(DEV), do.to(DEV).to(dtype)]


def ending_node_reference(q, k, v, b, mask):
    """a[i,j,k] = softmax_k(q[i,j].k[k,j]/sqrt(d) + b[k,i] + mask[k,j]*min); o[i,j] = sum_k a[i,j,k] v[k,j]."""
    d = q.shape[-1]
    s = torch.einsum("bhijd,bhkjd->bhijk", q, k) / math.sqrt(d)
    s = s + b.permute(0, 1, 3, 2)[:, :, :, None, :]  # [b,h,i,1,k] <- b[k,i]
    s = s + (mask.to(s.dtype) * torch.finfo(s.dtype).min).permute(0, 2, 1)[:, None, None, :, :]  # [b,1,1,j,k] <- mask[k,j]
    return torch.einsum("bhijk,bhkjd->bhijd", torch.softmax(s, dim=-1), v)


def _grads(fn, q, k, v, b, mask, do):
    q, k, v, b = (t.detach().clone().requires_grad_(True) for t in (q, k, v, b))
    o = fn(q, k, v, b, mask)
    o.backward(do)
    return o.detach(), q.grad, k.grad, v.grad, b.grad


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_ending_node_entry(dtype):
    q, k, v, b, mask, do = _inputs((2,), 2, 40, 32, dtype, seed=11)
    got = _grads(trifast_amd.triangle_attention_ending_node, q, k, v, b, mask, do)
    f32 = lambda t: t.float()
    ref = _grads(ending_node_reference, f32(q), f32(k), f32(v), f32(b), mask, f32(do))
    pt = _grads(ending_node_reference, q, k, v, b, mask, do)
    for name, x, p, r in zip(("o", "dq", "dk", "dv", "db"), got, pt, ref):
        assert x.shape == r.shape
        orc.compare_values(x, p, r, f"ending node {dtype} {name}", eps=orc.DTYPE_EPS[dtype])


@pytest.mark.parametrize("lead", [(), (2, 3)], ids=["no_batch", "two_batch_dims"])
def test_leading_batch_dims(lead):
    dtype = torch.bfloat16
    q, k, v, b, mask, do = _inputs(lead, 2, 33, 32, dtype, seed=5)
    got = _grads(trifast_amd.triangle_attention, q, k, v, b, mask, do)
    assert got[0].shape == q.shape and got[4].shape == b.shape
    # the same, one batch element at a time through the 5-D operator
    fold = lambda t, keep: t.reshape(-1, *t.shape[-keep:])
    fq, fk, fv, fb, fm, fdo = fold(q, 4), fold(k, 4), fold(v, 4), fold(b, 3), fold(mask, 2), fold(do, 4)
    for x in range(fq.shape[0]):
        one = _grads(trifast_amd.triangle_attention, fq[x : x + 1], fk[x : x + 1], fv[x : x + 1], fb[x : x + 1], fm[x : x + 1], fdo[x : x + 1])
        for name, a, c in zip(("o", "dq", "dk", "dv", "db"), got, one):
            assert torch.equal(fold(a, c.dim() - 1)[x : x + 1], c), f"batch element {x}: {name} differs"


def test_leading_dims_must_agree():
    q, k, v, b, mask, _ = _inputs((2, 3), 1, 16, 16, torch.float32, seed=1)
    with pytest.raises(ValueError, match="leading batch dims"):
        trifast_amd.triangle_attention(q, k, v, b[0], mask)


class PairAttentionBlock(torch.nn.Module):
    """Projections of a pair representation x [b, n, n, c] into q, k, v, bias, then the
    operator: the module of reference tests/unit/test_trifast.py:152-169, with the heads
    moved in front of the pair dims as the operator expects ([b, h, n, n, d])."""

    def __init__(self, h: int, d: int, attention):
        super().__init__()
        self.h, self.attention = h, attention
        self.q = torch.nn.Linear(d, h * d)
        self.k = torch.nn.Linear(d, h * d)
        self.v = torch.nn.Linear(d, h * d)
        self.b = torch.nn.Linear(d, h)

    def forward(self, x, mask):
        heads = lambda t: t.unflatten(-1, (self.h, -1)).permute(0, 3, 1, 2, 4)  # views: read in place
        return self.attention(heads(self.q(x)), heads(self.k(x)), heads(self.v(x)), self.b(x).permute(0, 3, 1, 2), mask)


@pytest.mark.parametrize(
    "n,h,d,do_mask,bs,dtype",
    [(16, 1, 16, False, 1, torch.float16), (32, 1, 32, False, 1, torch.bfloat16), (64, 1, 64, False, 4, torch.float32), (48, 4, 32, True, 2, torch.bfloat16)],
)
def test_weight_updates(n, h, d, do_mask, bs, dtype):
    """Reference tests/unit/test_trifast.py:172-210: every parameter of a module around the
    operator moves under Adam."""
    torch.manual_seed(0)
    x = torch.randn(bs, n, n, d, device=DEV, dtype=dtype, requires_grad=True)
    model = PairAttentionBlock(h, d, trifast_amd.triangle_attention).to(DEV, dtype)
    opt = torch.optim.Adam(model.parameters(), lr=1e-3)
    mask = torch.randint(0, 2, (bs, n, n), device=DEV, dtype=torch.bool) if do_mask else torch.zeros(bs, n, n, device=DEV, dtype=torch.bool)
    before = {name: p.detach().clone() for name, p in model.named_parameters()}
    for step in range(5):
        out = model(x, mask)
        label = torch.randn_like(out) * 4
        opt.zero_grad()
        torch.nn.functional.mse_loss(out, label).backward()
        if step == 0:
            # (later steps are Adam's business: in pure fp16 its epsilon underflows)
            assert torch.isfinite(out).all()
            for name, p in model.named_parameters():
                assert torch.isfinite(p.grad).all() and p.grad.abs().max() > 0, f"gradient of {name}"
        opt.step()
    for name, p in model.named_parameters():
        assert not torch.all(before[name] == p), f"parameter {name} did not update"


def test_parameter_gradients_match_the_oracle():
    """The same module around the oracle gives the same parameter and input gradients (fp32)."""
    torch.manual_seed(1)
    n, h, d, bs = 24, 2, 32, 2
    x = torch.randn(bs, n, n, d, device=DEV)
    mask = torch.rand(bs, n, n, device=DEV) < 0.2
    label = torch.randn(bs, h, n, n, d, device=DEV)
    ours = PairAttentionBlock(h, d, trifast_amd.triangle_attention).to(DEV)
    theirs = PairAttentionBlock(h, d, orc.attention_reference).to(DEV)
    theirs.load_state_dict(ours.state_dict())
    grads = []
    for model in (ours, theirs):
        xi = x.clone().requires_grad_(True)
        torch.nn.functional.mse_loss(model(xi, mask), label).backward()
        grads.append({"x": xi.grad, **{name: p.grad for name, p in model.named_parameters()}})
    for name in grads[0]:
        a, r = grads[0][name], grads[1][name]
        assert (a - r).abs().max().item() <= 2e-5 * max(r.abs().max().item(), 1e-6) + 1e-7, f"{name}: {(a - r).abs().max().item():.3e}"


def test_device_clock_export():
    """The benchmark's helper reports a plausible shader clock and rejects a bad device."""
    from trifast_amd import _lib

    lib = _lib.load()
    mhz = lib.trifast_device_clock_mhz(0)
    assert 500 <= mhz <= 5000, mhz
    assert lib.trifast_device_clock_mhz(10_000) < 0
    assert "clock" in _lib.last_error()


def test_gradients_take_the_layout_of_transposed_leaves():
    """Leaves that are pair-transposed views (the ending-node call pattern) receive
    gradients written in their own layout by the kernels: autograd stores them as they
    are instead of re-laying them out with a copy each (reference backward: gradients
    follow the saved, possibly strided inputs, src/trifast/torch.py:85-104)."""
    dtype = torch.float16
    q, k, v, b, mask, do = _inputs((2,), 2, 72, 64, dtype, seed=21)
    tq, tk, tv, tdo = (t.transpose(2, 3) for t in (q, k, v, do))
    tb, tm = b.transpose(-1, -2), mask.transpose(-1, -2)
    leaves = [t.detach().requires_grad_(True) for t in (tq, tk, tv, tb)]
    assert not any(t.is_contiguous() for t in leaves)
    from trifast_amd import torch as tt

    o, lse = tt._triangle_attention(*leaves, tm)
    raw = tt.triangle_attention_bwd(tdo, *(t.detach() for t in leaves), o.detach(), lse, tm)
    for g, leaf in zip(raw[:4], leaves):
        assert g.stride() == leaf.stride() and g.shape == leaf.shape
    o.backward(tdo)
    for g, leaf, r in zip((t.grad for t in leaves), leaves, raw[:4]):
        assert g.stride() == leaf.stride()
        assert torch.equal(g, r)
    # values: against the oracle on the same views
    f32 = lambda t: t.float()
    ref = orc.forward_backward(f32(tq), f32(tk), f32(tv), f32(tb), tm, f32(tdo))
    pt = orc.forward_backward(tq, tk, tv, tb, tm, tdo)
    got = (o.detach(), *(t.grad for t in leaves))
    for name, x, p, r in zip(("o", "dq", "dk", "dv", "db"), got, pt, ref):
        orc.compare_values(x, p, r, f"strided gradients {name}", eps=orc.DTYPE_EPS[dtype])
    # odd n: db rows are not 16-byte multiples, the strided scalar path is used
    q, k, v, b, mask, do = _inputs((1,), 2, 37, 32, torch.bfloat16, seed=22)
    tb = b.transpose(-1, -2)
    got = _grads(trifast_amd.triangle_attention, q, k, v, tb, mask, do)
    want = _grads(trifast_amd.triangle_attention, q, k, v, tb.contiguous(), mask, do)
    assert torch.equal(got[4], want[4])


def test_broadcast_upstream_gradient_is_not_materialised():
    """``o.sum().backward()`` hands the backward an all-ones tensor with every stride 0
    (the reference's own test and tuning protocol, tests/unit/test_trifast.py:51): it is
    read as one row through zero strides, so no tensor of q's size is allocated for it."""
    n, h, d = 256, 2, 32
    dtype = torch.bfloat16
    q, k, v, b, mask, _ = _inputs((1,), h, n, d, dtype, seed=23)
    from trifast_amd import torch as tt

    o, lse = tt._triangle_attention(q, k, v, b, mask)
    ones = torch.ones((), device=DEV, dtype=dtype).expand(q.shape)
    assert ones.stride() == (0, 0, 0, 0, 0)
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats()
    base = torch.cuda.memory_allocated()
    got = tt.triangle_attention_bwd(ones, q, k, v, b, o, lse, mask)
    torch.cuda.synchronize()
    extra = torch.cuda.max_memory_allocated() - base
    qbytes = q.numel() * q.element_size()
    ws = _ws_bytes(1, h, n, d)
    # three gradients of q's size, db, dmask, the workspace -- and not a fourth q-sized tensor
    assert extra < 3 * qbytes + ws + qbytes // 2, (extra, qbytes, ws)
    want = tt.triangle_attention_bwd(ones.contiguous(), q, k, v, b, o, lse, mask)
    for x, y in zip(got[:4], want[:4]):
        assert torch.equal(x, y)
    # one [d] row expanded over b, h, i, j is the other all-zero-stride case
    row = torch.randn(d, device=DEV).to(dtype).expand(q.shape)
    got = tt.triangle_attention_bwd(row, q, k, v, b, o, lse, mask)
    want = tt.triangle_attention_bwd(row.contiguous(), q, k, v, b, o, lse, mask)
    for x, y in zip(got[:4], want[:4]):
        assert torch.equal(x, y)


def _ws_bytes(b, h, n, d):
    from trifast_amd import _lib

    return _lib.load().trifast_bwd_workspace_bytes(b, h, n, d, _lib.BF16)


@pytest.mark.parametrize("shape", [(0, 2, 16, 32), (2, 0, 16, 32), (1, 2, 0, 32)], ids=["no_batch", "no_heads", "no_tokens"])
def test_empty_inputs_give_empty_outputs(shape):
    """An empty batch (a data loader's last, empty shard) passes through: empty output, empty
    gradients, no launch."""
    b, h, n, d = shape
    q, k, v = (torch.zeros(b, h, n, n, d, device=DEV, dtype=torch.bfloat16, requires_grad=True) for _ in range(3))
    bias = torch.zeros(b, h, n, n, device=DEV, dtype=torch.bfloat16, requires_grad=True)
    mask = torch.zeros(b, n, n, device=DEV, dtype=torch.bool)
    o = trifast_amd.triangle_attention(q, k, v, bias, mask)
    assert o.shape == q.shape and o.dtype == q.dtype
    o.sum().backward()
    for t in (q, k, v, bias):
        assert t.grad is not None and t.grad.shape == t.shape
