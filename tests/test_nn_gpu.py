"""The gated block around the operator (trifast_amd.nn) on the GPU.

The gate kernel is checked against its formula in fp64 with the rounding bound of one
result in the tensors' dtype; the block against the same block built from the oracle and
plain PyTorch ops with the same weights (values, input and parameter gradients).
"""

import pytest
import torch

import trifast_amd
from oracle import triangle_oracle as orc
from trifast_amd import nn

pytestmark = pytest.mark.gpu
DEV = "cuda"


def gate_reference(o, g):
    """y[*, i, j, h*d] = o[*, h, i, j, d] * sigmoid(g)."""
    return o.movedim(-4, -2).flatten(-2) * torch.sigmoid(g)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16], ids=["f32", "bf16", "f16"])
@pytest.mark.parametrize("lead,h,n,d", [((2,), 4, 33, 32), ((), 1, 7, 16), ((2, 2), 3, 20, 64), ((1,), 2, 130, 128)])
def test_gate_forward_and_backward(dtype, lead, h, n, d):
    gen = torch.Generator().manual_seed(n * 1000 + d)
    o = torch.randn(*lead, h, n, n, d, generator=gen).to(DEV, dtype)
    g = (3 * torch.randn(*lead, n, n, h * d, generator=gen)).to(DEV, dtype)
    dy = torch.randn(*lead, n, n, h * d, generator=gen).to(DEV, dtype)
    oo, gg = o.clone().requires_grad_(True), g.clone().requires_grad_(True)
    y = nn.gated_output(oo, gg)
    assert y.shape == g.shape and y.dtype == dtype
    y.backward(dy)
    ro, rg = o.double().requires_grad_(True), g.double().requires_grad_(True)
    ry = gate_reference(ro, rg)
    ry.backward(dy.double())
    # the kernel computes in fp32 (hardware exp2 of x log2 e: a few fp32 ulps) and rounds once to the dtype
    for name, got, want in (("y", y.detach(), ry.detach()), ("do", oo.grad, ro.grad), ("dg", gg.grad, rg.grad)):
        assert got.shape == want.shape, name
        err = (got.double() - want).abs()
        bound = 0.5 * torch.finfo(dtype).eps * want.abs() + 16 * 2.0**-23 * want.abs() + torch.finfo(dtype).smallest_normal
        assert bool((err <= bound).all()), f"{name} {dtype}: max excess {(err - bound).max().item():.3e}"


def test_gate_of_a_strided_operand_is_made_dense_first():
    o = torch.randn(2, 2, 16, 16, 32, device=DEV, dtype=torch.bfloat16).transpose(2, 3)
    g = torch.randn(2, 16, 16, 64, device=DEV, dtype=torch.bfloat16)
    assert torch.equal(nn.gated_output(o, g), nn.gated_output(o.contiguous(), g))


def test_empty_gate():
    o = torch.zeros(0, 2, 8, 8, 16, device=DEV)
    assert nn.gated_output(o, torch.zeros(0, 8, 8, 32, device=DEV)).shape == (0, 8, 8, 32)


class ReferenceBlock(torch.nn.Module):
    """trifast_amd.nn.TriangleAttention from the oracle and plain PyTorch ops, with copies
    where the product uses views; ending node by explicit transposition of the pair dims."""

    def __init__(self, c_in, h, d, ending_node):
        super().__init__()
        self.h, self.d, self.ending_node = h, d, ending_node
        self.q = torch.nn.Linear(c_in, h * d, bias=False)
        self.k = torch.nn.Linear(c_in, h * d, bias=False)
        self.v = torch.nn.Linear(c_in, h * d, bias=False)
        self.b = torch.nn.Linear(c_in, h, bias=False)
        self.g = torch.nn.Linear(c_in, h * d)
        self.out = torch.nn.Linear(h * d, c_in)

    def forward(self, x, mask):
        g = self.g(x)
        if self.ending_node:
            x, mask = x.transpose(-2, -3).contiguous(), mask.transpose(-1, -2).contiguous()
        heads = lambda t: t.unflatten(-1, (self.h, self.d)).permute(0, 3, 1, 2, 4).contiguous()
        o = orc.attention_reference(heads(self.q(x)), heads(self.k(x)), heads(self.v(x)), self.b(x).permute(0, 3, 1, 2).contiguous(), mask)
        o = o.permute(0, 2, 3, 1, 4).flatten(-2)
        if self.ending_node:
            o = o.transpose(-2, -3)
        return self.out(o * torch.sigmoid(g))


@pytest.mark.parametrize("ending_node", [False, True], ids=["starting", "ending"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_block_matches_the_reference_block(ending_node, dtype):
    torch.manual_seed(3)
    bs, n, c, h, d = 2, 40, 48, 2, 32
    x = torch.randn(bs, n, n, c, device=DEV)
    mask = torch.rand(bs, n, n, device=DEV) < 0.2
    label = torch.randn(bs, n, n, c, device=DEV)
    ours = nn.TriangleAttention(c, h, d, ending_node).to(DEV)
    ref32 = ReferenceBlock(c, h, d, ending_node).to(DEV)
    ref32.load_state_dict(ours.state_dict())

    def run(model, dt):
        model = model.to(dt)
        xi = x.to(dt).detach().requires_grad_(True)
        out = model(xi, mask)
        torch.nn.functional.mse_loss(out.float(), label).backward()
        res = {"out": out.detach().float(), "x": xi.grad.float(), **{k: p.grad.float() for k, p in model.named_parameters()}}
        model.zero_grad()
        return res

    want = run(ref32, torch.float32)
    got = run(ours, dtype)
    if dtype == torch.float32:
        for name in want:
            a, r = got[name], want[name]
            assert (a - r).abs().max().item() <= 3e-5 * max(r.abs().max().item(), 1e-6) + 1e-7, f"{name}: {(a - r).abs().max().item():.3e}"
        return
    # low precision: our block may be at most 3x as far from fp32 as the same reference block run in that dtype
    refl = ReferenceBlock(c, h, d, ending_node).to(DEV)
    refl.load_state_dict({k: v.float() for k, v in ours.state_dict().items()})
    pt = run(refl, dtype)
    for name in want:
        e_ours = (got[name] - want[name]).abs().max().item()
        e_pt = (pt[name] - want[name]).abs().max().item()
        assert e_ours <= 3 * e_pt + 1e-6, f"{name}: ours {e_ours:.3e} vs PyTorch in {dtype} {e_pt:.3e}"


def test_block_trains():
    """Reference tests/unit/test_trifast.py:172-210 on the gated block: every parameter moves."""
    torch.manual_seed(0)
    model = nn.TriangleAttention(32, 4, 32).to(DEV, torch.bfloat16)
    x = torch.randn(1, 48, 48, 32, device=DEV, dtype=torch.bfloat16)
    mask = torch.rand(1, 48, 48, device=DEV) < 0.3
    opt = torch.optim.Adam(model.parameters(), lr=1e-2)
    before = {k: p.detach().clone() for k, p in model.named_parameters()}
    for _ in range(3):
        opt.zero_grad()
        model(x, mask).float().square().mean().backward()
        opt.step()
    for k, p in model.named_parameters():
        assert torch.isfinite(p).all() and not torch.equal(before[k], p), k


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("rows,k,n", [(33 * 31, 128, 128), (5, 32, 6), (70000, 64, 4), (4099, 256, 260), (2 * 2048 + 1, 128, 36), (5000, 256, 32), (900001, 128, 4)])
def test_weight_gradient_against_float64(dtype, rows, k, n):
    """dy^T x with the rows split over workgroups: ragged row counts (the last chunk and its last
    32-row step are partial), output rows that are not a multiple of 8 or of 32, more than one
    group of 128 output rows, every compiled k."""
    gen = torch.Generator().manual_seed(rows + n)
    x = torch.randn(rows, k, generator=gen).to(DEV, dtype)
    dy = torch.randn(rows, n, generator=gen).to(DEV, dtype)
    got = nn.linear_weight_grad(dy, x)
    assert got.shape == (n, k) and got.dtype == dtype
    want = dy.double().t() @ x.double()
    size = dy.double().abs().t() @ x.double().abs()
    # fp32 accumulation of exact products in a fixed order, one rounding to the dtype
    bound = 0.5 * torch.finfo(dtype).eps * want.abs() + max(rows, 64) ** 0.5 * 2.0**-22 * size + torch.finfo(dtype).smallest_normal
    err = (got.double() - want).abs()
    assert bool((err <= bound).all()), f"max excess {(err - bound).max().item():.3e}"
    assert torch.equal(got, nn.linear_weight_grad(dy, x)), "two runs differ"
    # the bias gradient from the same pass
    dw2, db = nn.linear_weight_grad(dy, x, 0, True)
    assert torch.equal(dw2, got) and db.shape == (n,) and db.dtype == dtype
    want_b, size_b = dy.double().sum(0), dy.double().abs().sum(0)
    bound_b = 0.5 * torch.finfo(dtype).eps * want_b.abs() + max(rows, 64) ** 0.5 * 2.0**-22 * size_b + torch.finfo(dtype).smallest_normal
    assert bool(((db.double() - want_b).abs() <= bound_b).all())


def test_linear_gradients_are_those_of_the_layer():
    torch.manual_seed(5)
    dtype = torch.bfloat16
    x = torch.randn(3, 50, 50, 64, device=DEV, dtype=dtype)
    for n, wb in ((64, False), (4, False), (32, True)):
        m = torch.nn.Linear(64, n, bias=wb).to(DEV, dtype)
        dy = torch.randn(3, 50, 50, n, device=DEV, dtype=dtype)

        def grads(fn):
            xi = x.clone().requires_grad_(True)
            m.zero_grad()
            y = fn(xi)
            y.backward(dy)
            return [y.detach().float(), xi.grad.float()] + [p.grad.float().clone() for p in m.parameters()]

        got = grads(lambda xi: nn.linear(xi, m))
        want = grads(m)
        assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])  # the same library products
        for a, r in zip(got[2:], want[2:]):
            assert a.shape == r.shape
            # the same products, summed in another order and rounded to bf16 once
            assert (a - r).abs().max().item() <= 2.0**-7 * r.abs().max().item(), f"{(a - r).abs().max().item():.3e} of {r.abs().max().item():.3e}"


def test_linear_falls_back_to_torch_where_the_kernel_has_no_instance():
    x = torch.randn(10, 48, device=DEV, dtype=torch.bfloat16, requires_grad=True)  # 48 input channels are not compiled
    m = torch.nn.Linear(48, 8).to(DEV, torch.bfloat16)
    assert not nn._dw_ready(x, m.weight)
    nn.linear(x, m).sum().backward()
    assert m.weight.grad is not None and x.grad is not None
    x32 = torch.randn(10, 64, device=DEV)
    m32 = torch.nn.Linear(64, 8).to(DEV)
    assert torch.equal(nn.linear(x32, m32), m32(x32))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("rows,k,ns", [(33 * 31, 128, (128, 128, 128, 4, 128)), (5, 32, (6,)), (70001, 64, (64, 36, 4)), (300, 128, (260, 32))])
def test_input_gradient_against_float64(dtype, rows, k, ns):
    """sum_p dy_p W_p in one pass: the block's five layers on a ragged row count, fewer rows than
    a tile, output widths that are not multiples of 8 or 32 (scalar loads, partial chunks) and
    wider than one staging chunk."""
    gen = torch.Generator().manual_seed(rows + len(ns))
    dys = [torch.randn(rows, n, generator=gen).to(DEV, dtype) for n in ns]
    ws = [(torch.randn(n, k, generator=gen) * n**-0.5).to(DEV, dtype) for n in ns]
    got = nn.linear_input_grad(dys, ws)
    assert got.shape == (rows, k) and got.dtype == dtype
    want = sum(dy.double() @ w.double() for dy, w in zip(dys, ws))
    size = sum(dy.double().abs() @ w.double().abs() for dy, w in zip(dys, ws))
    # fp32 accumulation of exact products, one rounding to the dtype
    bound = 0.5 * torch.finfo(dtype).eps * want.abs() + sum(ns) * 2.0**-23 * size + torch.finfo(dtype).smallest_normal
    err = (got.double() - want).abs()
    assert bool((err <= bound).all()), f"max excess {(err - bound).max().item():.3e}"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("rows,k,ns,with_bias", [
    (33 * 31, 128, (128, 128, 128, 4, 128), (False, False, False, False, True)),  # the block's five layers, ragged rows
    (5, 32, (6,), (True,)),               # fewer rows than a tile, columns not a multiple of 4
    (2 * 64 * 64, 64, (100, 32), (True, False)),
    (4099, 128, (36, 260), (False, True)),
])
def test_linear_outputs_against_float64(dtype, rows, k, ns, with_bias):
    gen = torch.Generator().manual_seed(k + len(ns))
    x = torch.randn(rows, k, generator=gen).to(DEV, dtype)
    ws = [(torch.randn(n, k, generator=gen) * k**-0.5).to(DEV, dtype) for n in ns]
    bs = [torch.randn(n, generator=gen).to(DEV, dtype) if wb else None for n, wb in zip(ns, with_bias)]
    ys = nn.linear_outputs(x, ws, bs)
    x64 = x.double()
    for w, b, y in zip(ws, bs, ys):
        assert y.shape == (rows, w.shape[0]) and y.dtype == dtype
        want = torch.nn.functional.linear(x64, w.double(), None if b is None else b.double())
        size = torch.nn.functional.linear(x64.abs(), w.double().abs(), None if b is None else b.double().abs())
        # fp32 accumulation of exact products (k of them), one rounding to the dtype
        bound = 0.5 * torch.finfo(dtype).eps * want.abs() + k * 2.0**-23 * size + torch.finfo(dtype).smallest_normal
        err = (y.double() - want).abs()
        assert bool((err <= bound).all()), f"N={w.shape[0]}: max excess {(err - bound).max().item():.3e}"


def test_projection_gradients_are_those_of_the_layers():
    """project(x, layers) against the layers themselves: outputs, input and parameter gradients
    within bf16 rounding, also when one output is unused."""
    torch.manual_seed(6)
    dtype = torch.bfloat16
    x = torch.randn(2, 40, 40, 64, device=DEV, dtype=dtype)
    layers = [torch.nn.Linear(64, n, bias=wb).to(DEV, dtype) for n, wb in ((64, False), (4, False), (32, True))]
    dys = [torch.randn(2, 40, 40, m.out_features, device=DEV, dtype=dtype) for m in layers]
    for used in ((0, 1, 2), (0, 2)):
        def grads(fn):
            xi = x.clone().requires_grad_(True)
            for m in layers:
                m.zero_grad()
            outs = fn(xi)
            torch.autograd.backward([outs[u] for u in used], [dys[u] for u in used])
            return [o.detach().float() for o in outs], [xi.grad.float()] + [None if p.grad is None else p.grad.float().clone() for m in layers for p in m.parameters()]

        (o1, g1), (o2, g2) = grads(lambda xi: nn.project(xi, layers)), grads(lambda xi: [m(xi) for m in layers])
        for a, r in zip(o1, o2):
            assert (a - r).abs().max().item() <= 2.0**-7 * r.abs().max().item()
        for a, r in zip(g1, g2):
            assert (a is None) == (r is None)
            if a is not None:
                assert (a - r).abs().max().item() <= 2.0**-7 * r.abs().max().item(), f"{(a - r).abs().max().item():.3e} of {r.abs().max().item():.3e}"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
def test_heads_outermost_layers(dtype):
    """Layers whose outputs are kept [h, rows, d]: the forward writes that layout, the input and
    weight gradients read it; everything equals the plain-layout kernels on permuted copies, bit
    for bit (the same products in the same order)."""
    gen = torch.Generator().manual_seed(11)
    rows, k, h, d = 4099, 128, 4, 32
    x = torch.randn(rows, k, generator=gen).to(DEV, dtype)
    ws = [(torch.randn(n, k, generator=gen) * k**-0.5).to(DEV, dtype) for n in (h * d, 4, 2 * 64)]
    hds = (d, 0, 64)
    bs = [torch.randn(h * d, generator=gen).to(DEV, dtype), None, torch.randn(2 * 64, generator=gen).to(DEV, dtype)]
    ys = nn.linear_outputs(x, ws, bs, hds)
    plain = nn.linear_outputs(x, ws, bs)
    to_heads = lambda t, hd: t.unflatten(-1, (-1, hd)).movedim(-2, 0).contiguous() if hd else t
    for y, p, hd in zip(ys, plain, hds):
        assert y.shape == to_heads(p, hd).shape and torch.equal(y, to_heads(p, hd))
    dys = [torch.randn(rows, w.shape[0], generator=gen).to(DEV, dtype) for w in ws]
    dys_h = [to_heads(t, hd) for t, hd in zip(dys, hds)]
    assert torch.equal(nn.linear_input_grad(dys_h, ws, hds), nn.linear_input_grad(dys, ws))
    for t, th, hd in zip(dys, dys_h, hds):
        assert torch.equal(nn.linear_weight_grad(th, x, hd), nn.linear_weight_grad(t, x))
        (dw_h, db_h), (dw_p, db_p) = nn.linear_weight_grad(th, x, hd, True), nn.linear_weight_grad(t, x, 0, True)
        assert torch.equal(dw_h, dw_p) and torch.equal(db_h, db_p)


def test_projection_with_heads_outermost_outputs():
    """project(..., head_dims) through autograd against the layers themselves."""
    torch.manual_seed(8)
    dtype, h, d = torch.bfloat16, 2, 32
    x = torch.randn(2, 30, 30, 64, device=DEV, dtype=dtype)
    # (the second heads-outermost layer has a bias, like the layers of the module in reference
    # tests/unit/test_trifast.py:152-169)
    layers = [torch.nn.Linear(64, h * d, bias=False).to(DEV, dtype), torch.nn.Linear(64, 32, bias=True).to(DEV, dtype),
              torch.nn.Linear(64, h * d, bias=True).to(DEV, dtype)]
    dys = [torch.randn(2, 30, 30, m.out_features, device=DEV, dtype=dtype) for m in layers]

    def grads(fn):
        xi = x.clone().requires_grad_(True)
        for m in layers:
            m.zero_grad()
        outs = fn(xi)
        torch.autograd.backward(outs, dys)
        return [o.detach().float() for o in outs], [xi.grad.float()] + [p.grad.float().clone() for m in layers for p in m.parameters()]

    def ours(xi):
        q, g, k = nn.project(xi, layers, (d, 0, d))
        assert q.shape == (h, 2, 30, 30, d) and q.is_contiguous() and k.shape == q.shape and k.is_contiguous()
        return [q.movedim(0, -2).flatten(-2), g, k.movedim(0, -2).flatten(-2)]  # back to [*, h * d] for the comparison

    (o1, g1), (o2, g2) = grads(ours), grads(lambda xi: [m(xi) for m in layers])
    for a, r in zip(o1 + g1, o2 + g2):
        assert a.shape == r.shape
        assert (a - r).abs().max().item() <= 2.0**-7 * r.abs().max().item(), f"{(a - r).abs().max().item():.3e} of {r.abs().max().item():.3e}"


def test_block_kernels_are_well_formed_custom_ops():
    """The block's kernels are torch.library ops like the operator: schema, shape-only
    implementation and autograd registration agree with the real kernels."""
    from torch.library import opcheck

    gen = torch.Generator().manual_seed(21)
    dtype, h, n, d, k = torch.bfloat16, 2, 24, 16, 64
    o = torch.randn(1, h, n, n, d, generator=gen).to(DEV, dtype).requires_grad_(True)
    g = torch.randn(1, n, n, h * d, generator=gen).to(DEV, dtype).requires_grad_(True)
    opcheck(nn._gated_output, (o, g), raise_exception=True)
    opcheck(nn._gated_output_bwd, (torch.randn_like(g), o.detach(), g.detach()), raise_exception=True)
    rows = n * n
    x = torch.randn(rows, k, generator=gen).to(DEV, dtype)
    ws = [(torch.randn(m, k, generator=gen) * k**-0.5).to(DEV, dtype) for m in (h * d, 4)]
    bs = [None, torch.randn(4, generator=gen).to(DEV, dtype)]
    opcheck(nn._linear_outputs, (x, ws, bs, [d, 0]), raise_exception=True)
    dys = [torch.randn(h, rows, d, generator=gen).to(DEV, dtype), torch.randn(rows, 4, generator=gen).to(DEV, dtype)]
    opcheck(nn._linear_input_grad, (dys, ws, [d, 0]), raise_exception=True)
    opcheck(nn._linear_weight_grad, (dys[0], x, d, False), raise_exception=True)
    opcheck(nn._linear_weight_grad, (dys[1], x, 0, True), raise_exception=True)


@pytest.mark.parametrize("ending_node", [False, True], ids=["starting", "ending"])
def test_block_compiles_as_one_graph(ending_node):
    """torch.compile traces the whole block, forward and backward, without a graph break, and the
    compiled block gives the bits of the eager one (aot_eager: the traced graphs run as they are)."""
    torch.manual_seed(5)
    dtype = torch.bfloat16
    block = nn.TriangleAttention(64, 2, 32, ending_node=ending_node).to(DEV, dtype)
    x = torch.randn(2, 40, 40, 64, device=DEV, dtype=dtype)
    mask = torch.rand(2, 40, 40, device=DEV) < 0.3
    dy = torch.randn(2, 40, 40, 64, device=DEV, dtype=dtype)
    explanation = torch._dynamo.explain(block)(x, mask)
    assert explanation.graph_break_count == 0, explanation

    def run(fn):
        xi = x.clone().requires_grad_(True)
        block.zero_grad(set_to_none=True)
        y = fn(xi, mask)
        y.backward(dy)
        return [y.detach(), xi.grad] + [p.grad.clone() for p in block.parameters()]

    eager = run(block)
    compiled = run(torch.compile(block, fullgraph=True, backend="aot_eager"))
    for a, b in zip(compiled, eager):
        assert torch.equal(a, b)


def test_block_in_a_hip_graph():
    """Forward and backward of the block captured into one HIP graph: every replay, with new
    input values and eager work between the replays, gives the bits of the eager block."""
    torch.manual_seed(9)
    dtype = torch.bfloat16
    block = nn.TriangleAttention(64, 2, 32).to(DEV, dtype)
    gen = torch.Generator(device=DEV).manual_seed(3)
    rand = lambda *shape: torch.randn(*shape, device=DEV, dtype=dtype, generator=gen)
    x = rand(1, 72, 72, 64).requires_grad_(True)
    dy = rand(1, 72, 72, 64)
    mask = torch.rand(1, 72, 72, device=DEV, generator=gen) < 0.2
    params = list(block.parameters())

    def step():
        y = block(x, mask)
        y.backward(dy)
        return y

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):  # warm-up outside the capture
            step()
            x.grad = None
            block.zero_grad(set_to_none=True)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y = step()
    for trial in range(3):
        with torch.no_grad():
            x.copy_(rand(*x.shape))
            dy.copy_(rand(*dy.shape))
        graph.replay()
        torch.cuda.synchronize()
        got = [t.detach().clone() for t in [y, x.grad] + [p.grad for p in params]]
        captured = [p.grad for p in params]  # (the graph writes these buffers: put them back afterwards)
        ex = x.detach().clone().requires_grad_(True)
        block.zero_grad(set_to_none=True)
        ey = block(ex, mask)
        ey.backward(dy)
        torch.cuda.synchronize()
        want = [ey.detach(), ex.grad] + [p.grad for p in params]
        for i, (a, b) in enumerate(zip(got, want)):
            assert torch.equal(a, b), f"replay {trial}: tensor {i} differs from the eager result"
        for p, g in zip(params, captured):
            p.grad = g
