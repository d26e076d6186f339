"""The operator is a well-formed torch.library op: schema, fake (meta) kernel and
autograd registration agree with the real kernels, and torch.compile traces through
it without graph breaks.

Counterpart of reference tests/unit/test_trifast_opcheck.py:7-13 (same shapes) and of
the compile recipe in reference scripts/compile.py:5-24 (fullgraph, compiled forward
and backward).
"""

import pytest
import torch
from torch.library import opcheck

import trifast_amd
from oracle import triangle_oracle as orc
from trifast_amd import torch as tt
from trifast_amd.utils import gen_tensors

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n", [16, 128, 256])
@pytest.mark.parametrize("d", [16, 32, 64])
@pytest.mark.parametrize("h", [1, 4])
def test_opcheck_forward_op(n, d, h):
    q, k, v, b, m = gen_tensors(n, d, h, True, "cuda", dtype=torch.bfloat16)
    # opcheck raises on failure: schema, fake tensor, autograd registration, aot dispatch
    opcheck(tt._triangle_attention, (q, k, v, b, m), raise_exception=True)


def test_opcheck_backward_op():
    q, k, v, b, m = gen_tensors(64, 32, 2, True, "cuda", dtype=torch.bfloat16)
    with torch.no_grad():
        o, lse = tt._triangle_attention(q, k, v, b, m)
    do = torch.randn_like(o)
    args = tuple(t.detach() for t in (do, q, k, v, b, o, lse)) + (m,)
    opcheck(tt.triangle_attention_bwd, args, raise_exception=True)


def test_compile_fullgraph_matches_eager():
    q, k, v, b, m = gen_tensors(96, 32, 2, True, "cuda", dtype=torch.bfloat16, batch=2)
    explanation = torch._dynamo.explain(trifast_amd.triangle_attention)(q, k, v, b, m)
    assert explanation.graph_break_count == 0, explanation
    # aot_eager runs the traced forward and backward graphs (fake tensors, functionalised
    # autograd) without asking a code generator for anything else
    compiled = torch.compile(trifast_amd.triangle_attention, fullgraph=True, backend="aot_eager")
    qc, kc, vc, bc = (t.detach().clone().requires_grad_(True) for t in (q, k, v, b))
    qe, ke, ve, be = (t.detach().clone().requires_grad_(True) for t in (q, k, v, b))
    oc = compiled(qc, kc, vc, bc, m)
    oe = trifast_amd.triangle_attention(qe, ke, ve, be, m)
    assert torch.equal(oc, oe)
    do = torch.randn_like(oe)
    oc.backward(do)
    oe.backward(do)
    for name, x, y in zip(("dq", "dk", "dv", "db"), (qc.grad, kc.grad, vc.grad, bc.grad), (qe.grad, ke.grad, ve.grad, be.grad)):
        assert torch.equal(x, y), f"{name} differs between compiled and eager"
    ref = orc.attention_reference(q.float(), k.float(), v.float(), b.float(), m)
    assert (oc.float() - ref).abs().max() < 0.05


def test_hip_graph_capture_and_replay():
    """Forward and backward captured into one HIP graph (what `mode="reduce-overhead"`
    does underneath, reference scripts/compile.py:5-24): the library launches kernels
    only — no allocation, no memset, no synchronisation — so capture records it whole.
    Every replay, with eager work and a synchronisation between replays and new input
    values each time, must reproduce the eager result bit for bit."""
    n, h, d = 96, 2, 32
    dev, dtype = "cuda", torch.bfloat16
    gen = torch.Generator(device=dev).manual_seed(3)
    rand = lambda *shape: torch.randn(*shape, device=dev, dtype=dtype, generator=gen)
    q, k, v = (rand(1, h, n, n, d).requires_grad_(True) for _ in range(3))
    b = rand(1, h, n, n).requires_grad_(True)
    mask = torch.rand(1, n, n, device=dev, generator=gen) < 0.2
    do = rand(1, h, n, n, d)

    def step():
        o = trifast_amd.triangle_attention(q, k, v, b, mask)
        o.backward(do)
        return o

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):  # warm-up outside the capture, as graph capture of autograd needs
            step()
            for t in (q, k, v, b):
                t.grad = None
    torch.cuda.current_stream().wait_stream(side)

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        o = step()
    for trial in range(3):
        with torch.no_grad():
            for t in (q, k, v, b, do):
                t.copy_(rand(*t.shape))
        graph.replay()
        torch.cuda.synchronize()
        got = [x.detach().clone() for x in (o, q.grad, k.grad, v.grad, b.grad)]
        # the same step eagerly, on copies
        eq, ek, ev, eb = (t.detach().clone().requires_grad_(True) for t in (q, k, v, b))
        eo = trifast_amd.triangle_attention(eq, ek, ev, eb, mask)
        eo.backward(do)
        torch.cuda.synchronize()
        for name, x, e in zip(("o", "dq", "dk", "dv", "db"), got, (eo, eq.grad, ek.grad, ev.grad, eb.grad)):
            assert torch.equal(x, e.detach()), f"replay {trial}: {name} differs from the eager result"


def test_compile_with_dynamic_shapes():
    """One compiled graph with symbolic sizes serves several n (the shape-only implementations
    work on symbolic ints) and gives the eager bits, forward and backward."""
    compiled = torch.compile(trifast_amd.triangle_attention, fullgraph=True, backend="aot_eager", dynamic=True)
    for n in (48, 64, 80):
        q, k, v, b, m = gen_tensors(n, 32, 2, True, "cuda", dtype=torch.bfloat16)
        qc, kc, vc, bc = (t.detach().clone().requires_grad_(True) for t in (q, k, v, b))
        qe, ke, ve, be = (t.detach().clone().requires_grad_(True) for t in (q, k, v, b))
        oc = compiled(qc, kc, vc, bc, m)
        oe = trifast_amd.triangle_attention(qe, ke, ve, be, m)
        assert torch.equal(oc, oe)
        oc.sum().backward()
        oe.sum().backward()
        for name, x, y in zip(("dq", "dk", "dv", "db"), (qc.grad, kc.grad, vc.grad, bc.grad), (qe.grad, ke.grad, ve.grad, be.grad)):
            assert torch.equal(x, y), f"n={n}: {name} differs between compiled and eager"
