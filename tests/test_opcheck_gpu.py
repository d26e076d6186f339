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
