"""Pair tensors with more than 2^31 elements: n = 4096, h = 6, d = 32 in bf16.

Offsets into q/k/v/o and the gradients no longer fit 32 bits there, which the smaller
parity shapes never exercise.  The n^3 logits of the whole problem are out of reach for
a dense check (1 TiB in fp32), but triangle attention is local to a pair row: o[i], dq[i],
dk[i], dv[i] depend on row i of q, k, v, do only, and the bias gradient is the sum of
per-row terms.  With do zero outside a few chosen rows, db is the sum over those rows, so
everything is checked exactly against the row-wise restatement of
reference src/trifast/equiv.py:42-69 below, in float32, with the reference's tolerance rule
(tests/utils.py:31-36) against the same computation in bf16.
"""

import math

import pytest
import torch

import trifast_amd
from oracle import triangle_oracle as orc

pytestmark = pytest.mark.gpu

N, H, D = 4096, 6, 32
ROWS = (0, 1, 1777, 4095)  # first, second, one in the middle, last


def row_attention(q_i, k_i, v_i, bias, mask_i):
    """One pair row: q_i, k_i, v_i [h, n, d], bias [h, n, n], mask_i [n] (True = masked)."""
    s = torch.einsum("hjd,hkd->hjk", q_i, k_i) / math.sqrt(q_i.shape[-1]) + bias
    s = s + mask_i.to(s.dtype)[None, None, :] * torch.finfo(s.dtype).min
    return torch.einsum("hjk,hkd->hjd", torch.softmax(s, dim=-1), v_i)


def rows_reference(q, k, v, bias, mask, do, dtype, rows=ROWS):
    """o, dq, dk, dv of the chosen rows and db summed over them, computed in `dtype`."""
    out = {}
    db = torch.zeros_like(bias[0], dtype=torch.float32)
    for i in rows:
        q_i, k_i, v_i = (t[0, :, i].to(dtype).detach().requires_grad_(True) for t in (q, k, v))
        b = bias[0].to(dtype).detach().requires_grad_(True)
        o_i = row_attention(q_i, k_i, v_i, b, mask[0, i])
        o_i.backward(do[0, :, i].to(dtype))
        out[i] = tuple(t.detach().float() for t in (o_i, q_i.grad, k_i.grad, v_i.grad))
        db += b.grad.float()
    return out, db


def test_offsets_beyond_32_bits():
    assert H * N * N * D > 2**31
    dev = "cuda"
    g = torch.Generator(device=dev).manual_seed(4096)
    dtype = torch.bfloat16
    q, k, v = (torch.randn(1, H, N, N, D, device=dev, dtype=dtype, generator=g) for _ in range(3))
    bias = torch.randn(1, H, N, N, device=dev, dtype=dtype, generator=g)
    mask = torch.rand(1, N, N, device=dev, generator=g) < 0.3
    mask[0, 1777, :] = True  # a fully masked row among the checked ones
    do = torch.zeros_like(q)
    for i in ROWS:
        do[0, :, i] = torch.randn(H, N, D, device=dev, dtype=dtype, generator=g)

    q, k, v, bias = (t.requires_grad_(True) for t in (q, k, v, bias))
    o = trifast_amd.triangle_attention(q, k, v, bias, mask)
    o.backward(do)
    torch.cuda.synchronize()

    ref, db_ref = rows_reference(q, k, v, bias, mask, do, torch.float32)
    pt, db_pt = rows_reference(q, k, v, bias, mask, do, dtype)
    eps = orc.DTYPE_EPS[dtype]
    for i in ROWS:
        got = (o[0, :, i], q.grad[0, :, i], k.grad[0, :, i], v.grad[0, :, i])
        for name, x, p, r in zip(("o", "dq", "dk", "dv"), got, pt[i], ref[i]):
            assert torch.isfinite(x.float()).all(), f"row {i} {name}: non-finite values"
            orc.compare_values(x.detach(), p, r, f"n={N} row {i} {name}", eps=eps)
    orc.compare_values(bias.grad[0], db_pt, db_ref, f"n={N} db", eps=eps)
    # rows that received no upstream gradient have none to give
    for i in (2, 4094):
        assert not q.grad[0, :, i].any() and not k.grad[0, :, i].any() and not v.grad[0, :, i].any()


@pytest.mark.parametrize("n,h", [(1792, 3), (2048, 2), (2944, 1)])
def test_bias_gradient_with_few_head_groups(n, h):
    """Long rows with few heads: the bias-gradient kernel then has fewer (batch*head, row
    chunk) groups than the GPU has XCDs and deals the blocks of a group to several XCDs
    (3, 2 and 1 groups here).  db is checked through rows that carry all of the upstream
    gradient, as above."""
    dev, dtype = "cuda", torch.bfloat16
    rows = (0, n // 2 + 1, n - 1)
    g = torch.Generator(device=dev).manual_seed(n + h)
    q, k, v = (torch.randn(1, h, n, n, D, device=dev, dtype=dtype, generator=g) * D**-0.25 for _ in range(3))
    bias = torch.randn(1, h, n, n, device=dev, dtype=dtype, generator=g)
    mask = torch.rand(1, n, n, device=dev, generator=g) < 0.2
    do = torch.zeros_like(q)
    for i in rows:
        do[0, :, i] = torch.randn(h, n, D, device=dev, dtype=dtype, generator=g)
    q, k, v, bias = (t.requires_grad_(True) for t in (q, k, v, bias))
    trifast_amd.triangle_attention(q, k, v, bias, mask).backward(do)
    torch.cuda.synchronize()
    _, db_ref = rows_reference(q, k, v, bias, mask, do, torch.float32, rows)
    _, db_pt = rows_reference(q, k, v, bias, mask, do, dtype, rows)
    assert torch.isfinite(bias.grad.float()).all()
    orc.compare_values(bias.grad[0], db_pt, db_ref, f"n={n} h={h} db", eps=orc.DTYPE_EPS[dtype])


# (the last pass runs with 2, 8, 4, 6, 2 and 2 key tiles per wave)
@pytest.mark.parametrize("n,h,dtype", [(1030, 2, torch.bfloat16), (2048, 1, torch.bfloat16), (1500, 1, torch.float16), (1700, 1, torch.bfloat16), (2100, 1, torch.bfloat16), (4200, 1, torch.bfloat16)],
                         ids=["n1030_two_passes_ragged", "n2048_two_passes", "n1500_f16", "n1700", "n2100_three_passes", "n4200_five_passes"])
def test_row_resident_backward_in_several_passes(n, h, dtype, monkeypatch):
    """Rows longer than the row-resident kernel holds at once run it once per 1024 keys: dk, dv
    of each pass's keys and the dq summed over the passes are checked on a few pair rows, among
    them a fully masked one, one whose attended keys all lie in the last pass and one whose
    attended keys all lie in the first; db (from the db kernel, which reads the planes the first
    pass leaves) through the rows that carry the upstream gradient.  Two runs give the same bits."""
    from trifast_amd import _lib, tuner

    lib = _lib.load()
    code = _lib.BF16 if dtype == torch.bfloat16 else _lib.F16
    nt = lib.trifast_num_tiles(_lib.KERNEL_BWD_KV)
    tile = nt - 1
    assert lib.trifast_bwd_kv_tile_writes_dq(tile) and lib.trifast_supports(_lib.KERNEL_BWD_KV, tile, n, h, D, code)
    real_pick = tuner.pick
    monkeypatch.setattr(tuner, "pick", lambda kern, *a, **kw: tile if kern == _lib.KERNEL_BWD_KV else real_pick(kern, *a, **kw))
    dev = "cuda"
    rows = (0, 3, 4, 5, n // 2, n - 1)
    g = torch.Generator(device=dev).manual_seed(n)
    q, k, v = (torch.randn(1, h, n, n, D, device=dev, dtype=dtype, generator=g) * D**-0.25 for _ in range(3))
    bias = torch.randn(1, h, n, n, device=dev, dtype=dtype, generator=g)
    mask = torch.rand(1, n, n, device=dev, generator=g) < 0.2
    mask[0, 3, :] = True          # fully masked
    mask[0, 4, :1024] = True      # nothing to attend to in the first pass
    mask[0, 5, 1000:] = True      # nothing in the later passes (and a ragged edge inside the first)
    do = torch.zeros_like(q)
    for i in rows:
        do[0, :, i] = torch.randn(h, n, D, device=dev, dtype=dtype, generator=g)
    grads = []
    for _ in range(2):
        leaves = [t.detach().clone().requires_grad_(True) for t in (q, k, v, bias)]
        o = trifast_amd.triangle_attention(*leaves, mask)
        o.backward(do)
        torch.cuda.synchronize()
        grads.append([t.grad for t in leaves])
    for a, c in zip(*grads):
        assert torch.equal(a, c), "two runs differ"
    dq, dk, dv, db = grads[0]
    ref, db_ref = rows_reference(q, k, v, bias, mask, do, torch.float32, rows)
    pt, db_pt = rows_reference(q, k, v, bias, mask, do, dtype, rows)
    eps = orc.DTYPE_EPS[dtype]
    for i in rows:
        got = (dq[0, :, i], dk[0, :, i], dv[0, :, i])
        for name, x, p, r in zip(("dq", "dk", "dv"), got, pt[i][1:], ref[i][1:]):
            assert torch.isfinite(x.float()).all(), f"row {i} {name}: non-finite values"
            orc.compare_values(x.detach(), p, r, f"n={n} row {i} {name}", eps=eps)
    orc.compare_values(db[0], db_pt, db_ref, f"n={n} db", eps=eps)
    # masked-out keys get exactly zero dk, dv (row 4: the whole first pass)
    assert not dk[0, :, 4, :1024].any() and not dv[0, :, 4, :1024].any()
    # rows without upstream gradient have none to give
    assert not dq[0, :, 1].any() and not dk[0, :, n - 2].any()


def test_passes_write_strided_gradients():
    """The ending-node entry at a row length that needs two passes: q, k, v, dO and the gradients
    are pair-transposed views there, and dq travels between the passes through the strided dq
    tensor itself.  The same numbers must come out as from contiguous copies of the views."""
    n, h, dtype, dev = 1040, 1, torch.bfloat16, "cuda"
    g = torch.Generator(device=dev).manual_seed(7)
    q, k, v, do = (torch.randn(1, h, n, n, D, device=dev, dtype=dtype, generator=g) * D**-0.25 for _ in range(4))
    bias = torch.randn(1, h, n, n, device=dev, dtype=dtype, generator=g)
    mask = torch.rand(1, n, n, device=dev, generator=g) < 0.1

    def run(fn, *tensors):
        leaves = [t.detach().clone().requires_grad_(True) for t in tensors]
        out = fn(*leaves)
        return out, leaves

    o1, l1 = run(lambda a, b_, c, d_: trifast_amd.triangle_attention_ending_node(a, b_, c, d_, mask), q, k, v, bias)
    o1.backward(do)
    t = lambda x: x.transpose(2, 3).contiguous()
    o2, l2 = run(lambda a, b_, c, d_: trifast_amd.triangle_attention(a, b_, c, d_, mask.transpose(1, 2).contiguous()),
                 t(q), t(k), t(v), bias.transpose(2, 3).contiguous())
    o2.backward(t(do))
    torch.cuda.synchronize()
    assert torch.equal(o1, o2.transpose(2, 3))
    for name, a, c in zip(("dq", "dk", "dv"), l1[:3], l2[:3]):
        assert torch.equal(a.grad, c.grad.transpose(2, 3)), name
    assert torch.equal(l1[3].grad, l2[3].grad.transpose(2, 3)), "db"
