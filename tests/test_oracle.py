"""Pins the CPU oracle (oracle/triangle_oracle.py) without the reference package.

The reference's tests hold no stored vectors for this path, so the restatement
is pinned by (a) a library routine it must reduce to, (b) an explicit float64
loop nest that shares no code with it, (c) the reference's own second
formulation, (d) finite differences, and (e) invariants of softmax attention,
each chosen so that a plausible slip (wrong axis for bias or mask, scale applied
to the bias, mask polarity, a dropped delta term, a transposed operand) breaks
at least one of them.
"""

from pathlib import Path

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import triangle_oracle as orc

GOLDEN = Path(__file__).resolve().parent / "golden"


def rand_inputs(b, h, n, d, seed, p_mask=0.3, full_rows=(), dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    q, k, v = (torch.randn(b, h, n, n, d, generator=g, dtype=dtype) for _ in range(3))
    bias = torch.randn(b, h, n, n, generator=g, dtype=dtype)
    mask = torch.rand(b, n, n, generator=g) < p_mask
    # keep at least one key per row, then force the requested fully masked rows
    mask[:, :, 0] &= ~mask.all(dim=-1)
    for r in full_rows:
        mask[:, r, :] = True
    do = torch.randn(b, h, n, n, d, generator=g, dtype=dtype)
    return q, k, v, bias, mask, do


# ---------------------------------------------------------------- (a) library
@pytest.mark.parametrize("full_rows", [(), (1,)])
def test_forward_reduces_to_sdpa(full_rows):
    q, k, v, bias, mask, _ = rand_inputs(2, 3, 7, 8, seed=0, full_rows=full_rows)
    o = orc.attention_reference(q, k, v, bias, mask)
    # rows i become a batch axis: [b, i, h, j, d]; additive mask = bias[j,k] + min*mask[i,k]
    qp, kp, vp = (t.permute(0, 2, 1, 3, 4) for t in (q, k, v))
    add = bias[:, None, :, :, :] + (torch.finfo(torch.float32).min * mask.float())[:, :, None, None, :]
    ref = F.scaled_dot_product_attention(qp, kp, vp, attn_mask=add).permute(0, 2, 1, 3, 4)
    torch.testing.assert_close(o, ref, rtol=1e-5, atol=1e-5)


# ------------------------------------------------------------- (b) loop nest
@pytest.mark.parametrize("full_rows", [(), (2,)])
def test_against_float64_loops(full_rows):
    q, k, v, bias, mask, do = rand_inputs(2, 2, 5, 4, seed=1, full_rows=full_rows)
    o, dq, dk, dv, db = orc.forward_backward(q, k, v, bias, mask, do)
    lse = orc.lse_reference(q, k, bias, mask)
    o64, lse64, dq64, dk64, dv64, db64 = orc.brute_force_f64(q, k, v, bias, mask, do)
    for name, got, want in (("o", o, o64), ("lse", lse, lse64), ("dq", dq, dq64), ("dk", dk, dk64), ("dv", dv, dv64), ("db", db, db64)):
        want = torch.from_numpy(want)
        if name == "lse":
            # fully masked rows: logsumexp sits at finfo.min, compare relatively
            torch.testing.assert_close(got.double(), want, rtol=1e-6, atol=1e-5, msg=name)
        else:
            torch.testing.assert_close(got.double(), want, rtol=1e-4, atol=2e-5, msg=name)


def test_fully_masked_row_is_uniform_and_has_gradient():
    q, k, v, bias, mask, do = rand_inputs(1, 2, 6, 4, seed=2, full_rows=(3,))
    o, dq, dk, dv, db = orc.forward_backward(q, k, v, bias, mask, do)
    torch.testing.assert_close(o[:, :, 3], v[:, :, 3].mean(dim=2, keepdim=True).expand_as(o[:, :, 3]), rtol=1e-5, atol=1e-6)
    assert dq[:, :, 3].abs().max() > 1e-4 and dk[:, :, 3].abs().max() > 1e-4


# ---------------------------------------------------- (c) second formulation
def test_two_formulations_agree():
    q, k, v, bias, mask, do = rand_inputs(2, 2, 9, 8, seed=3)
    a = orc.forward_backward(q, k, v, bias, mask, do, fn=orc.attention_reference)
    b = orc.forward_backward(q, k, v, bias, mask, do, fn=orc.triangle_attention_simple)
    for x, y in zip(a, b):
        torch.testing.assert_close(x, y, rtol=1e-4, atol=1e-5)


# --------------------------------------------------------- (d) finite diffs
def test_gradcheck_float64():
    q, k, v, bias, mask, _ = rand_inputs(1, 2, 3, 2, seed=4, dtype=torch.float64)
    q, k, v, bias = (t.requires_grad_(True) for t in (q, k, v, bias))
    assert torch.autograd.gradcheck(lambda *a: orc.attention_reference(*a, mask), (q, k, v, bias), eps=1e-6, atol=1e-5)


# -------------------------------------------------------------- (e) invariants
def test_invariants():
    q, k, v, bias, mask, do = rand_inputs(2, 2, 8, 8, seed=5, p_mask=0.4)
    o, dq, dk, dv, db = orc.forward_backward(q, k, v, bias, mask, do)
    # rows of P sum to one: constant v gives constant o
    oc = orc.attention_reference(q, k, torch.full_like(v, 0.75), bias, mask)
    torch.testing.assert_close(oc, torch.full_like(oc, 0.75), rtol=1e-5, atol=1e-6)
    # softmax is shift invariant per (h, j): db sums to zero over keys
    assert db.sum(dim=-1).abs().max() < 1e-4
    # a constant added to bias[h, j, :] changes nothing
    o2 = orc.attention_reference(q, k, v, bias + torch.randn(2, 2, 8, 1), mask)
    torch.testing.assert_close(o, o2, rtol=1e-4, atol=1e-5)
    # masked keys of partially masked rows receive exactly zero gradient
    mk = mask[:, None, :, :, None].expand_as(dk)
    assert dk[mk].abs().max() == 0 and dv[mk].abs().max() == 0
    # permuting keys (k, v rows, bias columns, mask columns) permutes nothing in o
    perm = torch.randperm(8, generator=torch.Generator().manual_seed(9))
    o3 = orc.attention_reference(q, k[:, :, :, perm], v[:, :, :, perm], bias[..., perm], mask[..., perm])
    torch.testing.assert_close(o, o3, rtol=1e-4, atol=1e-5)
    # row i depends only on q[i], k[i], v[i], mask[i] and the shared bias
    o4 = orc.attention_reference(q[:, :, 2:5], k[:, :, 2:5], v[:, :, 2:5], bias, mask[:, 2:5])
    torch.testing.assert_close(o[:, :, 2:5], o4, rtol=1e-5, atol=1e-6)
    # bias is indexed [j, k] and the mask [i, k]: transposing either must change o
    assert (orc.attention_reference(q, k, v, bias.transpose(-1, -2), mask) - o).abs().max() > 1e-3
    assert (orc.attention_reference(q, k, v, bias, mask.transpose(-1, -2)) - o).abs().max() > 1e-3
    # scale is 1/sqrt(d) on q.k only: zero bias and mask reduce to textbook attention
    z = torch.zeros_like(bias)
    nomask = torch.zeros_like(mask)
    p = torch.softmax(torch.einsum("bhijd,bhikd->bhijk", q, k) / 8**0.5, dim=-1)
    torch.testing.assert_close(orc.attention_reference(q, k, v, z, nomask), torch.einsum("bhijk,bhikd->bhijd", p, v), rtol=1e-4, atol=1e-5)


def test_chunked_matches_unchunked():
    q, k, v, bias, mask, do = rand_inputs(1, 2, 11, 8, seed=6, full_rows=(4,))
    a = orc.forward_backward(q, k, v, bias, mask, do)
    b = orc.forward_backward_chunked(q, k, v, bias, mask, do, chunk=3)
    for x, y in zip(a, b):
        torch.testing.assert_close(x, y, rtol=1e-5, atol=1e-6)


def test_acceptance_rule_helpers():
    ref = torch.zeros(4)
    orc.compare_values(ref + 2e-3, ref + 1e-3, ref, eps=1e-3)  # 2e-3 <= 3 * (1e-3 + 1e-3)
    with pytest.raises(AssertionError):
        orc.compare_values(ref + 7e-3, ref + 1e-3, ref, eps=1e-3)


# ------------------------------------------------------------ golden fixtures
@pytest.mark.parametrize("name", ["tiny_n6_h2_d16", "plumb_n16_h4_d32", "ragged_n19_h2_d32"])
def test_golden_fixtures(name):
    z = np.load(GOLDEN / f"{name}.npz")
    t = {key: torch.from_numpy(z[key]) for key in z.files}
    o, dq, dk, dv, db = orc.forward_backward(t["q"], t["k"], t["v"], t["bias"], t["mask"], t["do"])
    lse = orc.lse_reference(t["q"], t["k"], t["bias"], t["mask"])
    for key, got in (("o", o), ("lse", lse), ("dq", dq), ("dk", dk), ("dv", dv), ("db", db)):
        torch.testing.assert_close(got, t[key], rtol=1e-5, atol=1e-6, msg=key)
        if f"{key}_f64" in t:
            torch.testing.assert_close(got.double(), t[f"{key}_f64"], rtol=1e-4, atol=2e-5, msg=key + "_f64")


# ------------------------------------------------- checker helpers, hand-computed
def test_cosine_similarity_hand_values():
    # (1,2,2).(2,1,2) = 8, both norms 3: cos = 8/9; orthogonal and opposite vectors
    a, b = torch.tensor([1.0, 2.0, 2.0]), torch.tensor([2.0, 1.0, 2.0])
    assert abs(orc.cosine_similarity(a, b) - 8.0 / 9.0) < 1e-6
    assert abs(orc.cosine_similarity(torch.tensor([1.0, 0.0, 0.0]), torch.tensor([0.0, 3.0, 0.0]))) < 1e-7
    assert abs(orc.cosine_similarity(a, -2 * a) + 1.0) < 1e-6
    # inputs of any shape and dtype are flattened and compared in float32
    assert abs(orc.cosine_similarity(a.reshape(1, 3).bfloat16(), b.reshape(3, 1).half()) - 8.0 / 9.0) < 1e-6
    # a zero vector gives 0, not NaN (the eps in the denominator)
    assert orc.cosine_similarity(torch.zeros(3), b) == 0.0


def test_direction_checks_hand_values():
    ref = torch.tensor([1.0, 0.0, 0.0])
    good = torch.tensor([1.0, 0.1, 0.0])      # cos = 1/sqrt(1.01) = 0.99504
    worse = torch.tensor([1.0, 0.15, 0.0])    # cos = 1/sqrt(1.0225) = 0.98894
    bad = torch.tensor([1.0, 1.0, 0.0])       # cos = 0.7071
    orc.compare_directions(good, good, ref)
    with pytest.raises(AssertionError, match="kernel->ref"):
        orc.compare_directions(worse, good, ref)  # 0.98894 < 0.99
    with pytest.raises(AssertionError, match="pt->ref"):
        orc.compare_directions(good, worse, ref)
    # relative rule: cos(kernel) >= 0.99 * cos(pt); 0.98894 >= 0.99 * 0.99504 = 0.98509
    orc.compare_relative_direction(worse, good, ref)
    orc.compare_relative_direction(bad, bad, ref)  # equal cosines always pass
    with pytest.raises(AssertionError, match="relative direction"):
        orc.compare_relative_direction(bad, good, ref)  # 0.7071 < 0.98509


def test_compare_dot_hand_values():
    # scores are dot(x, ref) / dot(ref, ref): ref.ref = 9; kernel 8/9, pt 9/9
    ref = torch.tensor([1.0, 2.0, 2.0])
    kern = torch.tensor([2.0, 1.0, 2.0])
    with pytest.raises(AssertionError, match="dot product"):
        orc.compare_dot(kern, ref, ref)  # 8/9 - 1 = -0.111 < -0.01
    orc.compare_dot(kern, ref, ref, threshold=0.12)
    orc.compare_dot(ref, kern, ref)       # a kernel better than pt is fine (+0.111)
    orc.compare_dot(0.995 * ref, ref, ref)  # -0.005 >= -0.01
    with pytest.raises(AssertionError):
        orc.compare_dot(0.98 * ref, ref, ref)  # -0.02


def test_gen_tensors_shapes_draw_order_and_mask():
    n, d, h, bs = 24, 8, 3, 2
    g = torch.Generator().manual_seed(5)
    q, k, v, b, m = orc.gen_tensors(n, d, h, True, "cpu", torch.float32, bs, 2.0, generator=g)
    assert q.shape == k.shape == v.shape == (bs, h, n, n, d) and b.shape == (bs, h, n, n) and m.shape == (bs, n, n)
    assert all(t.requires_grad and t.dtype == torch.float32 for t in (q, k, v, b)) and m.dtype == torch.bool
    # draw order q, k, v, bias, mask from one generator: replay the same draws by hand
    g2 = torch.Generator().manual_seed(5)
    for got in (q, k, v):
        assert torch.equal(got.detach(), torch.normal(0, 2.0, (bs, h, n, n, d), generator=g2))
    assert torch.equal(b.detach(), torch.normal(0, 2.0, (bs, h, n, n), generator=g2))
    assert torch.equal(m, torch.randint(0, 2, (bs, n, n), generator=g2).bool())
    # std is honoured; the mask is a fair coin (1152 draws: 3 sigma = 4.4 %)
    assert abs(q.detach().std().item() - 2.0) < 0.05
    assert abs(m.float().mean().item() - 0.5) < 0.06
    # without a mask: all False (nothing masked out)
    *_, m0 = orc.gen_tensors(n, d, h, False, "cpu", torch.float32, bs, 1.0, generator=g)
    assert m0.dtype == torch.bool and not m0.any()
