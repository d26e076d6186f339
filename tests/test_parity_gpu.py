"""GPU parity tests: the HIP kernels, called through the C ABI by the operator,
against the CPU-pinned oracle on the same seeded inputs.

Acceptance is the reference's own rule (tests/utils.py:31-36,
tests/unit/test_trifast.py:19-23): for every output x in (o, dq, dk, dv, db)
    max|kernel - ref| <= 3 * (max|pt - ref| + eps),  eps = 1e-3 (bf16/fp16), 1e-4 (fp32)
where ref is the oracle in float32 and pt the oracle in the kernel's dtype, plus
the direction tests of reference tests/unit/test_trifast.py:92-149.  float32
results are additionally held to 1e-5 relative (max-abs over max-abs of ref).
"""

import os
from pathlib import Path

import numpy as np
import pytest
import torch

import bench
import trifast_amd
from oracle import triangle_oracle as orc
from trifast_amd import _lib, tuner
from trifast_amd import torch as tt

pytestmark = pytest.mark.gpu

GOLDEN = Path(__file__).resolve().parent / "golden"
DEV = "cuda"
NAMES = ("o", "dq", "dk", "dv", "db")


def kernel_fwd_bwd(q, k, v, bias, mask, do):
    q, k, v, bias = (t.detach().clone().requires_grad_(True) if t.is_contiguous() else t.detach().requires_grad_(True) for t in (q, k, v, bias))
    o = trifast_amd.triangle_attention(q, k, v, bias, mask)
    o.backward(do)
    return o.detach(), q.grad, k.grad, v.grad, bias.grad


def oracle_fwd_bwd(q, k, v, bias, mask, do, chunk=None):
    n = q.shape[2]
    if chunk is None or chunk >= n:
        return orc.forward_backward(q, k, v, bias, mask, do)
    return orc.forward_backward_chunked(q, k, v, bias, mask, do, chunk=chunk)


def check_all(kernel, pt, ref, dtype, tag, directions=True, rel_floor=1e-30):
    eps = orc.DTYPE_EPS[dtype]
    report = []
    for name, x, p, r in zip(NAMES, kernel, pt, ref):
        assert torch.isfinite(x.float()).all(), f"{tag} {name}: non-finite values"
        a, b = orc.compare_values(x, p, r, f"{tag} {name}", eps=eps)
        report.append(f"{name}={a:.2e}(pt {b - eps:.2e})")
        if dtype == torch.float32:
            # (rel_floor: for answers that are zero by construction the bound is absolute)
            rel = a / max(r.abs().max().item(), rel_floor)
            assert rel < 2e-5, f"{tag} {name}: fp32 relative error {rel:.2e}"
        if directions:
            orc.compare_relative_direction(x, p, r, f"{tag} {name}")
            orc.compare_directions(x, p, r, f"{tag} {name}")
            orc.compare_dot(x, p, r, f"{tag} {name}")
    print(f"{tag}: " + " ".join(report))


# the second output of the operator: log-sum-exp of the logits (natural log, fp32).  The
# kernel sums the probabilities it feeds to the second product, i.e. rounded to the input
# dtype, so in 16-bit dtypes lse carries up to half an ulp of that dtype in relative error
# of the sum: 2^-9 (bf16), 2^-12 (fp16); the bounds below are twice that.  A row whose keys
# are all masked reports finfo(dtype).min + ln n (reference src/trifast/triton.py:104-109,130-132).
LSE_ABS_TOL = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -10}


def check_lse(low, m, dtype, tag):
    with torch.no_grad():
        _, lse = tt._triangle_attention(*low, m)
    n = m.shape[-1]
    ref = orc.lse_reference(low[0].float(), low[1].float(), low[3].float(), m)
    full = m.all(dim=-1)[:, None, :, None].expand_as(lse)  # rows whose keys are all masked
    assert torch.isfinite(lse).all(), f"{tag} lse: non-finite values"
    if (~full).any():
        err = (lse - ref)[~full].abs().max().item()
        if dtype == torch.float32:
            bound = 1e-5 * max(ref[~full].abs().max().item(), 1.0)
        else:
            bound = LSE_ABS_TOL[dtype]
        assert err <= bound, f"{tag} lse: max error {err:.3e} > {bound:.3e}"
    if full.any():
        want = torch.tensor(torch.finfo(dtype).min, dtype=torch.float32) + float(np.log(n))
        got = lse[full]
        assert torch.allclose(got, want.to(got.device).expand_as(got), rtol=1e-6, atol=0), f"{tag} lse of fully masked rows: {got.flatten()[:4].tolist()} != {want.item()}"


# ---------------------------------------------------------------------------
# the reference's own test grid (tests/unit/test_trifast.py:26-38), thinned over n
# unless TRIFAST_FULL_GRID=1
# ---------------------------------------------------------------------------
# (every n with TRIFAST_FULL_GRID=1: two minutes on the GPU; by default every fourth n and the
# sizes next to the tile edges)
_NS = list(range(17, 200)) if os.getenv("TRIFAST_FULL_GRID") == "1" else sorted(
    set(range(17, 200, 4)) | {17, 31, 32, 33, 47, 63, 64, 65, 95, 96, 97, 100, 127, 128, 129, 159, 160, 161, 191, 192, 193, 199})
_SHAPES = [(16, 1, 16), (32, 1, 32), (64, 1, 64), (16, 4, 128)] + [(n, 4, 32) for n in _NS]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=["f32", "f16", "bf16"])
@pytest.mark.parametrize("mask", [True, False], ids=["mask", "nomask"])
@pytest.mark.parametrize("bs", [1, 2])
@pytest.mark.parametrize("std", [1.0, 2.0])
@pytest.mark.parametrize("n,h,d", _SHAPES)
def test_values_and_vectors(n, h, d, mask, bs, dtype, std):
    g = torch.Generator().manual_seed(1337 + 7 * n + h + d + bs)
    q, k, v, b, m = orc.gen_tensors(n, d, h, mask, "cpu", torch.float32, bs, std, generator=g)
    q, k, v, b, m = (t.detach().to(DEV) for t in (q, k, v, b, m))
    # loss = o.sum(): the upstream gradient is an all-ones stride-0 tensor (reference :51)
    do32 = torch.ones((), device=DEV).expand(q.shape)
    ref = orc.forward_backward(q, k, v, b, m, do32)
    low = [t.to(dtype) for t in (q, k, v, b)]
    do = torch.ones((), device=DEV, dtype=dtype).expand(q.shape)
    pt = orc.forward_backward(*low, m, do)
    kern = kernel_fwd_bwd(*low, m, do)
    tag = f"n={n} h={h} d={d} bs={bs} std={std} mask={mask} {dtype}"
    check_all(kern, pt, ref, dtype, tag)
    check_lse(low, m, dtype, tag)


# ---------------------------------------------------------------------------
# every compiled tile of every kernel gives the same answer
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bf16", "f32"])
@pytest.mark.parametrize("n,h,d", [(70, 2, 32), (130, 1, 64), (40, 1, 16), (33, 1, 128)])
def test_every_tile(n, h, d, dtype, monkeypatch):
    lib = _lib.load()
    code = tt._DTYPE_CODE[dtype]
    g = torch.Generator().manual_seed(n)
    q, k, v, b, m = orc.gen_tensors(n, d, h, True, "cpu", torch.float32, 2, 1.0, generator=g)
    m[:, n // 2, :] = True  # one fully masked row
    do = torch.randn(q.shape, generator=g)
    q, k, v, b, m, do = (t.detach().to(DEV) for t in (q, k, v, b, m, do))
    low = [t.to(dtype) for t in (q, k, v, b)]
    ref = orc.forward_backward(*(t.float() for t in low), m, do.to(dtype).float())
    pt = orc.forward_backward(*low, m, do.to(dtype))
    ran = 0
    for tile in range(max(lib.trifast_num_tiles(kern) for kern in range(4))):
        tiles = {kern: tile if lib.trifast_supports(kern, tile, n, h, d, code) else None for kern in range(4)}
        if all(t is None for t in tiles.values()):
            continue
        monkeypatch.setattr(tuner, "pick", lambda kern, n_, h_, d_, dt, launch, extra_cost=None, tiles=tiles: tiles[kern] if tiles[kern] is not None else lib.trifast_default_tile(kern, n_, h_, d_, code))
        kern_out = kernel_fwd_bwd(*low, m, do.to(dtype))
        check_all(kern_out, pt, ref, dtype, f"tile {tile} n={n} d={d} {dtype}", directions=False)
        ran += 1
    # large head dims in fp32 leave few tiles that fit the register file and LDS
    assert ran >= (3 if d * (4 if dtype == torch.float32 else 2) <= 128 else 1)


# ---------------------------------------------------------------------------
# the forward's scheduled loop with masked keys (tiles of two and four pair rows, n a multiple
# of 32, no fully masked row in the workgroup): a random mask, padding (the workgroups with
# rows past the valid length take the general loop, the others stop at the last attended key
# tile), key tiles without an attended key at the start (the softmax reference starts on
# masked scores) and in the middle, rows that attend to a single key.
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("pattern", ["random", "padding", "first_dead", "middle_dead", "one_key"])
@pytest.mark.parametrize("n,h,d", [(256, 2, 32), (128, 1, 16), (160, 1, 32)])
def test_forward_scheduled_loop_masked(n, h, d, pattern, dtype, monkeypatch):
    lib = _lib.load()
    code = tt._DTYPE_CODE[dtype]
    g = torch.Generator().manual_seed(3 * n + d)
    q, k, v, b, m = orc.gen_tensors(n, d, h, pattern == "random", "cpu", torch.float32, 1, 1.0, generator=g)
    if pattern == "random":
        m[:, :, 0] &= ~m.all(dim=-1)  # (no fully masked row)
    elif pattern == "padding":
        valid = n - 37
        m[:, valid:, :] = True
        m[:, :, valid:] = True
    elif pattern == "first_dead":
        m[:, :, :64] = True
        m[:, 7, 70:] = True  # a row whose attended keys end early
    elif pattern == "middle_dead":
        m[:, :, 64:96] = True
    elif pattern == "one_key":
        m[:] = True
        m[0, torch.arange(n), torch.randint(0, n, (n,), generator=g)] = False
    do = torch.randn(q.shape, generator=g)
    q, k, v, b, m, do = (t.detach().to(DEV) for t in (q, k, v, b, m, do))
    low = [t.to(dtype) for t in (q, k, v, b)]
    ref = orc.forward_backward(*(t.float() for t in low), m, do.to(dtype).float())
    pt = orc.forward_backward(*low, m, do.to(dtype))
    scheduled = [t for t in range(lib.trifast_num_tiles(_lib.KERNEL_FWD)) if t >= 6 and lib.trifast_supports(_lib.KERNEL_FWD, t, n, h, d, code)]
    assert len(scheduled) == 2, "tiles 6 and 7 are the forward's scheduled loop"
    for tile in scheduled:
        monkeypatch.setattr(tuner, "pick", lambda kern, n_, h_, d_, dt, launch, extra_cost=None, tile=tile:
                            tile if kern == _lib.KERNEL_FWD else lib.trifast_default_tile(kern, n_, h_, d_, code))
        out = kernel_fwd_bwd(*low, m, do.to(dtype))
        tag = f"fwd tile {tile} n={n} d={d} {pattern} {dtype}"
        check_all(out, pt, ref, dtype, tag, directions=False)
        check_lse(low, m, dtype, tag)


# ---------------------------------------------------------------------------
# structured masks through the default tiles of every kernel, all dtypes and head dims:
# key tiles without an attended key at the start of every row (the online softmax must not
# take the mask value for its reference: exp2 of the rounding error of two numbers of the
# mask value's size is +inf for d = 16 and 64), in the middle, rows with a single attended
# key, padding; ragged and whole numbers of tiles.
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16], ids=["f32", "bf16", "f16"])
@pytest.mark.parametrize("pattern", ["padding", "first_dead", "middle_dead", "one_key"])
@pytest.mark.parametrize("n,h,d", [(96, 1, 16), (130, 2, 32), (256, 1, 64), (200, 1, 128)])
def test_structured_masks(n, h, d, pattern, dtype):
    g = torch.Generator().manual_seed(11 * n + d)
    q, k, v, b, m = orc.gen_tensors(n, d, h, False, "cpu", torch.float32, 1, 1.0, generator=g)
    if pattern == "padding":
        valid = n - 37
        m[:, valid:, :] = True
        m[:, :, valid:] = True
    elif pattern == "first_dead":
        m[:, :, :64] = True
        m[:, 7, 70:] = True
    elif pattern == "middle_dead":
        m[:, :, 32:64] = True
    elif pattern == "one_key":
        m[:] = True
        m[0, torch.arange(n), torch.randint(0, n, (n,), generator=g)] = False
    do = torch.randn(q.shape, generator=g)
    q, k, v, b, m, do = (t.detach().to(DEV) for t in (q, k, v, b, m, do))
    low = [t.to(dtype) for t in (q, k, v, b)]
    ref = orc.forward_backward(*(t.float() for t in low), m, do.to(dtype).float())
    pt = orc.forward_backward(*low, m, do.to(dtype))
    out = kernel_fwd_bwd(*low, m, do.to(dtype))
    tag = f"n={n} h={h} d={d} {pattern} {dtype}"
    # (a row with a single attended key has P = 1 there: dq, dk and db are exactly zero, as the
    # difference of terms dP and delta of size 10 to 40 each: the fp32 bound is taken against 16)
    check_all(out, pt, ref, dtype, tag, directions=False, rel_floor=16.0 if pattern == "one_key" else 1e-30)
    check_lse(low, m, dtype, tag)


# ---------------------------------------------------------------------------
# seeded mixtures: shape, dtype, batch, layout (contiguous, i<->j transposed views, the
# heads-interleaved [b, n, n, h, d] storage of a projection seen as [b, h, n, n, d]) and a
# structured mask per batch element (padding to its own length, a band, blocks on the
# diagonal, dead key ranges, dead leading keys per row), through the default tiles.
# ---------------------------------------------------------------------------
def _structured_mask(kind, bs, n, g):
    m = torch.zeros(bs, n, n, dtype=torch.bool)
    idx = torch.arange(n)
    for bi in range(bs):
        if kind == "padding":
            valid = int(torch.randint(max(1, n // 2), n + 1, (1,), generator=g))
            m[bi, valid:, :] = True
            m[bi, :, valid:] = True
        elif kind == "band":
            w = int(torch.randint(1, max(2, n // 3), (1,), generator=g))
            m[bi] = (idx[:, None] - idx[None, :]).abs() > w
        elif kind == "blocks":
            size = int(torch.randint(8, max(9, n // 2), (1,), generator=g))
            m[bi] = (idx[:, None] // size) != (idx[None, :] // size)
        elif kind == "dead_ranges":
            for _ in range(3):
                lo = int(torch.randint(0, n, (1,), generator=g))
                m[bi, :, lo:lo + int(torch.randint(1, 80, (1,), generator=g))] = True
            m[bi, :, int(torch.randint(0, n, (1,), generator=g))] = False  # (every row keeps a key)
        elif kind == "leading":
            first = torch.randint(0, n, (n,), generator=g)
            m[bi] = idx[None, :] < first[:, None]
    return m


@pytest.mark.parametrize("seed", range(30))
def test_seeded_mixtures(seed):
    g = torch.Generator().manual_seed(9000 + seed)
    pick = lambda xs: xs[int(torch.randint(0, len(xs), (1,), generator=g))]
    n = int(torch.randint(33, 420, (1,), generator=g))
    if pick([0, 1]):
        n = n // 32 * 32  # (whole key tiles: the scheduled loops)
    h, d, bs = pick([1, 2, 3]), pick([16, 32, 64]), pick([1, 2])
    dtype = pick([torch.bfloat16, torch.float16, torch.float32])
    kind = pick(["padding", "band", "blocks", "dead_ranges", "leading"])
    layout = pick(["contiguous", "transposed", "heads_interleaved"])
    q, k, v, b, _ = orc.gen_tensors(n, d, h, False, "cpu", torch.float32, bs, 1.0, generator=g)
    m = _structured_mask(kind, bs, n, g)
    do = torch.randn(q.shape, generator=g)
    q, k, v, b, m, do = (t.detach().to(DEV) for t in (q, k, v, b, m, do))
    low = [t.to(dtype) for t in (q, k, v, b)]
    do = do.to(dtype)
    if layout == "transposed":
        # the same values behind views whose i and j strides are swapped
        low = [t.transpose(2, 3).contiguous().transpose(2, 3) for t in low[:3]] + [low[3].transpose(-1, -2).contiguous().transpose(-1, -2)]
    elif layout == "heads_interleaved":
        low = [t.permute(0, 2, 3, 1, 4).contiguous().permute(0, 3, 1, 2, 4) for t in low[:3]] + [low[3].permute(0, 2, 3, 1).contiguous().permute(0, 3, 1, 2)]
    chunk = 64 if n > 300 else None
    ref = oracle_fwd_bwd(*(t.float() for t in low), m, do.float(), chunk)
    pt = oracle_fwd_bwd(*low, m, do, chunk)
    out = kernel_fwd_bwd(*low, m, do)
    tag = f"seed {seed}: n={n} h={h} d={d} bs={bs} {dtype} {kind} {layout}"
    # (rows with one attended key give gradients that are zero by cancellation: see test_structured_masks)
    check_all(out, pt, ref, dtype, tag, directions=False, rel_floor=16.0 if kind in ("band", "blocks", "leading") else 1e-30)
    check_lse(low, m, dtype, tag)


# ---------------------------------------------------------------------------
# more than 32 key tiles with the first 32 of them plain: the bitmaps over the key tiles are
# 64-bit words put together from two 32-bit halves, and a low half with its top bit set once
# spilled into the high half (tiles 32.. then passed for plain and live).  Padding at n = 1088:
# tile 31 has no masked key, tile 33 has; the forward and the dq kernel (three-kernel backward
# forced in the second pass) read those bitmaps.  At n = 2112 a bitmap is two words.
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("n,valid", [(1088, 1060), (2112, 2090)], ids=["34_tiles", "66_tiles"])
def test_key_tile_bitmaps_past_32_tiles(n, valid, monkeypatch):
    lib = _lib.load()
    h, d, dtype = 1, 32, torch.bfloat16
    code = tt._DTYPE_CODE[dtype]
    g = torch.Generator().manual_seed(n)
    q, k, v, b, m = orc.gen_tensors(n, d, h, False, "cpu", torch.float32, 1, 1.0, generator=g)
    m[:, valid:, :] = True
    m[:, :, valid:] = True
    if n > 2048:
        # (two 64-bit words per bitmap) a row without an attended key in the first word's tiles,
        # and one whose attended keys end in the first word
        m[:, 9, :2050] = True
        m[:, 70, 1000:] = True
    do = torch.randn(q.shape, generator=g)
    q, k, v, b, m, do = (t.detach().to(DEV) for t in (q, k, v, b, m, do))
    low = [t.to(dtype) for t in (q, k, v, b)]
    ref = oracle_fwd_bwd(*(t.float() for t in low), m, do.to(dtype).float(), 64)
    pt = oracle_fwd_bwd(*low, m, do.to(dtype), 64)
    out = kernel_fwd_bwd(*low, m, do.to(dtype))
    check_all(out, pt, ref, dtype, f"n={n} padding to {valid}, default tiles", directions=False)
    check_lse(low, m, dtype, f"n={n} padding to {valid}")
    # the same with the dq and dk/dv kernels instead of the row-resident one
    kv = next(t for t in range(lib.trifast_num_tiles(_lib.KERNEL_BWD_KV))
              if not lib.trifast_bwd_kv_tile_writes_dq(t) and lib.trifast_supports(_lib.KERNEL_BWD_KV, t, n, h, d, code))
    real_pick = tuner.pick
    monkeypatch.setattr(tuner, "pick", lambda kern, *a, **kw: kv if kern == _lib.KERNEL_BWD_KV else real_pick(kern, *a, **kw))
    out = kernel_fwd_bwd(*low, m, do.to(dtype))
    check_all(out, pt, ref, dtype, f"n={n} padding to {valid}, three-kernel backward", directions=False)


# ---------------------------------------------------------------------------
# the db kernel's pipelined walk of plain rows (blocks whose waves own two key tiles) and
# its hand-over to the general loop at the first row that is not plain: no mask at all,
# padding (keys and rows past a valid length), one masked row in the middle, a masked row
# near the start (nothing is pipelined then).  Several row chunks at these sizes.
# Each such tile must give db within the reference's bound of the oracle, and bit-identical
# to the 16-wave tile where every block is plain (same order of the sum over the rows, same
# arithmetic per element).
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("pattern", ["none", "padding", "middle", "early"])
@pytest.mark.parametrize("n,h,d", [(300, 2, 32), (256, 1, 16), (200, 1, 32)])
def test_db_pipelined_rows(n, h, d, pattern, dtype, monkeypatch):
    lib = _lib.load()
    code = tt._DTYPE_CODE[dtype]
    g = torch.Generator().manual_seed(n + d)
    q, k, v, b, m = orc.gen_tensors(n, d, h, False, "cpu", torch.float32, 1, 1.0, generator=g)
    if pattern == "padding":
        valid = n - 37
        m[:, valid:, :] = True
        m[:, :, valid:] = True
    elif pattern == "middle":
        m[:, n // 2, :] = torch.rand(n, generator=g) < 0.3
        m[:, n // 2 + 9, :] = True
    elif pattern == "early":
        m[:, 5, 1::2] = True
    do = torch.randn(q.shape, generator=g)
    q, k, v, b, m, do = (t.detach().to(DEV) for t in (q, k, v, b, m, do))
    low = [t.to(dtype) for t in (q, k, v, b)]
    ref = orc.forward_backward(*(t.float() for t in low), m, do.to(dtype).float())
    pt = orc.forward_backward(*low, m, do.to(dtype))
    infos = {t: _lib.tile_info(_lib.KERNEL_BWD_B, t) for t in range(lib.trifast_num_tiles(_lib.KERNEL_BWD_B))}
    two_key_tiles = [t for t, i in infos.items() if i["BLOCK_K"] // 32 == 2 * (i["num_waves"] // (i["BLOCK_J"] // 32))
                     and lib.trifast_supports(_lib.KERNEL_BWD_B, t, n, h, d, code)]
    plain_tile = max(t for t, i in infos.items() if i["num_waves"] == 16)
    assert len(two_key_tiles) >= 2, infos
    results = {}
    for tile in [plain_tile] + two_key_tiles:
        monkeypatch.setattr(tuner, "pick", lambda kern, n_, h_, d_, dt, launch, extra_cost=None, tile=tile:
                            tile if kern == _lib.KERNEL_BWD_B else lib.trifast_default_tile(kern, n_, h_, d_, code))
        out = kernel_fwd_bwd(*low, m, do.to(dtype))
        check_all(out, pt, ref, dtype, f"db tile {tile} n={n} d={d} {pattern} {dtype}", directions=False)
        results[tile] = out[NAMES.index("db")] if "db" in NAMES else out[-1]
    for tile in two_key_tiles:
        if pattern == "none" and n % 128 == 0:
            # every block plain: the same arithmetic in the same order
            assert torch.equal(results[tile], results[plain_tile]), f"db of tile {tile} differs from tile {plain_tile} ({pattern}, n={n})"
        else:
            # (-lse enters through a matrix instruction where the other tile adds it in the exponent)
            err = (results[tile].float() - results[plain_tile].float()).abs().max().item()
            assert err <= 2.0 ** -6 * results[plain_tile].float().abs().max().item(), f"db of tile {tile} vs tile {plain_tile}: {err} ({pattern}, n={n})"


# ---------------------------------------------------------------------------
# the row-resident backward (dq, dk, dv in one pass) at every size class it has:
# 2 to 8 key tiles per wave, ragged sizes, masked keys, fully masked rows
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("n,h,d", [(131, 2, 32), (300, 1, 32), (450, 1, 32), (520, 1, 32), (700, 1, 32), (800, 1, 32), (1000, 1, 32), (300, 1, 64), (450, 1, 64), (190, 1, 16), (330, 1, 16)])
def test_row_resident_backward_size_classes(n, h, d, dtype, monkeypatch):
    lib = _lib.load()
    code = tt._DTYPE_CODE[dtype]
    row_tiles = [t for t in range(lib.trifast_num_tiles(_lib.KERNEL_BWD_KV))
                 if lib.trifast_bwd_kv_tile_writes_dq(t) and lib.trifast_supports(_lib.KERNEL_BWD_KV, t, n, h, d, code)]
    assert row_tiles, "no row-resident tile supports this shape"
    tile = row_tiles[0]  # the smallest one that holds the row
    g = torch.Generator().manual_seed(n + d)
    q, k, v, b, m = orc.gen_tensors(n, d, h, True, "cpu", torch.float32, 1, 1.0, generator=g)
    m[:, 3, :] = True          # a fully masked row
    m[:, 5, : n - 7] = True    # a row that attends to its last keys only (dead key tiles)
    m[:, 7, :] = False         # a row with no masked key
    do = torch.randn(q.shape, generator=g)
    q, k, v, b, m, do = (t.detach().to(DEV) for t in (q, k, v, b, m, do))
    low = [t.to(dtype) for t in (q, k, v, b)]
    chunk = 64 if n > 400 else None
    ref = oracle_fwd_bwd(*(t.float() for t in low), m, do.to(dtype).float(), chunk)
    pt = oracle_fwd_bwd(*low, m, do.to(dtype), chunk)
    real_pick = tuner.pick
    monkeypatch.setattr(tuner, "pick", lambda kern, *a, **kw: tile if kern == _lib.KERNEL_BWD_KV else real_pick(kern, *a, **kw))
    kern_out = kernel_fwd_bwd(*low, m, do.to(dtype))
    check_all(kern_out, pt, ref, dtype, f"row-resident tile {tile} n={n} d={d} {dtype}", directions=False)
    again = kernel_fwd_bwd(*low, m, do.to(dtype))
    for name, x, y in zip(NAMES, kern_out, again):
        assert torch.equal(x, y), f"{name} differs between two runs"
    # masked keys of partially masked rows get exactly zero dk, dv
    assert kern_out[2][:, :, 5, : n - 7].abs().max() == 0 and kern_out[3][:, :, 5, : n - 7].abs().max() == 0


# ---------------------------------------------------------------------------
# golden fixtures (inputs and answers fixed on disk)
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("name", ["tiny_n6_h2_d16", "plumb_n16_h4_d32", "ragged_n19_h2_d32"])
def test_golden_fixtures_fp32(name):
    z = np.load(GOLDEN / f"{name}.npz")
    t = {key: torch.from_numpy(z[key]).to(DEV) for key in z.files}
    q, k, v, b = (t[x].clone().requires_grad_(True) for x in ("q", "k", "v", "bias"))
    o, lse = tt._triangle_attention(q, k, v, b, t["mask"])
    o.backward(t["do"])
    for key, got in (("o", o.detach()), ("dq", q.grad), ("dk", k.grad), ("dv", v.grad), ("db", b.grad)):
        torch.testing.assert_close(got, t[key], rtol=2e-5, atol=2e-5, msg=f"{name} {key}")
    # the saved log-sum-exp is a public output; fully masked rows report finfo.min
    torch.testing.assert_close(lse, t["lse"], rtol=1e-5, atol=1e-5, msg=f"{name} lse")


# ---------------------------------------------------------------------------
# the benchmark configurations at their full sizes
# ---------------------------------------------------------------------------
def _run_config(name, chunk):
    dtype = bench.WORKLOADS[name][0]
    q, k, v, bias, mask, do = bench.make_workload(name, DEV)
    kern = kernel_fwd_bwd(q, k, v, bias, mask, do)
    ref = oracle_fwd_bwd(q.float(), k.float(), v.float(), bias.float(), mask, do.float(), chunk)
    pt = oracle_fwd_bwd(q, k, v, bias, mask, do, chunk) if dtype != torch.float32 else ref
    return q, k, v, bias, mask, do, kern, pt, ref


def test_config_c1_fp32_plumbing():
    *_, kern, pt, ref = _run_config("C1", None)
    check_all(kern, pt, ref, torch.float32, "C1")


def test_config_c2_bf16_dense():
    *_, kern, pt, ref = _run_config("C2", 64)
    check_all(kern, pt, ref, torch.bfloat16, "C2")


def test_config_c3_padding_mask_and_fully_masked_rows():
    q, k, v, bias, mask, do, kern, pt, ref = _run_config("C3", 32)
    check_all(kern, pt, ref, torch.bfloat16, "C3")
    full = mask.all(dim=-1)[0]  # rows i >= L: every key masked
    assert full.any() and not full.all()
    # reported separately so a disagreement on those rows cannot be averaged away:
    # they attend uniformly (o = mean of v) and do carry gradient
    for name, x, p, r in zip(NAMES[:4], kern[:4], pt[:4], ref[:4]):
        a, b_ = orc.compare_values(x[:, :, full], p[:, :, full], r[:, :, full], f"C3 fully-masked rows {name}", eps=1e-3)
        print(f"C3 fully-masked rows {name}: {a:.2e} (pt {b_:.2e})")
    o_full = kern[0][:, :, full].float()
    want = v[:, :, full].float().mean(dim=3, keepdim=True).expand_as(o_full)
    assert (o_full - want).abs().max() < 2e-2
    assert kern[1][:, :, full].float().abs().max() > 0  # dq of fully masked rows is not zero
    # padded keys of attended rows get exactly zero dk / dv
    L = int((~full).sum())
    assert kern[2][:, :, :L, L:].abs().max() == 0 and kern[3][:, :, :L, L:].abs().max() == 0


@pytest.mark.parametrize("name", ["C4a", "C4b"])
def test_config_c4_fp16_transposed_views(name):
    q, k, v, bias, mask, do, kern, pt, ref = _run_config(name, 32)
    assert not q.is_contiguous() and not bias.is_contiguous() and not mask.is_contiguous()
    check_all(kern, pt, ref, torch.float16, name)


def test_config_m_headline_shape():
    *_, kern, pt, ref = _run_config("M", 32)
    check_all(kern, pt, ref, torch.bfloat16, "M")


def test_config_c5_large_outliers_memory_and_lse():
    name = "C5"
    q, k, v, bias, mask, do = bench.make_workload(name, DEV)
    b, h, n, _, d = q.shape
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats()
    base = torch.cuda.memory_allocated()
    qq, kk, vv, bb = (t.detach().requires_grad_(True) for t in (q, k, v, bias))
    o, lse = tt._triangle_attention(qq, kk, vv, bb, mask)
    o.backward(do)
    torch.cuda.synchronize()
    extra = torch.cuda.max_memory_allocated() - base
    logits_bytes = b * h * n**3 * 2
    # o + lse + 3 grads + db + delta workspace + temporaries: O(n^2 d), nowhere near n^3
    assert extra < 8 * q.numel() * q.element_size(), extra
    assert extra < logits_bytes / 4
    assert torch.isfinite(lse).all()
    kern = (o.detach(), qq.grad, kk.grad, vv.grad, bb.grad)
    ref = orc.forward_backward_chunked(q.float(), k.float(), v.float(), bias.float(), mask, do.float(), chunk=16)
    pt = orc.forward_backward_chunked(q, k, v, bias, mask, do, chunk=16)
    check_all(kern, pt, ref, torch.bfloat16, "C5")
    lse_ref = torch.cat([orc.lse_reference(q[:, :, i0:i0 + 64].float(), k[:, :, i0:i0 + 64].float(), bias.float(), mask[:, i0:i0 + 64]) for i0 in range(0, n, 64)], dim=2)
    # the row sum is taken over the bf16-rounded probabilities that feed the P.V MFMA (so o is
    # normalised by exactly what was accumulated): lse carries up to 2^-9 relative error of the sum
    assert (lse - lse_ref).abs().max() < 2.0 ** -8


# ---------------------------------------------------------------------------
# size-independent properties at the headline size
# ---------------------------------------------------------------------------
def test_properties_at_full_size():
    q, k, v, bias, mask, do = bench.make_workload("M", DEV)
    a = kernel_fwd_bwd(q, k, v, bias, mask, do)
    b = kernel_fwd_bwd(q, k, v, bias, mask, do)
    for name, x, y in zip(NAMES, a, b):  # deterministic: bitwise equal run to run
        assert torch.equal(x, y), f"{name} differs between two runs"
    # softmax shift invariance: db sums to ~0 over keys (bf16 rounding of 1024 terms)
    assert a[4].float().sum(dim=-1).abs().max() < 0.5
    # rows of P sum to one: constant v gives constant o
    vc = torch.full_like(v, 0.75)
    oc = trifast_amd.triangle_attention(q, k, vc, bias, mask)
    assert (oc.float() - 0.75).abs().max() < 4e-3
    # adding a per-(h, j) constant to the bias changes nothing
    shift = torch.randn(1, 4, q.shape[2], 1, device=DEV).to(bias.dtype)
    o2 = trifast_amd.triangle_attention(q, k, v, (bias.float() + shift.float()).to(bias.dtype), mask)
    assert (o2.float() - a[0].float()).abs().max() < 5e-2
