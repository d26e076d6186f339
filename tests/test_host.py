"""Host-side logic that needs no GPU: operator schema and fake kernels, input
validation, stride handling, the tile cache and the tune CLI."""

import json

import pytest
import torch

import trifast
import trifast_amd
from trifast_amd import _lib, tune, tuner
from trifast_amd import torch as tt


def meta_inputs(b=1, h=2, n=8, d=16, dtype=torch.bfloat16):
    q = torch.empty(b, h, n, n, d, device="meta", dtype=dtype)
    bias = torch.empty(b, h, n, n, device="meta", dtype=dtype)
    mask = torch.empty(b, n, n, device="meta", dtype=torch.bool)
    return q, q, q, bias, mask


def test_public_surface_matches_reference_names():
    # reference src/trifast/__init__.py:1-3, src/trifast/torch.py:17,68,185,210,220
    assert trifast.triangle_attention is trifast_amd.triangle_attention
    import trifast.torch as rt

    for name in ("triangle_attention", "_triangle_attention", "triangle_attention_bwd", "backwards", "setup_context"):
        assert hasattr(rt, name)
    assert hasattr(torch.ops.trifast, "triangle_attention")
    assert hasattr(torch.ops.trifast, "triangle_attention_backward")
    from trifast.utils import clone_and_clear_grad, disable_tf32, enable_tf32, gen_tensors  # noqa: F401


def test_fake_kernels_give_reference_shapes():
    q, k, v, b, m = meta_inputs()
    o, lse = torch.ops.trifast.triangle_attention(q, k, v, b, m)
    assert o.shape == q.shape and o.dtype == q.dtype
    assert lse.shape == (1, 2, 8, 8) and lse.dtype == torch.float32
    outs = torch.ops.trifast.triangle_attention_backward(o, q, k, v, b, o, lse, m)
    assert [t.shape for t in outs] == [q.shape, q.shape, q.shape, b.shape, m.shape]
    assert outs[4].dtype == torch.bool


def test_cpu_tensors_are_rejected_not_computed():
    g = torch.Generator().manual_seed(0)
    q = torch.randn(1, 1, 4, 4, 16, generator=g)
    b = torch.randn(1, 1, 4, 4, generator=g)
    m = torch.zeros(1, 4, 4, dtype=torch.bool)
    with pytest.raises(RuntimeError, match="GPU only"):
        trifast_amd.triangle_attention(q, q, q, b, m)


@pytest.mark.parametrize(
    "mutate, err",
    [
        (lambda a: a.__setitem__(0, a[0][..., :3, :, :]), ValueError),      # not square
        (lambda a: a.__setitem__(3, a[3][..., :3]), ValueError),            # bias shape
        (lambda a: a.__setitem__(4, a[4].to(torch.uint8)), TypeError),      # mask dtype
        (lambda a: a.__setitem__(1, a[1].to(torch.float16)), TypeError),    # mixed dtypes
        (lambda a: a.__setitem__(0, a[0][0]), ValueError),                  # rank
    ],
)
def test_input_validation(mutate, err):
    q = torch.zeros(1, 2, 4, 4, 16, dtype=torch.bfloat16)
    args = [q, q.clone(), q.clone(), torch.zeros(1, 2, 4, 4, dtype=torch.bfloat16), torch.zeros(1, 4, 4, dtype=torch.bool)]
    mutate(args)
    with pytest.raises(err):
        tt._check_inputs(*args)


def test_vector_ready_keeps_transposed_views_and_copies_the_rest():
    x = torch.zeros(1, 2, 8, 8, 16, dtype=torch.bfloat16)
    assert tt._vector_ready(x) is x
    xt = x.transpose(2, 3)
    assert tt._vector_ready(xt) is xt                       # i<->j view: read in place
    assert tt._vector_ready(x[..., ::2]).is_contiguous()    # d stride 2: copied
    ones = torch.ones((), dtype=torch.bfloat16).expand(1, 2, 8, 8, 16)
    assert tt._vector_ready(ones).is_contiguous()           # stride-0 upstream gradient
    assert tt._strides(torch.zeros(1, 2, 8, 8, 16))[0] == 0  # size-1 dims report stride 0


def test_key_and_closest_n():
    assert tuner.closest_n(1) == 1 and tuner.closest_n(17) == 32 and tuner.closest_n(1024) == 1024 and tuner.closest_n(1025) == 2048
    assert tuner.make_key(191, 4, 32, torch.bfloat16) == "4_32_256_torch.bfloat16"


def test_tile_cache_roundtrip_and_corruption(tmp_path, monkeypatch, capsys):
    monkeypatch.setenv("TRIFAST_CONFIG_DIR", str(tmp_path))
    monkeypatch.setattr(tuner, "_device_tag", lambda device=None: "Test-GPU_9-5")
    tuner.reset()
    c = tuner.TileCache(_lib.KERNEL_FWD)
    assert c.cache_file == tmp_path / "_fwd_Test-GPU_9-5.json"
    c.cache["4_32_1024_torch.bfloat16"] = 1
    c.write()
    raw = json.loads(c.cache_file.read_text())
    assert raw["4_32_1024_torch.bfloat16"]["tile"] == 1
    assert raw["4_32_1024_torch.bfloat16"]["kwargs"] == {k: v for k, v in _lib.tile_info(0, 1).items() if k != "num_waves"}
    assert tuner.TileCache(_lib.KERNEL_FWD).cache == {"4_32_1024_torch.bfloat16": 1}
    # an entry from another tile table is dropped, a corrupt file is reported and ignored
    raw["4_32_1024_torch.bfloat16"]["kwargs"]["BLOCK_J"] = 12345
    c.cache_file.write_text(json.dumps(raw))
    assert tuner.TileCache(_lib.KERNEL_FWD).cache == {}
    c.cache_file.write_text("{not json")
    assert tuner.TileCache(_lib.KERNEL_FWD).cache == {}
    assert "Could not load autotune cache" in capsys.readouterr().out
    tuner.reset()


def test_pick_without_autotune_uses_library_heuristic(monkeypatch):
    monkeypatch.setenv("TRIFAST_AUTOTUNE", "0")
    monkeypatch.delenv("TRIFAST_FORCE_TUNE", raising=False)
    called = []
    t = tuner.pick(_lib.KERNEL_FWD, 1024, 4, 32, torch.bfloat16, called.append)
    assert t == _lib.load().trifast_default_tile(0, 1024, 4, 32, _lib.BF16) and called == []


def test_pick_times_every_supported_tile_on_a_miss(tmp_path, monkeypatch):
    monkeypatch.setenv("TRIFAST_CONFIG_DIR", str(tmp_path))
    monkeypatch.setenv("TRIFAST_AUTOTUNE", "1")
    monkeypatch.delenv("TRIFAST_FORCE_TUNE", raising=False)
    monkeypatch.setattr(tuner, "_device_tag", lambda device=None: "Test-GPU_9-5")
    fake_ms = {0: 3.0, 1: 1.0, 2: 5.0, 3: 2.0}
    monkeypatch.setattr(tuner, "_time_launch", lambda launch, tile, **kw: fake_ms.get(tile, 9.0))
    tuner.reset()
    assert tuner.pick(_lib.KERNEL_FWD, 300, 4, 32, torch.bfloat16, lambda t: None) == 1
    assert json.loads((tmp_path / "_fwd_Test-GPU_9-5.json").read_text())["4_32_512_torch.bfloat16"]["tile"] == 1
    # a hit does not time again
    monkeypatch.setattr(tuner, "_time_launch", lambda *a, **k: pytest.fail("re-tuned on a cache hit"))
    assert tuner.pick(_lib.KERNEL_FWD, 400, 4, 32, torch.bfloat16, lambda t: None) == 1
    # TRIFAST_FORCE_TUNE re-tunes even on a hit
    monkeypatch.setenv("TRIFAST_FORCE_TUNE", "yes")
    monkeypatch.setattr(tuner, "_time_launch", lambda launch, tile, **kw: float(tile != 3))
    assert tuner.pick(_lib.KERNEL_FWD, 400, 4, 32, torch.bfloat16, lambda t: None) == 3
    tuner.reset()


def test_pick_prefers_the_default_tile_on_a_near_tie(tmp_path, monkeypatch):
    monkeypatch.setenv("TRIFAST_CONFIG_DIR", str(tmp_path))
    monkeypatch.setenv("TRIFAST_AUTOTUNE", "1")
    monkeypatch.delenv("TRIFAST_FORCE_TUNE", raising=False)
    monkeypatch.setattr(tuner, "_device_tag", lambda device=None: "Test-GPU_9-5")
    default = _lib.load().trifast_default_tile(_lib.KERNEL_BWD_KV, 1024, 4, 32, _lib.BF16)
    other = next(t for t in tuner.supported_tiles(_lib.KERNEL_BWD_KV, 1024, 4, 32, torch.bfloat16) if t != default)
    # 1 % faster is within the scatter of the timings: the default stays
    monkeypatch.setattr(tuner, "_time_launch", lambda launch, tile, **kw: 0.99 if tile == other else (1.0 if tile == default else 5.0))
    tuner.reset()
    assert tuner.pick(_lib.KERNEL_BWD_KV, 1024, 4, 32, torch.bfloat16, lambda t: None) == default
    # 10 % faster replaces it
    monkeypatch.setenv("TRIFAST_FORCE_TUNE", "1")
    monkeypatch.setattr(tuner, "_time_launch", lambda launch, tile, **kw: 0.9 if tile == other else (1.0 if tile == default else 5.0))
    assert tuner.pick(_lib.KERNEL_BWD_KV, 1024, 4, 32, torch.bfloat16, lambda t: None) == other
    tuner.reset()


def test_pick_charges_a_tile_what_it_leaves_to_other_kernels(tmp_path, monkeypatch):
    """dk/dv tiles that do not also produce dq are charged the dq kernel's time: the
    row-resident tile wins although its own launch is the longest."""
    monkeypatch.setenv("TRIFAST_CONFIG_DIR", str(tmp_path))
    monkeypatch.setenv("TRIFAST_AUTOTUNE", "1")
    monkeypatch.delenv("TRIFAST_FORCE_TUNE", raising=False)
    monkeypatch.setattr(tuner, "_device_tag", lambda device=None: "Test-GPU_9-5")
    lib = _lib.load()
    tiles = tuner.supported_tiles(_lib.KERNEL_BWD_KV, 1024, 4, 32, torch.bfloat16)
    fused = [t for t in tiles if lib.trifast_bwd_kv_tile_writes_dq(t)]
    assert len(fused) == 1 and len(tiles) > 1  # 1024 keys: only the largest row-resident tile fits
    monkeypatch.setattr(tuner, "_time_launch", lambda launch, tile, **kw: 2.1 if tile in fused else 1.6)
    tuner.reset()
    assert tuner.pick(_lib.KERNEL_BWD_KV, 1024, 4, 32, torch.bfloat16, lambda t: None) not in fused
    monkeypatch.setenv("TRIFAST_FORCE_TUNE", "1")
    extra = lambda t: 0.0 if lib.trifast_bwd_kv_tile_writes_dq(t) else 1.4
    assert tuner.pick(_lib.KERNEL_BWD_KV, 1024, 4, 32, torch.bfloat16, lambda t: None, extra_cost=extra) == fused[0]
    tuner.reset()


def test_row_resident_tiles_in_the_library_tables():
    """The row-resident kernel appears as the last eight tiles of the dk/dv family: seven for rows
    of up to 256, 384, ..., 1024 keys, for 16-bit inputs, and one that runs longer rows (up to
    8192 keys at head dim 32) in passes of 1024 keys; they are the default where they are fastest."""
    lib = _lib.load()
    nt = lib.trifast_num_tiles(_lib.KERNEL_BWD_KV)
    fused = [t for t in range(nt) if lib.trifast_bwd_kv_tile_writes_dq(t)]
    assert fused == list(range(nt - 8, nt))
    assert not lib.trifast_bwd_kv_tile_writes_dq(-1) and not lib.trifast_bwd_kv_tile_writes_dq(nt)
    passes = fused[7]
    sup = lambda n, d, code: bool(lib.trifast_supports(_lib.KERNEL_BWD_KV, passes, n, 4, d, code))
    assert sup(1025, 32, _lib.BF16) and sup(8192, 32, _lib.F16) and sup(2047, 32, _lib.BF16)
    assert not sup(1024, 32, _lib.BF16) and not sup(8193, 32, _lib.BF16)
    assert not sup(2048, 64, _lib.BF16) and not sup(2048, 16, _lib.BF16) and not sup(2048, 32, _lib.F32)
    # its low parts of dq live in the workspace tail, which is at least one more 16-bit tensor
    ws = lambda n, d: lib.trifast_bwd_workspace_bytes(1, 4, n, d, _lib.BF16)
    assert ws(2048, 32) - ws(2048, 64) >= 4 * 2048 * 2048 * 32 * 2 - 4 * 4 * 2048 * 2048 * 4
    for t, keys in zip(fused[:7], (256, 384, 512, 640, 768, 896, 1024)):
        assert _lib.tile_info(_lib.KERNEL_BWD_KV, t)["BLOCK_K"] == keys
        assert lib.trifast_supports(_lib.KERNEL_BWD_KV, t, keys, 4, 32, _lib.BF16)
        assert lib.trifast_supports(_lib.KERNEL_BWD_KV, t, keys - 37, 2, 32, _lib.F16)
        assert not lib.trifast_supports(_lib.KERNEL_BWD_KV, t, keys + 1, 4, 32, _lib.BF16)
        assert not lib.trifast_supports(_lib.KERNEL_BWD_KV, t, keys, 4, 32, _lib.F32)
        assert not lib.trifast_supports(_lib.KERNEL_BWD_KV, t, keys, 4, 128, _lib.BF16)
    default = lambda n, d, code: lib.trifast_default_tile(_lib.KERNEL_BWD_KV, n, 4, d, code)
    assert default(1024, 32, _lib.BF16) == fused[6] and default(300, 32, _lib.F16) == fused[1] and default(385, 32, _lib.F16) == fused[2]
    assert default(640, 32, _lib.BF16) == fused[3] and default(641, 32, _lib.BF16) == fused[4] and default(896, 32, _lib.BF16) == fused[5]
    assert default(129, 32, _lib.BF16) == fused[0] and default(1025, 32, _lib.BF16) == passes and default(8193, 32, _lib.BF16) not in fused
    # (from the smallest rows on: one launch instead of two; head dim 16 like 32, head dim 64 up to 384 keys)
    assert default(128, 32, _lib.BF16) == fused[0] and default(16, 32, _lib.F16) == fused[0]
    assert default(700, 16, _lib.BF16) == fused[4] and default(1025, 16, _lib.BF16) not in fused
    assert default(300, 64, _lib.F16) == fused[1] and default(385, 64, _lib.F16) not in fused and default(512, 64, _lib.BF16) not in fused
    assert default(512, 32, _lib.F32) not in fused and default(64, 128, _lib.BF16) not in fused


def test_tune_cli_flags_and_sweep():
    p = tune.build_parser()
    a = p.parse_args([])
    assert (a.min_n, a.max_n, a.h, a.d, a.dtype) == (16, 1024, [4], [32], [torch.bfloat16])
    a = p.parse_args(["--min-n", "64", "--max-n", "300", "--dtype", "float16,float32", "--h", "1,4", "--d", "16,64"])
    assert a.h == [1, 4] and a.d == [16, 64] and set(a.dtype) == {torch.float16, torch.float32}
    assert tune.sweep_ns(a.min_n, a.max_n) == [64, 128, 256]
    assert len(tune.valid_dtypes("all")) == 3
    with pytest.raises(SystemExit):
        p.parse_args(["--dtype", "int8"])


def test_equiv_module_matches_the_oracle():
    """``trifast.equiv`` (the reference's public pure-PyTorch functions) gives the
    oracle's numbers, fully masked rows included."""
    from trifast.equiv import attention_reference, triangle_attention_simple
    from oracle import triangle_oracle as orc

    g = torch.Generator().manual_seed(3)
    q, k, v, b, m = orc.gen_tensors(9, 8, 2, True, "cpu", torch.float32, 2, 1.0, generator=g)
    m[:, 4, :] = True
    q, k, v, b = (t.detach() for t in (q, k, v, b))
    torch.testing.assert_close(attention_reference(q, k, v, b, m), orc.attention_reference(q, k, v, b, m), rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(triangle_attention_simple(q, k, v, b, m), orc.triangle_attention_simple(q, k, v, b, m), rtol=1e-6, atol=1e-6)


def test_wide_j_strides_are_copied_and_their_gradients_allocated_contiguous():
    # the kernels address the rows of a tile through 32-bit offsets: a stride between
    # consecutive j of 2^24 bytes or more is not run in place (the library would refuse it)
    t = torch.empty_strided((1, 1, 2, 2, 8), (0, 0, 64, 1 << 24, 1), dtype=torch.bfloat16, device="meta")
    assert tt._vector_ready(t).is_contiguous()
    assert tt._grad_like(t).is_contiguous()
    ok = torch.empty_strided((1, 1, 2, 2, 8), (0, 0, 8, 16, 1), dtype=torch.bfloat16, device="meta")  # transposed view
    assert tt._vector_ready(ok) is ok


def test_equiv_simple_takes_any_number_of_batch_dims():
    from trifast_amd import equiv

    g = torch.Generator().manual_seed(5)
    q, k, v = (torch.randn(2, 3, 2, 5, 5, 4, generator=g) for _ in range(3))
    b = torch.randn(2, 3, 2, 5, 5, generator=g)
    m = torch.rand(2, 3, 5, 5, generator=g) < 0.3
    whole = equiv.triangle_attention_simple(q, k, v, b, m)
    parts = torch.stack([equiv.attention_reference(q[x], k[x], v[x], b[x], m[x]) for x in range(2)])
    assert torch.allclose(whole, parts, atol=1e-6)
    assert torch.allclose(equiv.triangle_attention_simple(q[0, 0], k[0, 0], v[0, 0], b[0, 0], m[0, 0]), whole[0, 0], atol=1e-6)
