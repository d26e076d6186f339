"""The tile tuner and the ``trifast-tune`` CLI on the GPU, with real timing.

Counterpart of the reference's tuning behaviour: on a cache miss every candidate is
benchmarked and the winner persisted (reference src/trifast/autotune.py:110-137), one
JSON file per kernel named ``{kernel}_{device}_{major}-{minor}.json`` with keys
``H_DIM_CLOSESTN_dtype`` (:73-75, :114-120); a later process reloads the file and
hits; ``trifast-tune`` sweeps the powers of two between --min-n and --max-n
(reference src/trifast/tune.py:45-63).
"""

import json

import pytest
import torch

import trifast_amd
from oracle import triangle_oracle as orc
from trifast_amd import _lib, tune, tuner

pytestmark = pytest.mark.gpu

KERNEL_FILES = ("_fwd", "_bwd_q", "_bwd_kv", "_bwd_b")


@pytest.fixture
def tuning_on(tmp_path, monkeypatch):
    monkeypatch.setenv("TRIFAST_CONFIG_DIR", str(tmp_path))
    monkeypatch.setenv("TRIFAST_AUTOTUNE", "1")
    monkeypatch.delenv("TRIFAST_FORCE_TUNE", raising=False)
    tuner.reset()
    yield tmp_path
    # main() sets these in os.environ; monkeypatch restores what it knows about
    monkeypatch.delenv("TRIFAST_FORCE_TUNE", raising=False)
    monkeypatch.delenv("TRIFAST_PRINT_AUTOTUNING", raising=False)
    tuner.reset()


def _parity(n, h=4, d=32, dtype=torch.bfloat16, seed=0):
    g = torch.Generator().manual_seed(seed)
    q, k, v, b, m = orc.gen_tensors(n, d, h, True, "cpu", torch.float32, 1, 1.0, generator=g)
    do = torch.randn(q.shape, generator=g)
    q, k, v, b, m, do = (t.detach().cuda() for t in (q, k, v, b, m, do))
    low = [t.to(dtype).requires_grad_(True) for t in (q, k, v, b)]
    o = trifast_amd.triangle_attention(*low, m)
    o.backward(do.to(dtype))
    kern = (o.detach(), *(t.grad for t in low))
    ref = orc.forward_backward(*(t.detach().float() for t in low), m, do.to(dtype).float())
    pt = orc.forward_backward(*(t.detach() for t in low), m, do.to(dtype))
    for name, x, p, r in zip(("o", "dq", "dk", "dv", "db"), kern, pt, ref):
        assert torch.isfinite(x.float()).all(), name
        orc.compare_values(x, p, r, f"tuned n={n} {name}", eps=orc.DTYPE_EPS[dtype])


def test_tune_cli_writes_cache_that_a_fresh_process_state_hits(tuning_on, monkeypatch, capsys):
    tune.main(["--min-n", "64", "--max-n", "128"])
    out = capsys.readouterr().out
    assert "Tuning: N: 64, H: 4, D: 32" in out and "Tuning: N: 128, H: 4, D: 32" in out
    assert "trifast autotuning for _fwd" in out  # TRIFAST_PRINT_AUTOTUNING is switched on by the CLI
    files = sorted(p.name for p in tuning_on.glob("*.json"))
    tag = tuner._device_tag()
    assert files == sorted(f"{k}_{tag}.json" for k in KERNEL_FILES)
    lib = _lib.load()
    for kernel, name in enumerate(KERNEL_FILES):
        raw = json.loads((tuning_on / f"{name}_{tag}.json").read_text())
        assert sorted(raw) == ["4_32_128_torch.bfloat16", "4_32_64_torch.bfloat16"]
        for key, entry in raw.items():
            assert set(entry) == {"tile", "kwargs", "num_waves"} and set(entry["kwargs"]) == {"BLOCK_J", "BLOCK_K"}
            n = int(key.split("_")[2])
            assert lib.trifast_supports(kernel, entry["tile"], n, 4, 32, _lib.BF16) == 1

    # a new process state: caches are read back from the files, nothing is timed again
    monkeypatch.delenv("TRIFAST_FORCE_TUNE", raising=False)
    tuner.reset()
    timed = []
    monkeypatch.setattr(tuner, "_time_launch", lambda launch, tile, **kw: timed.append(tile) or 1.0)
    for kernel, name in enumerate(KERNEL_FILES):
        cache = tuner.TileCache(kernel)
        raw = json.loads((tuning_on / f"{name}_{tag}.json").read_text())
        assert cache.cache == {key: entry["tile"] for key, entry in raw.items()}
    for n in (64, 100, 128):  # 100 shares the bucket of 128
        _parity(n)
    assert timed == []


def test_miss_times_on_first_call_then_hits(tuning_on, monkeypatch):
    calls = []
    real = tuner._time_launch
    monkeypatch.setattr(tuner, "_time_launch", lambda launch, tile, **kw: calls.append(tile) or real(launch, tile, **kw))
    _parity(48, h=2, d=32, seed=1)  # miss: every kernel with more than one candidate is timed
    assert len(calls) >= 4
    assert len(list(tuning_on.glob("*.json"))) == 4
    n_first = len(calls)
    _parity(48, h=2, d=32, seed=2)  # hit
    assert len(calls) == n_first
    # the backward kernels are timed on a workspace that _bwd_q has filled: outputs stay finite
    # even when only the later kernels miss
    tuner.reset()
    tag = tuner._device_tag()
    for name in ("_bwd_kv", "_bwd_b"):
        (tuning_on / f"{name}_{tag}.json").unlink()
    _parity(48, h=2, d=32, seed=3)
    assert len(calls) > n_first


def test_no_timing_under_stream_capture(tuning_on):
    """A cache miss during HIP-graph capture takes the heuristic tile: timing would
    synchronise and invalidate the capture."""
    n, h, d = 64, 1, 32
    q, k, v = (torch.randn(1, h, n, n, d, device="cuda", dtype=torch.bfloat16) for _ in range(3))
    b = torch.randn(1, h, n, n, device="cuda", dtype=torch.bfloat16)
    m = torch.zeros(1, n, n, device="cuda", dtype=torch.bool)
    eager_env = trifast_amd.triangle_attention(q, k, v, b, m)  # tunes key 1_32_64 outside capture
    q2, k2, v2 = (torch.randn(1, h, 2 * n, 2 * n, d, device="cuda", dtype=torch.bfloat16) for _ in range(3))
    b2 = torch.randn(1, h, 2 * n, 2 * n, device="cuda", dtype=torch.bfloat16)
    m2 = torch.zeros(1, 2 * n, 2 * n, device="cuda", dtype=torch.bool)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            o2 = trifast_amd.triangle_attention(q2, k2, v2, b2, m2)  # key 1_32_128: a miss, under capture
    torch.cuda.current_stream().wait_stream(side)
    graph.replay()
    torch.cuda.synchronize()
    assert "1_32_128_torch.bfloat16" not in tuner._cache_for(_lib.KERNEL_FWD).cache
    ref = orc.attention_reference(q2.float(), k2.float(), v2.float(), b2.float(), m2)
    assert (o2.float() - ref).abs().max() < 3e-2
    del eager_env
