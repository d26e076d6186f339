"""The allocation-free forward entry point against the ordinary one.

``trifast_fwd_static`` takes no workspace: its scratch is a static device array inside
the library.  Called through the C ABI it must give bit-for-bit what ``trifast_fwd``
gives with a caller-provided workspace, on two calls in a row on the same GPU (the
second with a smaller input, so stale contents of the shared array would show), and
it must reject shapes whose scratch does not fit.
"""

import pytest
import torch

from trifast_amd import _lib
from trifast_amd import torch as tt

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _call(static, q, k, v, bias, mask, tile=-1):
    lib = _lib.load()
    b, h, n, _, d = q.shape
    code = tt._DTYPE_CODE[q.dtype]
    mu8 = mask.view(torch.uint8)
    o = torch.full((b, h, n, n, d), float("nan"), dtype=q.dtype, device=q.device)
    lse = torch.full((b, h, n, n), float("nan"), dtype=torch.float32, device=q.device)
    S = lambda t: _lib.i64_array(tt._strides(t))
    stream = torch.cuda.current_stream().cuda_stream
    common = (o.data_ptr(), lse.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), bias.data_ptr(), mu8.data_ptr(),
              b, h, n, d, code, S(q), S(k), S(v), S(bias), S(mu8), tile)
    if static:
        rc = lib.trifast_fwd_static(*common, stream)
    else:
        ws = torch.empty(lib.trifast_fwd_workspace_bytes(b, h, n, d, code), dtype=torch.uint8, device=q.device)
        rc = lib.trifast_fwd(*common, ws.data_ptr(), ws.numel(), stream)
    torch.cuda.synchronize()
    return rc, o, lse


def _inputs(b, h, n, d, dtype, seed, p_mask):
    g = torch.Generator(device=DEV).manual_seed(seed)
    q, k, v = (torch.randn(b, h, n, n, d, device=DEV, generator=g).to(dtype) for _ in range(3))
    bias = torch.randn(b, h, n, n, device=DEV, generator=g).to(dtype)
    mask = torch.rand(b, n, n, device=DEV, generator=g) < p_mask
    mask[:, n // 3, :] = True  # one fully masked row
    return q, k, v, bias, mask


def test_static_forward_matches_workspace_forward_twice():
    lib = _lib.load()
    # first call: a large shape that nearly fills the static array; second: a smaller,
    # ragged one in another dtype, which reuses the front of the same array
    for (b, h, n, d, dtype, seed) in ((1, 4, 1024, 32, torch.bfloat16, 1), (2, 3, 77, 64, torch.float16, 2), (1, 2, 40, 32, torch.float32, 3)):
        q, k, v, bias, mask = _inputs(b, h, n, d, dtype, seed, 0.3)
        before = torch.cuda.memory_allocated()
        rc, o_s, lse_s = _call(True, q, k, v, bias, mask)
        assert rc == 0, _lib.last_error()
        rc, o_w, lse_w = _call(False, q, k, v, bias, mask)
        assert rc == 0, _lib.last_error()
        assert torch.isfinite(o_s.float()).all() and torch.isfinite(lse_s[~mask.all(-1)[:, None, :, None].expand_as(lse_s)]).all()
        assert torch.equal(o_s, o_w), f"o differs for n={n} {dtype}"
        assert torch.equal(lse_s, lse_w), f"lse differs for n={n} {dtype}"
        del o_s, o_w, lse_s, lse_w
        assert torch.cuda.memory_allocated() == before
    # the same small shape again after the others: still the same answer (nothing stale is read)
    q, k, v, bias, mask = _inputs(1, 2, 40, 32, torch.float32, 3, 0.3)
    _, o_s, lse_s = _call(True, q, k, v, bias, mask)
    _, o_w, lse_w = _call(False, q, k, v, bias, mask)
    assert torch.equal(o_s, o_w) and torch.equal(lse_s, lse_w)


def test_static_forward_takes_no_device_memory_and_runs_under_capture():
    """After one warm-up call (the first call on a device looks up the array's address and
    may raise a kernel's LDS limit: both happen outside a capture), a call changes the
    device's free memory by nothing, and the entry point can be recorded into a HIP graph
    and replayed, with the bits of ``trifast_fwd``."""
    lib = _lib.load()
    q, k, v, bias, mask = _inputs(1, 2, 256, 32, torch.bfloat16, 7, 0.2)
    b, h, n, _, d = q.shape
    code = tt._DTYPE_CODE[q.dtype]
    mu8 = mask.view(torch.uint8)
    S = lambda t: _lib.i64_array(tt._strides(t))
    o = torch.empty((b, h, n, n, d), dtype=q.dtype, device=DEV)
    lse = torch.empty((b, h, n, n), dtype=torch.float32, device=DEV)

    def call(stream):
        return lib.trifast_fwd_static(o.data_ptr(), lse.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), bias.data_ptr(), mu8.data_ptr(),
                                      b, h, n, d, code, S(q), S(k), S(v), S(bias), S(mu8), -1, stream)

    assert call(torch.cuda.current_stream().cuda_stream) == 0, _lib.last_error()  # warm-up
    torch.cuda.synchronize()
    # the driver's own count of free bytes sees any allocation, the library's included
    free_before = torch.cuda.mem_get_info()[0]
    assert call(torch.cuda.current_stream().cuda_stream) == 0, _lib.last_error()
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    _, o_w, lse_w = _call(False, q, k, v, bias, mask)

    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            assert call(side.cuda_stream) == 0, _lib.last_error()
    torch.cuda.current_stream().wait_stream(side)
    for rep in range(3):
        o.fill_(float("nan"))
        lse.fill_(float("nan"))
        torch.cuda.synchronize()  # (eager work and a synchronisation between the replays)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(o, o_w) and torch.equal(lse, lse_w), f"replay {rep} differs from trifast_fwd"


def test_static_forward_rejects_what_does_not_fit():
    lib = _lib.load()
    # bf16 b=1 h=8 n=1024 needs 16 MiB of packed bias: more than the static array
    assert lib.trifast_fwd_workspace_bytes(1, 8, 1024, 32, _lib.BF16) > 12 * 1024 * 1024
    q = torch.zeros(1, 8, 1024, 1024, 32, dtype=torch.bfloat16, device=DEV)
    bias = torch.zeros(1, 8, 1024, 1024, dtype=torch.bfloat16, device=DEV)
    mask = torch.zeros(1, 1024, 1024, dtype=torch.bool, device=DEV)
    rc, o, _ = _call(True, q, q, q, bias, mask)
    assert rc == -4 and "static" in _lib.last_error()
    assert torch.isnan(o.float()).all()  # nothing was launched
