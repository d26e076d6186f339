"""The C-ABI library loads and exports what include/trifast_hip.h declares.

No kernel is launched here: the checks stop at argument validation and the
host-side tile tables, none of which touch the GPU.
"""

import ctypes
import re
from pathlib import Path

import pytest

from trifast_amd import _lib

ROOT = Path(__file__).resolve().parent.parent
HEADER = ROOT / "include" / "trifast_hip.h"


def declared_functions():
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    return sorted(set(re.findall(r"\b(trifast_\w+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound():
    lib = _lib.load()
    names = declared_functions()
    assert len(names) >= 11
    for name in names:
        assert hasattr(lib, name), f"{name} is declared in the header but not exported"
        assert name in _lib.SIGNATURES, f"{name} has no ctypes signature"
    assert sorted(_lib.SIGNATURES) == names


def test_abi_version_matches_header():
    want = int(re.search(r"#define TRIFAST_ABI_VERSION (\d+)", HEADER.read_text()).group(1))
    assert _lib.load().trifast_abi_version() == want == _lib.ABI_VERSION


def test_tile_tables():
    lib = _lib.load()
    for kernel in range(4):
        nt = lib.trifast_num_tiles(kernel)
        assert 1 <= nt <= 12
        for t in range(nt):
            info = _lib.tile_info(kernel, t)
            assert info["BLOCK_J"] % 32 == 0 and info["BLOCK_K"] % 32 == 0 and info["num_waves"] in (1, 2, 4, 8, 16)
        with pytest.raises(ValueError):
            _lib.tile_info(kernel, nt)
    assert lib.trifast_num_tiles(99) < 0


@pytest.mark.parametrize("dtype", [_lib.F32, _lib.BF16, _lib.F16])
@pytest.mark.parametrize("d", [16, 32, 64, 128])
def test_every_shape_has_a_default_tile(dtype, d):
    lib = _lib.load()
    for kernel in range(4):
        for n in (1, 17, 256, 2048):
            t = lib.trifast_default_tile(kernel, n, 4, d, dtype)
            assert t >= 0, _lib.last_error()
            assert lib.trifast_supports(kernel, t, n, 4, d, dtype) == 1


def test_unsupported_head_dim_and_dtype():
    lib = _lib.load()
    assert lib.trifast_supports(0, 0, 64, 4, 48, _lib.BF16) == 0
    assert lib.trifast_supports(0, 0, 64, 4, 32, 7) == 0
    assert lib.trifast_default_tile(0, 64, 4, 48, _lib.BF16) < 0


def test_workspace_sizes_are_quadratic_in_n():
    lib = _lib.load()
    f1 = lib.trifast_fwd_workspace_bytes(1, 4, 1024, 32, _lib.BF16)
    b1 = lib.trifast_bwd_workspace_bytes(1, 4, 1024, 32, _lib.BF16)
    b2 = lib.trifast_bwd_workspace_bytes(1, 4, 2048, 32, _lib.BF16)
    plane = 4 * 1024 * 1024  # h * n * n elements
    # forward: keep words, row flags and one packed copy of the bias in the input dtype
    assert plane * 2 <= f1 <= plane * 2 + (1 << 20)
    # backward: two packed bias copies, two 32-bit per-query planes (delta and lse) and at
    # most 8 fp32 db partials
    assert plane * (2 * 2 + 2 * 4) <= b1 <= plane * (2 * 2 + 2 * 4 + 8 * 4) + (1 << 20)
    # rows too long for one pass of the row-resident kernel (n > 1024 at head dim 32) add the low
    # parts of dq between its passes: one more tensor of the inputs' size, shared with the db partials
    assert plane * 4 * (2 * 2 + 2 * 4) <= b2 <= plane * 4 * (2 * 2 + 2 * 4 + 32 * 2) + (1 << 20)
    # O(n^2): doubling n may not cost more than four times the memory
    b4 = lib.trifast_bwd_workspace_bytes(1, 4, 4096, 32, _lib.BF16)
    assert 1.9 < b4 / b2 < 4.1
    assert lib.trifast_fwd_workspace_bytes(0, 4, 16, 32, _lib.BF16) < 0


def test_argument_errors_come_back_as_codes_not_crashes():
    lib = _lib.load()
    st5 = _lib.i64_array([0, 0, 0, 32, 1])
    st4 = _lib.i64_array([0, 0, 8, 1])
    st3 = _lib.i64_array([0, 8, 1])
    args = lambda d, q: (0x1000, 0x1000, q, 0x1000, 0x1000, 0x1000, 0x1000, 1, 1, 8, d, _lib.BF16, st5, st5, st5, st4, st3, -1, None, 0, None)
    rc = lib.trifast_fwd(*args(48, 0x1000))
    assert rc == -2 and "head dim" in _lib.last_error()
    rc = lib.trifast_fwd(*args(32, 0x1008))
    assert rc == -3 and "aligned" in _lib.last_error()
    rc = lib.trifast_fwd(*args(32, 0x1000))  # passes the pointer checks, has no workspace
    assert rc == -4 and "workspace" in _lib.last_error()
    with pytest.raises(ValueError):
        _lib.check(rc, "trifast_fwd")
    bad_stride = _lib.i64_array([0, 0, 0, 32, 2])
    rc = lib.trifast_fwd(0x1000, 0x1000, 0x1000, 0x1000, 0x1000, 0x1000, 0x1000, 1, 1, 8, 32, _lib.BF16, bad_stride, st5, st5, st4, st3, -1, None, 0, None)
    assert rc == -3 and "last stride" in _lib.last_error()
    far_rows = _lib.i64_array([0, 0, 32, 1 << 23, 1])  # 16 MiB between the rows of a bf16 tile
    rc = lib.trifast_fwd(0x1000, 0x1000, 0x1000, 0x1000, 0x1000, 0x1000, 0x1000, 1, 1, 8, 32, _lib.BF16, st5, far_rows, st5, st4, st3, -1, None, 0, None)
    assert rc == -2 and "stride 3" in _lib.last_error()
    none4 = (None, None, None, None)
    rc = lib.trifast_bwd_one(0, *([0x1000] * 12), 1, 1, 8, 32, _lib.BF16, st5, st5, st5, st5, st4, st3, *none4, -1, None, 0, None)
    assert rc == -1 and "backward kernel" in _lib.last_error()


def test_gate_argument_errors_come_back_as_codes():
    """The gate entries check sizes, dtype and pointers before they launch anything."""
    lib = _lib.load()
    ok = 0x1000
    assert lib.trifast_gate_fwd(ok, ok, ok, 1, 2, 8, 48, _lib.BF16, None) == -2 and "head dim" in _lib.last_error()
    assert lib.trifast_gate_fwd(None, ok, ok, 1, 2, 8, 32, _lib.BF16, None) == -1 and "null" in _lib.last_error()
    assert lib.trifast_gate_fwd(ok, ok + 8, ok, 1, 2, 8, 32, _lib.BF16, None) == -3 and "o is not 16-byte" in _lib.last_error()
    assert lib.trifast_gate_bwd(ok, ok, None, ok, ok, 1, 2, 8, 32, _lib.BF16, None) == -1 and "dy" in _lib.last_error()
    assert lib.trifast_gate_bwd(ok + 4, ok, ok, ok, ok, 1, 2, 8, 32, _lib.F32, None) == -3 and "do" in _lib.last_error()
    assert lib.trifast_gate_bwd(ok, ok, ok, ok, ok, 1, 2, 8, 32, 7, None) < 0


def test_weight_gradient_argument_errors_come_back_as_codes():
    lib = _lib.load()
    ok = 0x1000
    call = lambda dw, dy, x, rows, k, n, dtype=_lib.BF16, ws=ok, nbytes=1 << 40, hd=0: lib.trifast_linear_dw(dw, None, dy, x, rows, k, n, hd, dtype, ws, nbytes, None)
    assert call(ok, ok, ok, 100, 48, 8) == -2 and "input channels" in _lib.last_error()
    assert call(ok, ok, ok, 100, 64, 8, _lib.F32) == -2 and "16-bit" in _lib.last_error()
    assert call(ok, ok, ok, 0, 64, 8) == -1 and "positive" in _lib.last_error()
    assert call(None, ok, ok, 100, 64, 8) == -1 and "null" in _lib.last_error()
    assert call(ok, ok + 8, ok, 100, 64, 8) == -3 and "aligned" in _lib.last_error()
    assert call(ok, ok, ok, 100, 64, 8, nbytes=16) == -4 and "workspace" in _lib.last_error()
    assert call(ok, ok, ok, 100, 64, 48, hd=32) == -1 and "head dim" in _lib.last_error()  # 32 does not divide 48
    assert call(ok, ok, ok, 100, 64, 48, hd=12) == -1 and "head dim" in _lib.last_error()  # not a multiple of 8
    # the partials: one [n, k] fp32 matrix per chunk of at least 1024 rows, at most 768 chunks
    # (plus one [n] fp32 vector per chunk for the bias gradient)
    assert lib.trifast_linear_dw_workspace_bytes(1024, 128, 128) == 128 * 128 * 4 + 128 * 4
    assert lib.trifast_linear_dw_workspace_bytes(3000, 128, 128) == 3 * 128 * 128 * 4 + 3 * 128 * 4
    assert 700 * 128 * 129 * 4 <= lib.trifast_linear_dw_workspace_bytes(1 << 20, 128, 128) <= 768 * 128 * 129 * 4
    assert lib.trifast_linear_dw_workspace_bytes(1 << 24, 128, 4) <= 768 * 129 * 4 * 4 + 512
    assert lib.trifast_linear_dw_workspace_bytes(0, 128, 4) < 0


def test_linear_forward_argument_errors_come_back_as_codes():
    import ctypes

    lib = _lib.load()
    ok = 0x1000
    vp = lambda *v: (ctypes.c_void_p * len(v))(*v)
    n1 = _lib.i64_array([8])
    call = lambda x, k, nl, w, y, n, dtype=_lib.BF16, rows=4, hd=None: lib.trifast_linear_fwd(x, rows, k, nl, w, None, y, n, hd, dtype, None)
    assert call(ok, 256, 1, vp(ok), vp(ok), n1) == -2 and "input channels" in _lib.last_error()
    assert call(ok, 64, 1, vp(ok), vp(ok), n1, _lib.F32) == -2 and "16-bit" in _lib.last_error()
    assert call(ok, 64, 7, vp(*[ok] * 7), vp(*[ok] * 7), _lib.i64_array([8] * 7)) == -1 and "layers per call" in _lib.last_error()
    assert call(ok + 8, 64, 1, vp(ok), vp(ok), n1) == -3 and "x is not" in _lib.last_error()
    assert call(ok, 64, 1, vp(ok), vp(ok + 4), n1) == -3 and "layer 0" in _lib.last_error()
    assert call(ok, 64, 1, vp(None), vp(ok), n1) == -1 and "null" in _lib.last_error()
    assert call(ok, 64, 1, vp(ok), vp(ok), n1, rows=0) == -1 and "rows" in _lib.last_error()
    assert call(ok, 64, 1, vp(ok), vp(ok), n1, hd=_lib.i64_array([16])) == -1 and "head dim" in _lib.last_error()


def test_input_gradient_argument_errors_come_back_as_codes():
    import ctypes

    lib = _lib.load()
    ok = 0x1000
    vp = lambda *v: (ctypes.c_void_p * len(v))(*v)
    n1 = _lib.i64_array([8])
    call = lambda dx, k, nl, dy, wt, n, dtype=_lib.BF16, rows=4, hd=None: lib.trifast_linear_dx(dx, rows, k, nl, dy, wt, n, hd, dtype, None)
    assert call(ok, 256, 1, vp(ok), vp(ok), n1) == -2 and "input channels" in _lib.last_error()
    assert call(ok, 64, 1, vp(ok), vp(ok), n1, _lib.F32) == -2 and "16-bit" in _lib.last_error()
    assert call(ok, 64, 7, vp(*[ok] * 7), vp(*[ok] * 7), _lib.i64_array([8] * 7)) == -1 and "layers per call" in _lib.last_error()
    assert call(ok + 8, 64, 1, vp(ok), vp(ok), n1) == -3 and "dx is not" in _lib.last_error()
    assert call(ok, 64, 1, vp(ok), vp(ok + 4), n1) == -3 and "layer 0" in _lib.last_error()
    assert call(ok, 64, 1, vp(None), vp(ok), n1) == -1 and "null" in _lib.last_error()
    assert call(ok, 64, 1, vp(ok), vp(ok), _lib.i64_array([0])) == -1 and "outputs" in _lib.last_error()
    assert call(ok, 64, 1, vp(ok), vp(ok), n1, rows=0) == -1 and "rows" in _lib.last_error()
    assert call(ok, 64, 1, vp(ok), vp(ok), n1, hd=_lib.i64_array([16])) == -1 and "head dim" in _lib.last_error()


def test_gated_output_checks_shapes_on_the_host():
    import torch

    from trifast_amd import nn

    o = torch.zeros(1, 2, 8, 8, 16)
    with pytest.raises(ValueError, match="g must be"):
        nn.gated_output(o, torch.zeros(1, 8, 8, 16))
    with pytest.raises(TypeError):
        nn.gated_output(o, torch.zeros(1, 8, 8, 32, dtype=torch.bfloat16))
    with pytest.raises(RuntimeError, match="GPU only"):  # no CPU fallback
        nn.gated_output(o, torch.zeros(1, 8, 8, 32))
    block = nn.TriangleAttention(24, 2, 16, ending_node=True)
    assert block.heads(torch.zeros(3, 8, 8, 32)).shape == (3, 2, 8, 8, 16)
    # linear layers over CPU tensors are torch's own
    assert nn.linear(torch.zeros(2, 24), block.b).shape == (2, 2)
    assert [t.shape for t in nn.project(torch.zeros(2, 24), (block.q, block.b))] == [(2, 32), (2, 2)]
    # heads-outermost outputs: [h, *, d]; on tensors the kernels do not take, a permuted copy
    assert [t.shape for t in nn.project(torch.zeros(3, 5, 24), (block.q, block.b), (16, 0))] == [(2, 3, 5, 16), (3, 5, 2)]
    # (a layer with a bias too)
    assert nn.project(torch.zeros(2, 24), (block.g,), (16,))[0].shape == (2, 2, 16)
    assert {n for n, _ in block.named_parameters()} == {"q.weight", "k.weight", "v.weight", "b.weight", "g.weight", "g.bias", "out.weight", "out.bias"}


def test_output_pointers_and_strides_are_checked():
    """Gradients and lse are written / read with vector accesses: a misaligned pointer or
    a stride the kernels cannot write comes back as TRIFAST_EALIGN, not as a fault."""
    lib = _lib.load()
    st5 = _lib.i64_array([0, 0, 8 * 32, 32, 1])
    st4 = _lib.i64_array([0, 0, 8, 1])
    st3 = _lib.i64_array([0, 8, 1])
    ws_bytes = lib.trifast_bwd_workspace_bytes(1, 1, 8, 32, _lib.BF16)

    def bwd(dq=0x1000, dk=0x1000, dv=0x1000, db=0x1000, lse=0x1000, out_strides=(None, None, None, None)):
        # (the workspace check comes after every pointer check, so a null workspace ends a
        # call whose pointers were accepted with TRIFAST_EWORKSPACE before anything is launched)
        return lib.trifast_bwd(dq, dk, dv, db, 0x1000, 0x1000, 0x1000, 0x1000, 0x1000, 0x1000, 0x1000, lse,
                               1, 1, 8, 32, _lib.BF16, st5, st5, st5, st5, st4, st3, *out_strides, None, None, ws_bytes, None)

    assert bwd() == -4
    assert bwd(db=0x1002) == -3 and "db" in _lib.last_error()
    assert bwd(lse=0x1002) == -3 and "lse" in _lib.last_error()
    assert bwd(dq=0x1008) == -3 and "dq" in _lib.last_error()
    assert bwd(dv=0x1004) == -3 and "dv" in _lib.last_error()
    assert bwd(db=None) == -1 and "db" in _lib.last_error()
    bad = _lib.i64_array([0, 0, 8 * 32, 32, 2])
    assert bwd(out_strides=(bad, None, None, None)) == -3 and "dq" in _lib.last_error()
    odd = _lib.i64_array([0, 0, 8 * 36, 36, 1])  # rows that are not 16-byte aligned
    assert bwd(out_strides=(None, odd, None, None)) == -3 and "dk" in _lib.last_error()
    transposed = _lib.i64_array([0, 0, 32, 8 * 32, 1])  # i <-> j transposed layout is fine
    assert bwd(out_strides=(transposed, transposed, transposed, _lib.i64_array([0, 0, 1, 8]))) == -4
    # forward: lse
    rc = lib.trifast_fwd(0x1000, 0x1002, 0x1000, 0x1000, 0x1000, 0x1000, 0x1000, 1, 1, 8, 32, _lib.BF16, st5, st5, st5, st4, st3, -1, None, 0, None)
    assert rc == -3 and "lse" in _lib.last_error()


def test_db_chunks_do_not_inflate_the_workspace():
    """One chunk of pair rows stays one chunk whatever b*h is (no partials, no reduce
    pass): an odd head count costs no more workspace per head than an even one."""
    lib = _lib.load()
    per_head = lambda h, n: lib.trifast_bwd_workspace_bytes(1, h, n, 32, _lib.BF16) / h
    assert per_head(5, 2048) <= 1.01 * per_head(8, 2048)
    assert per_head(5, 4096) <= 1.01 * per_head(8, 4096)
    assert per_head(1, 4096) <= 1.01 * per_head(8, 4096)
    # The split follows where the (batch*head, chunk) groups land on the 8 XCDs: at n = 1024,
    # h = 4 one chunk fills the GPU (no partials); at n = 768 two chunks would leave 36 workgroups
    # on 32 CUs, and eight run; tiny rows split down to 16 rows per chunk.  The partials are
    # fp32 [chunks, b*h, n, n] in the workspace tail (d = 64 has no other use for the tail).
    # (before the tail: the lse and delta planes and two packed copies of the bias, three such units)
    chunks = lambda h, n: lib.trifast_bwd_workspace_bytes(1, h, n, 64, _lib.BF16) // (h * n * n * 4) - 3
    assert chunks(4, 1024) == chunks(4, 2048) == 0
    assert chunks(4, 768) == 8 and chunks(4, 64) == 4 and chunks(4, 256) == 8
    assert chunks(64, 256) == 0  # many heads fill the GPU with one chunk


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", tmp_path / "libtrifast_hip.so")
    with pytest.raises(ImportError, match="no fallback"):
        _lib.load()
