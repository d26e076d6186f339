"""Where the db kernel's pipelined walk spends its clocks, measured by the kernel itself.

The library is built once more with ``-DTRI_DB_TIMING`` (csrc/tri_bwd_b.hpp): every wave of
the db kernel then reads the shader clock around the counted wait and the barrier that end a
pair row, and leaves its totals where the ``db`` argument points.  This script runs that
kernel alone (``trifast_bwd_one``, kernel 3, a block whose waves own two key tiles) on an
unmasked workload and prints clocks per row in total, in the counted wait and in the barrier
(per wave: the two waves of a SIMD are waves w and w + 4 of the 8-wave block), and the shader
clock rate inside the walk.

    python3 benchmark/microbench/db_timeline.py [--workload M] [--tile 3] [--loads 1|0|2]

``--loads 0`` builds the probe without the walk's global loads, ``--loads 2`` with loads that
re-read one row (traffic from L2 to LDS but not from memory): the difference to ``--loads 1``
is what the memory traffic costs the arithmetic beside it, in clocks per row and in clock rate.
Each variant is a library of its own under trifast_amd/ (built if it is not there; the regular
library is left alone).  The readings cost about 40 clocks per row and wave.
"""
import argparse
import pathlib
import sys

ROOT = pathlib.Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--workload", default="M")
    ap.add_argument("--tile", type=int, default=3)
    ap.add_argument("--loads", type=int, default=1, choices=(0, 1, 2))
    ap.add_argument("--build-only", action="store_true")
    args = ap.parse_args()
    lib_path = ROOT / "trifast_amd" / f"libtrifast_db_timeline_loads{args.loads}.so"
    if not lib_path.exists():
        from trifast_amd import build
        build.build(out=lib_path, extra=("-DTRI_DB_TIMING", f"-DTRI_DB_TIMING_LOADS={args.loads}"))
    if args.build_only:
        return

    import torch
    import bench
    from trifast_amd import _lib
    from trifast_amd import torch as tt

    q, k, v, bias, mask, do = bench.make_workload(args.workload, "cuda")
    if mask.any():
        sys.exit("the pipelined walk covers plain rows: pick a workload without a mask")
    b, h, n, _, d = q.shape
    code = tt._DTYPE_CODE[q.dtype]
    with torch.no_grad():
        o, lse = tt._triangle_attention(q, k, v, bias, mask)  # (the regular library)
    regular = _lib.load()
    info = _lib.tile_info(_lib.KERNEL_BWD_B, args.tile)
    nw = info["num_waves"]
    ws = torch.zeros(regular.trifast_bwd_workspace_bytes(b, h, n, d, code), dtype=torch.uint8, device="cuda")
    dq, dk, dv = (torch.zeros_like(o) for _ in range(3))
    db = torch.zeros_like(bias)
    mu8 = mask.view(torch.uint8)
    S = lambda t: _lib.i64_array(tt._strides(t))
    stream = torch.cuda.current_stream().cuda_stream

    def run(lib, kernel, tile):
        rc = lib.trifast_bwd_one(kernel, dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), db.data_ptr(), do.data_ptr(),
                                 q.data_ptr(), k.data_ptr(), v.data_ptr(), bias.data_ptr(), mu8.data_ptr(), o.data_ptr(), lse.data_ptr(),
                                 b, h, n, d, code, S(do), S(q), S(k), S(v), S(bias), S(mu8), None, None, None, None, tile,
                                 ws.data_ptr(), ws.numel(), stream)
        _lib.check(rc, "trifast_bwd_one")

    # the dq / row-resident kernel leaves the per-query words the db kernel reads
    row_tile = regular.trifast_default_tile(_lib.KERNEL_BWD_KV, n, h, d, code)
    if not regular.trifast_bwd_kv_tile_writes_dq(row_tile):
        run(regular, _lib.KERNEL_BWD_Q, regular.trifast_default_tile(_lib.KERNEL_BWD_Q, n, h, d, code))
    run(regular, _lib.KERNEL_BWD_KV, row_tile)
    torch.cuda.synchronize()
    _lib.LIB_PATH = lib_path
    _lib._lib = None
    probe = _lib.load()
    def timed(lib):
        # (twenty launches first: the clock takes a while to come up after a pause)
        for _ in range(20):
            run(lib, _lib.KERNEL_BWD_B, args.tile)
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        run(lib, _lib.KERNEL_BWD_B, args.tile)
        e.record()
        e.synchronize()
        return s.elapsed_time(e)

    regular_ms = timed(regular)
    probe_ms = timed(probe)
    db.zero_()  # (the library's kernel wrote db; the probe writes its records only)
    run(probe, _lib.KERNEL_BWD_B, args.tile)
    torch.cuda.synchronize()
    # one record per wave at the workgroup's linear index in the grid, whose last extent is
    # the (batch*head, row chunk) groups (at most 8 chunks) padded to a multiple of 8; db was
    # zero before the launch, so every other word still is
    blocks = ((n + info["BLOCK_J"] - 1) // info["BLOCK_J"]) * ((n + info["BLOCK_K"] - 1) // info["BLOCK_K"])
    slots = min(blocks * ((b * h * 8 + 7) // 8 * 8), db.numel() * db.element_size() // (8 * nw * 4))
    rec = db.view(torch.int64).flatten()[: slots * nw * 4].view(-1, nw, 4).cpu().double()
    rec = rec[rec[:, 0, 0] > 0]
    tot, wait, bar, real = rec[..., 0], rec[..., 1], rec[..., 2], rec[..., 3]
    loads = {0: "no global loads in the walk", 1: "as in the library", 2: "loads re-read one row"}[args.loads]
    print(f"workload {args.workload}, db tile {args.tile} ({nw} waves), probe build ({loads}): {probe_ms:.3f} ms per launch (the library's kernel: {regular_ms:.3f} ms)")
    rows = n  # (one chunk of rows at the sizes this probe is meant for; otherwise per chunk)
    print(f"{len(rec)} workgroups x {nw} waves, {n} pair rows each; shader clock inside the walk {float((tot / (real / 100)).mean()):.0f} MHz")
    print(f"clocks per row: total {float(tot.mean()) / n:.0f}, in the counted wait {float(wait.mean()) / n:.0f}, at the barrier {float(bar.mean()) / n:.0f}")
    print("  per wave, counted wait:", [round(float(x) / n) for x in wait.mean(0)])
    print("  per wave, barrier:     ", [round(float(x) / n) for x in bar.mean(0)])
    print(f"walk {float(real.mean()) / 100:.1f} us per workgroup (min {float(real.min()) / 100:.1f}, max {float(real.max()) / 100:.1f})")


if __name__ == "__main__":
    main()
