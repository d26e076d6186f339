"""Timeline of the row-resident backward kernel, measured by the kernel itself.

The library is built once more with ``-DTRI_ROW_TIMING`` (csrc/tri_bwd_row.hpp): wave 0 of
every workgroup then reads the 100 MHz counter at kernel entry, at four marks of the
prologue, at the start and the end of the query-tile loop and after the dk/dv stores are
issued, and the shader clock between the steps of the loop; it leaves the readings where the
``db`` argument points.  This script runs that kernel alone (``trifast_bwd_one``, kernel 2) on
the benchmark's workload and prints, per workgroup and per compute unit:

* prologue / loop / epilogue / gap to the next workgroup on the same compute unit (us),
* when the prologue's loads were issued, when V had arrived, when delta was done,
* shader clocks per step of a query tile (step -1 starts tile 0, step KT finishes tile KT-1),
  per partial-tile store and per barrier, and the shader clock rate inside the loop.

    python3 benchmark/microbench/row_timeline.py [--workload M] [--lib PATH]

``--lib`` names the timing build of the library (default: trifast_amd/libtrifast_row_timeline.so,
built if it is not there; the regular library is left alone).  The readings perturb the
kernel (each costs a scalar memory round trip): the timing build runs about 5 % slower.
"""
import argparse
import collections
import pathlib
import sys

ROOT = pathlib.Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--workload", default="M")
    ap.add_argument("--lib", default=str(ROOT / "trifast_amd" / "libtrifast_row_timeline.so"))
    ap.add_argument("--build-only", action="store_true")
    args = ap.parse_args()
    lib_path = pathlib.Path(args.lib)
    if not lib_path.exists():
        from trifast_amd import build
        build.build(out=lib_path, extra=("-DTRI_ROW_TIMING",))
    if args.build_only:
        return

    import torch
    import bench
    from trifast_amd import _lib
    from trifast_amd import torch as tt

    q, k, v, bias, mask, do = bench.make_workload(args.workload, "cuda")
    b, h, n, _, d = q.shape
    code = tt._DTYPE_CODE[q.dtype]
    with torch.no_grad():
        o, lse = tt._triangle_attention(q, k, v, bias, mask)  # (the regular library)
    _lib.LIB_PATH = lib_path
    _lib._lib = None
    lib = _lib.load()
    tile = lib.trifast_default_tile(_lib.KERNEL_BWD_KV, n, h, d, code)
    if not lib.trifast_bwd_kv_tile_writes_dq(tile):
        sys.exit(f"the default dk/dv tile of workload {args.workload} is not the row-resident kernel")
    kt = lib.trifast_num_tiles(_lib.KERNEL_BWD_KV)  # (only to show the tile id range)
    rows = b * h * n
    ws = torch.zeros(lib.trifast_bwd_workspace_bytes(b, h, n, d, code), dtype=torch.uint8, device="cuda")
    dq, dk, dv = (torch.zeros_like(o) for _ in range(3))
    rec_buf = torch.zeros(max(rows * 32, bias.numel() // 4 + 1), dtype=torch.int64, device="cuda")
    mu8 = mask.view(torch.uint8)
    S = lambda t: _lib.i64_array(tt._strides(t))
    stream = torch.cuda.current_stream().cuda_stream

    def run():
        rc = lib.trifast_bwd_one(_lib.KERNEL_BWD_KV, dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), rec_buf.data_ptr(), do.data_ptr(),
                                 q.data_ptr(), k.data_ptr(), v.data_ptr(), bias.data_ptr(), mu8.data_ptr(), o.data_ptr(), lse.data_ptr(),
                                 b, h, n, d, code, S(do), S(q), S(k), S(v), S(bias), S(mu8), None, None, None, None, tile,
                                 ws.data_ptr(), ws.numel(), stream)
        _lib.check(rc, "trifast_bwd_one")

    for _ in range(3):
        run()
    torch.cuda.synchronize()
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    s.record()
    run()
    e.record()
    e.synchronize()
    info = _lib.tile_info(_lib.KERNEL_BWD_KV, tile)
    KT = info["BLOCK_K"] // 128
    print(f"workload {args.workload}: row-resident tile {tile} of {kt} ({KT} key tiles per wave), timing build: {s.elapsed_time(e):.3f} ms per launch")

    rec = rec_buf[: rows * 32].view(rows, 32).cpu()
    rec = rec[rec[:, 0] != 0]
    t0 = int(rec[:, 0].min())
    us = lambda a, bcol: (rec[:, bcol] - rec[:, a]).double() / 100
    stat = lambda x: f"{x.mean():7.2f} (min {x.min():.2f}, max {x.max():.2f})"
    print(f"{len(rec)} workgroups; microseconds per workgroup, 100 MHz counter:")
    print(f"  prologue           {stat(us(0, 5))}")
    print(f"    loads issued at  {stat(us(0, 1))}")
    print(f"    V arrived at     {stat(us(0, 2))}")
    print(f"    delta done at    {stat(us(0, 3))}")
    print(f"    last wait from   {stat(us(0, 4))}")
    print(f"  query-tile loop    {stat(us(5, 6))}")
    print(f"  dk/dv stores       {stat(us(6, 7))}   (until the last one is issued)")
    percu = collections.defaultdict(list)
    for r in rec.tolist():
        hw, xcc = r[8], r[9]
        percu[(xcc & 0xF, (hw >> 13) & 7, (hw >> 12) & 1, (hw >> 8) & 0xF)].append((r[0] - t0, r[7] - t0))
    counts = collections.Counter(len(x) for x in percu.values())
    gaps = []
    for x in percu.values():
        x.sort()
        gaps += [(x[i + 1][0] - x[i][1]) / 100 for i in range(len(x) - 1)]
    print(f"  {len(percu)} compute units; workgroups per compute unit: {sorted(counts.items())}")
    if gaps:
        g = torch.tensor(gaps)
        print(f"  gap to the next workgroup on the compute unit {g.mean():.2f} (median {g.median():.2f}, max {g.max():.2f})")
    print(f"  first entry to last end {(int(rec[:, 7].max()) - t0) / 100:.1f}")
    clocks = rec[:, 10].double()
    loop_us = us(5, 6)
    print(f"shader clock inside the loop: {float((clocks / loop_us).mean()):.0f} MHz")
    nj = (n + 31) // 32
    names = ["before step -1"] + [f"step {t}" for t in range(-1, KT + 1)] + ["partial-tile store", "barrier"]
    print("shader clocks per query tile (mean over the workgroups):")
    total = 0.0
    for idx, name in enumerate(names):
        x = rec[:, 11 + idx].double() / nj
        total += float(x.mean())
        print(f"  {name:20s} {x.mean():8.1f}  (min {x.min():.1f}, max {x.max():.1f})")
    print(f"  {'sum':20s} {total:8.1f}")


if __name__ == "__main__":
    main()
