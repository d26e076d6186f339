"""What masks cost each kernel of the step at one shape.

Times the forward (through the operator), the row-resident dq + dk + dv kernel and the db kernel
(8-wave and 16-wave blocks) at a benchmark workload's shape with its tensors and four masks:
none, a 50 % random mask (the reference's benchmark protocol), keys past a length masked, and
padding (rows and keys past a length).  Default tiles, no tuner; median of six rounds of ten
launches after ten warm-up launches.

    python3 benchmark/microbench/mask_cost.py [--workload M] [--length 900]
"""
import argparse
import os
import pathlib
import statistics
import sys

ROOT = pathlib.Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))
os.environ["TRIFAST_AUTOTUNE"] = "0"


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--workload", default="M")
    ap.add_argument("--length", type=int, default=900)
    args = ap.parse_args()

    import torch
    import bench
    from trifast_amd import _lib
    from trifast_amd import torch as tt

    lib = _lib.load()
    q, k, v, bias, _, do = bench.make_workload(args.workload, "cuda")
    b, h, n, _, d = q.shape
    code = tt._DTYPE_CODE[q.dtype]
    g = torch.Generator(device="cuda").manual_seed(5)
    L = min(args.length, n)
    none = torch.zeros(b, n, n, dtype=torch.bool, device="cuda")
    rand = torch.rand(b, n, n, device="cuda", generator=g) < 0.5
    keys = none.clone()
    keys[:, :, L:] = True
    pad = keys.clone()
    pad[:, L:, :] = True
    S = lambda t: _lib.i64_array(tt._strides(t))
    stream = torch.cuda.current_stream().cuda_stream
    ws = torch.empty(lib.trifast_bwd_workspace_bytes(b, h, n, d, code), dtype=torch.uint8, device="cuda")
    dq, dk, dv = (torch.zeros_like(q) for _ in range(3))
    db = torch.zeros_like(bias)

    def timeit(fn):
        for _ in range(10):
            fn()
        ts = []
        for _ in range(6):
            s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            s.record()
            for _ in range(10):
                fn()
            e.record()
            e.synchronize()
            ts.append(s.elapsed_time(e) / 10)
        return statistics.median(ts)

    row_tile = lib.trifast_default_tile(_lib.KERNEL_BWD_KV, n, h, d, code)
    if not lib.trifast_bwd_kv_tile_writes_dq(row_tile):
        sys.exit("the default dk/dv tile at this shape is not the row-resident kernel")
    infos = {t: _lib.tile_info(_lib.KERNEL_BWD_B, t) for t in range(lib.trifast_num_tiles(_lib.KERNEL_BWD_B))}
    db_tiles = [t for t, i in infos.items() if (i["BLOCK_J"], i["BLOCK_K"]) == (128, 128) and i["num_waves"] in (8, 16)
                and lib.trifast_supports(_lib.KERNEL_BWD_B, t, n, h, d, code)]
    print(f"workload {args.workload}: {tuple(q.shape)} {q.dtype}, lengths {L} of {n}; ms per launch")
    print(f"{'mask':28s} {'forward':>9s} {'dq+dk+dv':>9s} " + " ".join(f"{'db ' + str(infos[t]['num_waves']) + ' waves':>12s}" for t in db_tiles))
    for name, mask in (("none", none), ("random, 50 %", rand), (f"keys past {L}", keys), (f"rows and keys past {L}", pad)):
        mu8 = mask.view(torch.uint8)
        with torch.no_grad():
            o, lse = tt._triangle_attention(q, k, v, bias, mask)

        def fwd():
            with torch.no_grad():
                tt._triangle_attention(q, k, v, bias, mask)

        def bwd(kernel, tile):
            rc = lib.trifast_bwd_one(kernel, dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), db.data_ptr(), do.data_ptr(), q.data_ptr(),
                                     k.data_ptr(), v.data_ptr(), bias.data_ptr(), mu8.data_ptr(), o.data_ptr(), lse.data_ptr(), b, h, n, d, code,
                                     S(do), S(q), S(k), S(v), S(bias), S(mu8), None, None, None, None, tile, ws.data_ptr(), ws.numel(), stream)
            _lib.check(rc, "trifast_bwd_one")

        t_f = timeit(fwd)
        t_r = timeit(lambda: bwd(_lib.KERNEL_BWD_KV, row_tile))
        t_b = [timeit(lambda t=t: bwd(_lib.KERNEL_BWD_B, t)) for t in db_tiles]
        print(f"{name:28s} {t_f:9.3f} {t_r:9.3f} " + " ".join(f"{x:12.3f}" for x in t_b), flush=True)


if __name__ == "__main__":
    main()
