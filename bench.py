#!/usr/bin/env python3
"""Benchmark of the fused triangle attention on one MI355X.

A "step" is one forward + one backward pass of ``trifast.triangle_attention`` over
one batch of synthetic pair tensors that are already resident in HBM.  The default
workload is the one the headline metric is quoted on: bf16, b=1, h=4, d=32,
n=1024, all keys attended.  Prints ONE JSON line:

  value        fwd+bwd TFLOP/s, counting 14*b*h*n^3*d FLOP per step
               (forward 4*b*h*n^3*d: two GEMMs; backward 10*b*h*n^3*d: five GEMMs)
  roofline     the slowest kernel of the step against the dense bf16 MFMA peak,
               its launch duration measured here with events on the launch stream
  cpu_baseline the PyTorch restatement of the reference's pure-PyTorch triangle
               attention, forward + autograd backward, on the host cores, on a
               bounded sample of rows of the same workload

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload M|C2|C3|C4a|C4b|C5|F32]
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

import torch

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16/fp16 MFMA
PEAK_F32_TFLOPS = 157.3
PEAK_HBM_GBS = 8000.0

# HBM bytes per launch (fetch + write) of the kernels of workload M with the tiles the
# tuner picks there, from the FETCH_SIZE / WRITE_SIZE counter runs summarised in
# profiles/bench_M_hbm_traffic.txt (readings scaled by a plain 256 MiB copy).  Reported
# as roofline.traffic when the benchmark runs that workload with that tile (keyed by the
# tile's index in the library's table of the kernel).
MEASURED_TRAFFIC_MIB = {
    ("M", "_fwd", 7): 1537.0,
    ("M", "_bwd_kv", 10): 2563.8,
    ("M", "_bwd_b", 4): 1586.0,
    ("M", "_bwd_b", 3): 1585.0,
}

# name -> (dtype, b, n, h, d, description)
WORKLOADS = {
    "C1": (torch.float32, 1, 32, 4, 32, "fp32 b1 n32 h4 d32, 10% random mask"),
    "C2": (torch.bfloat16, 1, 256, 4, 32, "bf16 b1 n256 h4 d32, no mask"),
    "C3": (torch.bfloat16, 1, 512, 4, 32, "bf16 b1 n512 h4 d32, padding mask"),
    "C4a": (torch.float16, 1, 768, 8, 64, "fp16 b1 n768 h8 d64, transposed views"),
    "C4b": (torch.float16, 2, 384, 8, 64, "fp16 b2 n384 h8 d64, transposed views"),
    "C5": (torch.bfloat16, 1, 2048, 4, 32, "bf16 b1 n2048 h4 d32, bias outliers, 5% random mask"),
    "M": (torch.bfloat16, 1, 1024, 4, 32, "bf16 b1 n1024 h4 d32, no mask"),
    # not one of the reference's configurations: the fp32-MFMA path at a size that fills the GPU
    "F32": (torch.float32, 1, 512, 4, 32, "fp32 b1 n512 h4 d32, no mask"),
}


def make_workload(name: str, device, seed: int = 1337):
    """Seeded synthetic inputs q, k, v, bias, mask, do of one benchmark config.

    Drawn in fp32 in the order q, k, v, bias, mask, do and then cast.  Small
    configs draw from a CPU generator; above 2**27 elements per tensor the draw
    moves to the device's generator (same seed) to keep set-up time bounded.
    """
    dtype, b, n, h, d, _ = WORKLOADS[name]
    numel = b * h * n * n * d
    gdev = torch.device(device) if numel > 2**27 else torch.device("cpu")
    g = torch.Generator(device=gdev).manual_seed(seed)

    def randn(*shape):
        return torch.randn(*shape, generator=g, device=gdev)

    def rand(*shape):
        return torch.rand(*shape, generator=g, device=gdev)

    std = d**-0.5
    if name in ("C4a", "C4b"):
        q, k, v = randn(b, h, n, n, d), randn(b, h, n, n, d), randn(b, h, n, n, d)
    else:
        q, k, v = randn(b, h, n, n, d) * std, randn(b, h, n, n, d) * std, randn(b, h, n, n, d) * std
    bias = randn(b, h, n, n)
    if name == "C1":
        bias = bias * std
        mask = rand(b, n, n) < 0.1
        full = mask.all(dim=-1)  # leave at least one attended key per row
        mask[..., 0] &= ~full
    elif name == "C3":
        # per batch element a valid length L in [n/2, n]; everything >= L is padding
        L = torch.randint(n // 2, n + 1, (b,), generator=g, device=gdev)
        idx = torch.arange(n, device=gdev)
        pad = idx[None, :] >= L[:, None]
        mask = pad[:, :, None] | pad[:, None, :]
    elif name in ("C4a", "C4b"):
        mask = rand(b, n, n) < 0.5
    elif name == "C5":
        u = rand(b, h, n, n)
        bias = torch.where(u < 0.025, torch.full_like(bias, 8.0), bias)
        bias = torch.where(u > 0.975, torch.full_like(bias, -8.0), bias)
        mask = rand(b, n, n) < 0.05
    else:
        mask = torch.zeros(b, n, n, dtype=torch.bool, device=gdev)
    do = randn(b, h, n, n, d)
    q, k, v, bias, do = (t.to(device=device, dtype=dtype) for t in (q, k, v, bias, do))
    mask = mask.to(device)
    if name in ("C4a", "C4b"):
        # ending-node variant: every input is an i<->j transposed, non-contiguous view
        q, k, v, do = (t.transpose(2, 3) for t in (q, k, v, do))
        bias = bias.transpose(-1, -2)
        mask = mask.transpose(-1, -2)
    return q, k, v, bias, mask, do


def flops(b, h, n, d):
    unit = b * h * n**3 * d
    return 4 * unit, 10 * unit  # forward, backward


def _event_ms(fn, reps):
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(reps):
        fn()
    end.record()
    end.synchronize()
    return start.elapsed_time(end) / reps


def _quantile(sorted_values, q):
    """Linear-interpolated quantile of an ascending list."""
    if not sorted_values:
        return None
    x = q * (len(sorted_values) - 1)
    lo = int(x)
    hi = min(lo + 1, len(sorted_values) - 1)
    return sorted_values[lo] + (sorted_values[hi] - sorted_values[lo]) * (x - lo)


def kernel_breakdown(q, k, v, bias, mask, do, reps):
    """Average launch duration (ms) of the four kernels, each timed with events on the
    stream it is launched on (torch's current stream), through the C ABI."""
    from trifast_amd import _lib, tuner
    from trifast_amd import torch as tt

    lib = _lib.load()
    b, h, n, _, d = q.shape
    code = tt._DTYPE_CODE[q.dtype]
    qv, kv, vv, dov = (tt._vector_ready(t) for t in (q, k, v, do))
    bv = bias
    mu8 = mask.view(torch.uint8)
    o, lse = tt._triangle_attention(q, k, v, bias, mask)
    dq, dk, dv = (torch.empty_like(o) for _ in range(3))
    db = torch.empty(bias.shape, dtype=bias.dtype, device=bias.device)
    ws = torch.empty(lib.trifast_bwd_workspace_bytes(b, h, n, d, code), dtype=torch.uint8, device=q.device)
    stream = torch.cuda.current_stream().cuda_stream
    S = lambda t: _lib.i64_array(tt._strides(t))
    out = {}

    def fwd(tile):
        rc = lib.trifast_fwd(o.data_ptr(), lse.data_ptr(), qv.data_ptr(), kv.data_ptr(), vv.data_ptr(), bv.data_ptr(), mu8.data_ptr(),
                             b, h, n, d, code, S(qv), S(kv), S(vv), S(bv), S(mu8), tile, ws.data_ptr(), ws.numel(), stream)
        _lib.check(rc, "trifast_fwd")

    def bwd_one(kernel, tile):
        rc = lib.trifast_bwd_one(kernel, dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), db.data_ptr(), dov.data_ptr(), qv.data_ptr(), kv.data_ptr(),
                                 vv.data_ptr(), bv.data_ptr(), mu8.data_ptr(), o.data_ptr(), lse.data_ptr(), b, h, n, d, code,
                                 S(dov), S(qv), S(kv), S(vv), S(bv), S(mu8), None, None, None, None, tile, ws.data_ptr(), ws.numel(), stream)
        _lib.check(rc, "trifast_bwd_one")

    # (the tiles the operator itself runs with: its cache is warm after the timed steps)
    for kernel in (_lib.KERNEL_FWD, _lib.KERNEL_BWD_Q, _lib.KERNEL_BWD_KV, _lib.KERNEL_BWD_B):
        launch = fwd if kernel == _lib.KERNEL_FWD else (lambda t, kern=kernel: bwd_one(kern, t))
        tile = tuner.pick(kernel, n, h, d, q.dtype, launch)
        for _ in range(20):  # (after a pause the clocks take some twenty milliseconds to come back up)
            launch(tile)
        torch.cuda.synchronize()
        out[_lib.KERNEL_NAMES[kernel]] = {"ms": _event_ms(lambda: launch(tile), reps), "tile": dict(_lib.tile_info(kernel, tile), id=tile)}
    # a dk/dv tile that also produces dq replaces the dq kernel: the step does not launch it
    fused = bool(lib.trifast_bwd_kv_tile_writes_dq(out["_bwd_kv"]["tile"]["id"]))
    out["_bwd_kv"]["writes_dq"] = fused
    out["_bwd_q"]["in_step"] = not fused
    # every timed launch includes the two pre-passes (mask bits, bias re-tiling), which the entry
    # points do not launch alone: their cost stays inside each figure (about 0.02 ms at n = 1024)
    return out


def other_workloads(names, warmup: int = 5, steps: int = 10):
    """fwd+bwd step and forward of the other configurations, in the same run as the headline
    one: ``warmup`` untimed steps, then ``steps`` timed ones between synchronisations, with the
    library's default tiles (nothing is tuned here, so the figures do not depend on a cache)."""
    import trifast_amd

    out = {}
    saved = os.environ.get("TRIFAST_AUTOTUNE")
    os.environ["TRIFAST_AUTOTUNE"] = "0"
    try:
        for name in names:
            dtype, b, n, h, d, _ = WORKLOADS[name]
            q, k, v, bias, mask, do = make_workload(name, "cuda:0")
            q.requires_grad_(True), k.requires_grad_(True), v.requires_grad_(True), bias.requires_grad_(True)

            def step():
                trifast_amd.triangle_attention(q, k, v, bias, mask).backward(do)
                q.grad = k.grad = v.grad = bias.grad = None

            def fwd_only():
                with torch.no_grad():
                    trifast_amd.triangle_attention(q, k, v, bias, mask)

            for _ in range(warmup):
                step()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(steps):
                step()
            torch.cuda.synchronize()
            ms = (time.perf_counter() - t0) * 1e3 / steps
            fwd_only()
            torch.cuda.synchronize()
            ms_fwd = _event_ms(fwd_only, steps)
            f_fwd, f_bwd = flops(b, h, n, d)
            peak = PEAK_F32_TFLOPS if dtype == torch.float32 else PEAK_BF16_TFLOPS
            out[name] = {"ms_per_step": round(ms, 4), "frac_of_peak": round((f_fwd + f_bwd) / ms / 1e9 / peak, 4),
                         "fwd_ms": round(ms_fwd, 4), "fwd_frac_of_peak": round(f_fwd / ms_fwd / 1e9 / peak, 4)}
            del q, k, v, bias, mask, do
            torch.cuda.empty_cache()
    finally:
        if saved is None:
            os.environ.pop("TRIFAST_AUTOTUNE", None)
        else:
            os.environ["TRIFAST_AUTOTUNE"] = saved
    return out


def _cpu_model() -> str:
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(name: str, tensors, budget_s: float = 20.0):
    """The oracle restatement on the host cores, on the first pair rows of the workload's own
    seeded tensors (rows are independent; the b*h*n^3 logits of the full job would not fit in
    host memory at once, so rows go through in chunks of 8).  Two legs, fp32 and the workload's
    dtype, each one warm-up plus the median of three repetitions, forward + autograd backward
    and forward alone.  Returns the JSON object for the bench line."""
    from oracle import triangle_oracle as orc

    dtype, b, n, h, d, _ = WORKLOADS[name]
    # the host share of a one-GPU box is 16 cores, whatever the machine reports
    cores = int(os.environ.get("OMP_NUM_THREADS", 0)) or min(os.cpu_count() or 1, 16)
    torch.set_num_threads(cores)
    q, k, v, bias, mask, do = tensors
    chunk = 8

    def host(rows, dt):
        qs, ks, vs, dos = (t[:, :, :rows].detach().to("cpu", dt).contiguous() for t in (q, k, v, do))
        return qs, ks, vs, bias.detach().to("cpu", dt).contiguous(), mask[:, :rows].cpu().contiguous(), dos

    def run(ten, backward):
        qs, ks, vs, bs, ms, dos = ten
        rows = qs.shape[2]
        t0 = time.perf_counter()
        for i0 in range(0, rows, chunk):
            sl = slice(i0, min(rows, i0 + chunk))
            if backward:
                qc, kc, vc = (t[:, :, sl].clone().requires_grad_(True) for t in (qs, ks, vs))
                bc = bs.clone().requires_grad_(True)
                orc.attention_reference(qc, kc, vc, bc, ms[:, sl]).backward(dos[:, :, sl])
            else:
                with torch.no_grad():
                    orc.attention_reference(qs[:, :, sl], ks[:, :, sl], vs[:, :, sl], bs, ms[:, sl])
        return time.perf_counter() - t0

    def leg(dt, budget):
        probe = host(min(n, chunk), dt)
        run(probe, True)  # warm-up of the probe
        t_probe = run(probe, True)
        # five timed-or-warm passes of fwd+bwd and of fwd (about a third of that) per leg
        rows = int(max(chunk, min(n, chunk * budget / (5.5 * max(t_probe, 1e-6))) // chunk * chunk))
        rows = min(rows, n)
        ten = host(rows, dt)
        out = {"rows": rows}
        for key, backward, fl in (("fwd_bwd", True, sum(flops(b, h, n, d))), ("fwd", False, flops(b, h, n, d)[0])):
            run(ten, backward)  # warm-up
            t = sorted(run(ten, backward) for _ in range(3))[1]
            out[key] = {"s": t, "tflops": fl * rows / n / t / 1e12, "full_job_s": t * n / rows}
        return out

    f32 = leg(torch.float32, budget_s * 0.6)
    res = {
        "value": f32["fwd_bwd"]["tflops"],
        "unit": "TFLOP/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"first {f32['rows']} of {n} pair rows of the workload's own seeded tensors in chunks of {chunk}, fp32, "
                  f"fwd + autograd bwd, 1 warm-up + median of 3: {f32['fwd_bwd']['s']:.2f} s "
                  f"(full job extrapolates to {f32['fwd_bwd']['full_job_s']:.1f} s)",
        "fwd_value": f32["fwd"]["tflops"],
        "fwd_full_job_s": f32["fwd"]["full_job_s"],
        "cpu_model": _cpu_model(),
        "os_cpu_count": os.cpu_count(),
    }
    if dtype != torch.float32:
        low = leg(dtype, budget_s * 0.4)
        res["workload_dtype"] = {
            "dtype": str(dtype).split(".")[-1], "rows": low["rows"],
            "value": low["fwd_bwd"]["tflops"], "fwd_value": low["fwd"]["tflops"],
            "full_job_s": low["fwd_bwd"]["full_job_s"],
        }
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="M", choices=[w for w in WORKLOADS if w != "C1"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-other-workloads", action="store_true",
                    help="skip the short fwd+bwd timings of the other configurations that the default run adds")
    ap.add_argument("--cpu-budget", type=float, default=20.0)
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also launch one plain 256 MiB device copy, the known-size kernel that "
                         "FETCH_SIZE / WRITE_SIZE counter readings are scaled by")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py needs a GPU: the operator has no CPU path", file=sys.stderr)
        sys.exit(2)

    import trifast_amd
    from trifast_amd import tuner

    dev = torch.device("cuda:0")
    dtype, b, n, h, d, desc = WORKLOADS[args.workload]
    q, k, v, bias, mask, do = make_workload(args.workload, dev)
    q.requires_grad_(True), k.requires_grad_(True), v.requires_grad_(True), bias.requires_grad_(True)

    def step():
        o = trifast_amd.triangle_attention(q, k, v, bias, mask)
        o.backward(do)
        q.grad = k.grad = v.grad = bias.grad = None

    def fwd_only():
        with torch.no_grad():
            trifast_amd.triangle_attention(q, k, v, bias, mask)

    if args.calibrate_copy:
        src = torch.zeros(256 << 20, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)  # reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del src, dst

    for _ in range(args.warmup):  # also warms the tile cache
        step()
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats()
    base_mem = torch.cuda.memory_allocated()
    # the K timed steps: wall clock around all of them (the headline), and an event pair
    # per step for the spread (median, 10th and 90th percentile)
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps + 1)]
    t0 = time.perf_counter()
    marks[0].record()
    for i in range(args.steps):
        step()
        marks[i + 1].record()
    torch.cuda.synchronize()
    ms_step = (time.perf_counter() - t0) * 1e3 / args.steps
    per_step = sorted(marks[i].elapsed_time(marks[i + 1]) for i in range(args.steps))
    peak_extra = torch.cuda.max_memory_allocated() - base_mem

    fwd_only()
    torch.cuda.synchronize()
    ms_fwd = _event_ms(fwd_only, args.steps)
    # matrix peak at the device's maximum shader clock: 4096 dense bf16/fp16 FLOP per clock and CU
    from trifast_amd import _lib

    clock_mhz = _lib.load().trifast_device_clock_mhz(dev.index or 0)
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    peak_at_clock = cus * 4096 * clock_mhz / 1e6 if clock_mhz > 0 else None

    dname = {torch.bfloat16: "bf16", torch.float16: "f16", torch.float32: "f32"}[dtype]
    f_fwd, f_bwd = flops(b, h, n, d)
    peak = PEAK_F32_TFLOPS if dtype == torch.float32 else PEAK_BF16_TFLOPS
    tf_step = (f_fwd + f_bwd) / ms_step / 1e9
    tf_fwd = f_fwd / ms_fwd / 1e9

    kern = kernel_breakdown(q.detach(), k.detach(), v.detach(), bias.detach(), mask, do, max(3, args.steps // 2))
    # GEMMs each kernel needs for its own outputs (S and dP are recomputed per kernel; the
    # row-resident dk/dv tile computes them once for dq, dk and dv)
    gemms = {"_fwd": 2, "_bwd_q": 3, "_bwd_kv": 5 if kern["_bwd_kv"]["writes_dq"] else 4, "_bwd_b": 2}
    for name, rec in kern.items():
        rec["tflops"] = gemms[name] * 2 * b * h * n**3 * d / rec["ms"] / 1e9
    in_step = [name for name in kern if kern[name].get("in_step", True)]
    bwd_ms = sum(kern[name]["ms"] for name in in_step if name != "_fwd")
    dom = max(in_step, key=lambda key: kern[key]["ms"])
    tile = kern[dom]["tile"]
    mib = MEASURED_TRAFFIC_MIB.get((args.workload, dom, tile["id"]))
    traffic = None if mib is None else mib * 2**20
    roofline = {
        "kernel": dom,
        "bound": "mfma",
        "achieved": kern[dom]["tflops"],
        "peak": peak,
        "unit": "TFLOP/s",
        "frac": kern[dom]["tflops"] / peak,
        "traffic": traffic,
        "launch_ms": kern[dom]["ms"],
        "flop_per_launch": gemms[dom] * 2 * b * h * n**3 * d,
    }

    line = {
        "metric": f"fwd+bwd TFLOP/s & % {dname} MFMA peak, {dname} h={h} d={d} n={n}, 1xMI355X",
        "value": tf_step,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": dname,
        "data": "synthetic",
        "config": {"workload": f"{args.workload}: {desc}", "b": b, "h": h, "n": n, "d": d},
        "frac_of_peak": tf_step / peak,
        "fwd_ms": ms_fwd,
        "fwd_tflops": tf_fwd,
        "fwd_frac_of_peak": tf_fwd / peak,
        "peak_extra_mem_mib": peak_extra / 2**20,
        "step_ms_quantiles": {"p10": _quantile(per_step, 0.1), "median": _quantile(per_step, 0.5), "p90": _quantile(per_step, 0.9)},
        "peak_tflops_nominal": peak,
        "max_clock_mhz": clock_mhz,
        "peak_tflops_at_max_clock": None if dtype == torch.float32 else peak_at_clock,
        "kernels": {name: {"ms": round(rec["ms"], 4), "tflops": round(rec["tflops"], 1), "tile": rec["tile"],
                           "in_step": rec.get("in_step", True)} for name, rec in kern.items()},
        # the backward as a whole, counted as the five GEMMs it needs (10 b h n^3 d) whatever the
        # kernels recompute, over the launch durations of its kernels
        "bwd_credited": {"ms": bwd_ms, "tflops": f_bwd / bwd_ms / 1e9, "frac_of_peak": f_bwd / bwd_ms / 1e9 / peak},
        "kernel_ms_include": "mask and bias pre-passes (and the db partial reduce where rows are split), about 0.01 ms at n=1024",
        "roofline": roofline,
        "autotune": tuner.autotune_enabled(),
    }
    if args.workload == "M" and not args.no_other_workloads:
        del q, k, v, bias, mask, do
        torch.cuda.empty_cache()
        line["workloads"] = other_workloads(["C2", "C3", "C4a", "C4b", "C5", "F32"])
        line["workloads_note"] = "fwd+bwd steps of the other configurations in this run: 5 warm-up + 10 timed steps each, library default tiles"
        q, k, v, bias, mask, do = make_workload(args.workload, dev)
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(args.workload, (q, k, v, bias, mask, do), args.cpu_budget)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
