"""Runtime and peak-memory sweeps over the sequence length, written in the layout the
reference keeps its own results in (``benchmark/<device>/runtime/*.csv``,
``benchmark/<device>/memory/memory.parquet``), so that MI355X results sit beside the
A100 / RTX 3090 files.

    python -m trifast_amd.sweep runtime [--out benchmark] [--n-max 2048] [--step 32]
    python -m trifast_amd.sweep memory  [--out benchmark] [--n-max 2048] [--step 32]
    python -m trifast_amd.sweep block   [--n 1024] [--c-in 128]

Same protocol as reference scripts/benchmark.py:13-105 and scripts/memory.py:25-131:
bf16, h=4, d=32, 50 % random mask, n = 32..2048 in steps of 32; "fwd" times the forward,
"bwd" times ``o.sum().backward()`` alone (retain_graph), median of the timed calls in
milliseconds; memory is ``torch.cuda.max_memory_allocated`` around one forward
(+ backward) in MiB.  Only the "Trifast" column is produced: the other columns of the
reference's tables are other implementations.

``block`` has no counterpart in the reference: it times the gated block of
``trifast_amd.nn`` (projections, operator, gate, output projection; forward + backward)
against the same block with the layout copies, the unfused gate and the linear layers a
caller would write in plain PyTorch around the operator, and the gate and weight-gradient
kernels alone against the HBM bytes they must move.
"""

from __future__ import annotations

import argparse
import statistics
from pathlib import Path

import torch

from .torch import triangle_attention
from .utils import gen_tensors

H, D = 4, 32
DTYPE = torch.bfloat16


def device_name() -> str:
    # reference src/trifast/autotune_helpers.py:19
    return torch.cuda.get_device_name().replace(" ", "-")


def _median_ms(fn, warmup: int = 5, rep_ms: float = 100.0, min_calls: int = 10, max_calls: int = 200) -> float:
    """Median duration of fn() in ms: `warmup` untimed calls, then calls timed one by one
    with events until `rep_ms` of GPU time or `max_calls` (mirrors triton's do_bench)."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    times, total = [], 0.0
    while len(times) < min_calls or (total < rep_ms and len(times) < max_calls):
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        fn()
        end.record()
        end.synchronize()
        times.append(start.elapsed_time(end))
        total += times[-1]
    return statistics.median(times)


def runtime(out: Path, ns: list[int]) -> None:
    out = out / device_name() / "runtime"
    out.mkdir(parents=True, exist_ok=True)
    rows = {"fwd": [], "bwd": []}
    for n in ns:
        q, k, v, bias, mask = gen_tensors(n, D, H, True, torch.device("cuda"), DTYPE)
        fwd = lambda: triangle_attention(q, k, v, bias, mask)
        ms_fwd = _median_ms(fwd)
        s = fwd().sum()
        ms_bwd = _median_ms(lambda: s.backward(retain_graph=True))
        q.grad = k.grad = v.grad = bias.grad = None
        rows["fwd"].append((n, ms_fwd))
        rows["bwd"].append((n, ms_bwd))
        print(f"n={n:5d} fwd {ms_fwd:8.4f} ms  bwd {ms_bwd:8.4f} ms", flush=True)
    for mode, data in rows.items():
        path = out / f"tri_attn_{mode}_{DTYPE}.csv"
        with open(path, "w") as f:
            f.write("n,Trifast\n")
            for n, ms in data:
                f.write(f"{float(n):.6f},{ms:.6f}\n")
        print(f"wrote {path}")


def memory(out: Path, ns: list[int], repeat: int = 3) -> None:
    import pandas as pd

    out = out / device_name() / "memory"
    out.mkdir(parents=True, exist_ok=True)
    rows = []
    for n in ns:
        for mode in ("fwd", "bwd"):
            for it in range(1 + repeat):  # the first pass warms the tile cache and is not recorded
                torch.cuda.synchronize()
                torch.cuda.reset_peak_memory_stats()
                q, k, v, bias, mask = gen_tensors(n, D, H, True, torch.device("cuda"), DTYPE)
                base = torch.cuda.max_memory_allocated() / 1024**2
                o = triangle_attention(q, k, v, bias, mask)
                torch.cuda.synchronize()
                if mode == "bwd":
                    o.sum().backward()
                    torch.cuda.synchronize()
                peak = torch.cuda.max_memory_allocated() / 1024**2
                if it > 0:
                    rows.append({"n": n, "base_memory": base, "peak_memory": peak, "model": "trifast", "mode": mode, "dtype": str(DTYPE)})
                del q, k, v, bias, mask, o
        print(f"n={n:5d} peak fwd {rows[-1 - repeat]['peak_memory']:10.1f} MiB  bwd {rows[-1]['peak_memory']:10.1f} MiB", flush=True)
    df = pd.DataFrame(rows)
    df.to_parquet(out / "memory.parquet")
    pivot = df.groupby(["n", "mode"])[["base_memory", "peak_memory"]].mean().reset_index()
    pivot.to_csv(out / "memory.csv", index=False, float_format="%.3f")
    print(f"wrote {out / 'memory.parquet'} and {out / 'memory.csv'}")


def block(n: int, c_in: int) -> None:
    from . import nn

    dev = torch.device("cuda")
    torch.manual_seed(0)
    fused = nn.TriangleAttention(c_in, H, D).to(dev, DTYPE)

    def unfused(x, mask):
        m = fused
        heads = lambda t: t.unflatten(-1, (H, D)).permute(0, 3, 1, 2, 4).contiguous()
        o = triangle_attention(heads(m.q(x)), heads(m.k(x)), heads(m.v(x)), m.b(x).permute(0, 3, 1, 2).contiguous(), mask)
        return m.out(o.permute(0, 2, 3, 1, 4).flatten(-2) * torch.sigmoid(m.g(x)))

    x = torch.randn(1, n, n, c_in, device=dev, dtype=DTYPE, requires_grad=True)
    mask = torch.rand(1, n, n, device=dev) < 0.5
    dy = torch.randn(1, n, n, c_in, device=dev, dtype=DTYPE)

    def step(fn):
        fn(x, mask).backward(dy)
        x.grad = None
        fused.zero_grad(set_to_none=True)

    ms_fused = _median_ms(lambda: step(fused))
    ms_unfused = _median_ms(lambda: step(unfused))
    print(f"block n={n} c_in={c_in} h={H} d={D} {DTYPE}: forward+backward {ms_fused:.3f} ms with views and the fused gate, "
          f"{ms_unfused:.3f} ms with layout copies and the gate in PyTorch ops ({ms_unfused / ms_fused:.2f}x)")
    o = torch.randn(1, H, n, n, D, device=dev, dtype=DTYPE)
    g = torch.randn(1, n, n, H * D, device=dev, dtype=DTYPE)
    gy = torch.randn_like(g)
    size = o.numel() * o.element_size()
    ms = _median_ms(lambda: nn.gated_output(o, g))
    print(f"gate forward  {ms * 1e3:8.1f} us  {3 * size / ms / 1e6:7.1f} GB/s of 3 tensors x {size / 2**20:.0f} MiB")
    oo, gg = o.clone().requires_grad_(True), g.clone().requires_grad_(True)
    y = nn.gated_output(oo, gg)
    ms = _median_ms(lambda: torch.autograd.grad(y, (oo, gg), gy, retain_graph=True))
    print(f"gate backward {ms * 1e3:8.1f} us  {5 * size / ms / 1e6:7.1f} GB/s of 5 tensors x {size / 2**20:.0f} MiB")
    ms = _median_ms(lambda: gy.copy_(g))
    print(f"(a plain device copy of one such tensor {ms * 1e3:8.1f} us  {2 * size / ms / 1e6:7.1f} GB/s read + written)")
    x2 = x.detach().reshape(-1, c_in)
    widths = (H * D, H * D, H * D, H, H * D)  # q, k, v, bias, gate
    dys = [torch.randn(x2.shape[0], w, device=dev, dtype=DTYPE) for w in widths]
    ws = [torch.randn(w, c_in, device=dev, dtype=DTYPE) for w in widths]
    nbytes = (sum(t.numel() for t in dys) + x2.numel()) * x2.element_size()
    ms = _median_ms(lambda: nn.linear_input_grad(dys, ws))

    def blas_dx():
        dx = dys[0] @ ws[0]
        for dy, w in zip(dys[1:], ws[1:]):
            dx = dx + dy @ w  # (what autograd does with the layers' separate input gradients)
        return dx

    nb_fwd = (sum(t.numel() for t in dys) + x2.numel()) * x2.element_size()
    ms_fwd = _median_ms(lambda: nn.linear_outputs(x2, ws, [None] * len(ws)))
    ms_fwd_blas = _median_ms(lambda: [torch.nn.functional.linear(x2, w) for w in ws])
    print(f"the five projections of x              {ms_fwd * 1e3:8.1f} us  {nb_fwd / ms_fwd / 1e6:7.1f} GB/s of x and the outputs ({nb_fwd / 2**20:.0f} MiB); "
          f"the BLAS library's five products {ms_fwd_blas * 1e3:8.1f} us")
    ms_blas = _median_ms(blas_dx)
    print(f"input gradient of the five projections {ms * 1e3:8.1f} us  {nbytes / ms / 1e6:7.1f} GB/s of the dy and dx ({nbytes / 2**20:.0f} MiB); "
          f"the BLAS library's five products and four additions {ms_blas * 1e3:8.1f} us")
    del dys, ws
    for n_out in (H * D, H):
        dy2 = torch.randn(x2.shape[0], n_out, device=dev, dtype=DTYPE)
        nbytes = (x2.numel() + dy2.numel()) * x2.element_size()
        ms = _median_ms(lambda: nn.linear_weight_grad(dy2, x2))
        ms_blas = _median_ms(lambda: dy2.t() @ x2)
        print(f"weight gradient [{n_out} x {c_in}] over {x2.shape[0]} rows {ms * 1e3:8.1f} us  {nbytes / ms / 1e6:7.1f} GB/s of x and dy "
              f"({nbytes / 2**20:.0f} MiB); the BLAS library's product {ms_blas * 1e3:8.1f} us")


def main() -> None:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("what", choices=["runtime", "memory", "block"])
    ap.add_argument("--out", default="benchmark")
    ap.add_argument("--n-max", type=int, default=2048)
    ap.add_argument("--step", type=int, default=32)
    ap.add_argument("--n", type=int, default=1024, help="block: sequence length")
    ap.add_argument("--c-in", type=int, default=128, help="block: channels of the pair representation")
    args = ap.parse_args()
    if not torch.cuda.is_available():
        raise SystemExit("the sweeps need a GPU: the operator has no CPU path")
    if args.what == "block":
        return block(args.n, args.c_in)
    ns = list(range(args.step, args.n_max + 1, args.step))
    (runtime if args.what == "runtime" else memory)(Path(args.out), ns)


if __name__ == "__main__":
    main()
