"""``trifast-tune``: time every compiled tile for a sweep of shapes and persist the
winners.  Same flags and defaults as reference src/trifast/tune.py:66-100
(``--min-n --max-n --dtype --h --d``); n runs over the powers of two between
min-n and max-n (reference :46)."""

from __future__ import annotations

import argparse
import os
from math import log2

import torch


def valid_dtypes(value: str) -> list[torch.dtype]:
    dtype_map = {"float32": torch.float32, "bfloat16": torch.bfloat16, "float16": torch.float16}
    allowed = set(dtype_map) | {"all"}
    dtypes = {x.strip().lower() for x in value.split(",")}
    invalid = dtypes - allowed
    if invalid:
        raise argparse.ArgumentTypeError(f"Invalid dtype(s): {invalid}. Allowed values are: {allowed}")
    if "all" in dtypes:
        return list(dtype_map.values())
    return [dtype_map[x] for x in dtypes]


def parse_int_list(value: str) -> list[int]:
    try:
        return [int(x.strip()) for x in value.split(",")]
    except ValueError:
        raise argparse.ArgumentTypeError('Invalid format. Please provide comma-separated integers (e.g., "256,512,1024")')


def sweep_ns(min_n: int, max_n: int) -> list[int]:
    return [2**i for i in range(int(log2(min_n)), int(log2(max_n)) + 1)]


def tune(min_n, max_n, heads, dims, dtypes):
    from trifast_amd.torch import triangle_attention
    from trifast_amd.utils import gen_tensors

    for d in dims:
        for h in heads:
            for n in sweep_ns(min_n, max_n):
                for dtype in dtypes:
                    print(f"Tuning: N: {n}, H: {h}, D: {d}, dtype: {dtype}")
                    q, k, v, bias, mask = gen_tensors(n, d, h, use_mask=True, device=torch.device("cuda"), dtype=dtype, std=1.0)
                    out = triangle_attention(q, k, v, bias, mask)
                    out.sum().backward()
    torch.cuda.synchronize()


def build_parser() -> argparse.ArgumentParser:
    parser = argparse.ArgumentParser(description="Autotune TriFast kernels over these parameters.")
    parser.add_argument("--min-n", type=int, help="Miniumum sequence length to tune.", default=16)
    parser.add_argument("--max-n", type=int, help="Maximum sequence length to tune.", default=1024)
    parser.add_argument(
        "--dtype",
        type=valid_dtypes,
        help="PyTorch datatypes to use (comma-separated). Options: float32, bfloat16, float16, all",
        default=[torch.bfloat16],
    )
    parser.add_argument("--h", type=parse_int_list, help='List of number of heads (comma-separated integers, e.g., "1,2,4")', default=[4])
    parser.add_argument("--d", type=parse_int_list, help='List of dims (comma-separated integers, e.g., "16,32,64")', default=[32])
    return parser


def main(argv=None):
    args = build_parser().parse_args(argv)
    # the reference sets these at import (src/trifast/tune.py:4-5) because its config
    # lists are built at import; the tuner here reads them at each pick
    os.environ["TRIFAST_FORCE_TUNE"] = "1"
    os.environ["TRIFAST_PRINT_AUTOTUNING"] = "1"
    tune(args.min_n, args.max_n, args.h, args.d, args.dtype)


if __name__ == "__main__":
    main()
